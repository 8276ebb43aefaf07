// bf16 MFMA prefill for gfx950 (K == V == D in {64,128,256}, M == 64 slots), fp32 accumulation.
//
// Everything is computed "transposed" so that each lane owns ONE query column of a 16x16
// accumulator block (v_mfma_f32_16x16x32_bf16: A[i][8*(l/16)+e], B[8*(l/16)+e][j], C[4*(l/16)+r][l%16]):
//   S^T[key][q]  = K  Q^T      A = K rows from LDS (16-byte reads), B = Q fragments kept in registers
//   O^T[d][q]   += V^T P^T     A = V^T via ds_read_b64_tr_b16 on the row-major V tile, B = P from the
//                              accumulator layout of S^T directly (contraction index permuted the same
//                              way on both operands), so P never moves between lanes
// Row statistics of the online softmax are per-lane scalars (+2 cross-lane steps over l/16).
// The slot branch is folded into the same machinery: slot logits are an "S tile" against the
// transposed chunk-start state hkT[m][d] and the slot read is a "PV tile" against hv[m][v]; the
// intra-chunk terms use the chunk algebra of nha_fla/ops/nha/chunk_fused.py:186-222, :242-275 with
// 16-row sub-blocks and sub-block-start decay references (:182-184, :203-204).
//
//   state pass  (mfma_state_kernel): per (sequence, kv-head, 16-slot block) sweep over 64-row chunks
//               with the fp32 state held in MFMA accumulators (chunk_fused.py:30-113).
//   output pass (mfma_out_kernel)  : per (chunk, kv-head, group of <=4 q-heads).
#include "mfma_common.h"

#include <mutex>
#include <stdlib.h>

namespace nha {
namespace {

using namespace mf;

// ------------------------------------------------------------------------------------------
// cooperative 64-row tile copy, global -> registers -> LDS (16-byte pieces, zero fill)
// ------------------------------------------------------------------------------------------
template <int ROWS, int D, int NTHR>
struct TileRegs {
  uint4 r[ROWS * D / 8 / NTHR];
};

// rows of the tile map to global rows grow0 + j; rows outside [vlo, vhi) are zero
template <int ROWS, int D, int NTHR>
__device__ __forceinline__ void tile_g2r(TileRegs<ROWS, D, NTHR>& t, const bf16_t* base, int64_t row_stride,
                                         int64_t grow0, int vlo, int vhi, int tid) {
#pragma unroll
  for (int u = 0; u < ROWS * D / 8 / NTHR; ++u) {
    const int c = tid + NTHR * u;
    const int row = c / (D / 8), col = (c % (D / 8)) * 8;
    uint4 x = make_uint4(0, 0, 0, 0);
    if (row >= vlo && row < vhi) x = *reinterpret_cast<const uint4*>(base + (grow0 + row) * row_stride + col);
    t.r[u] = x;
  }
}
template <int ROWS, int D, int NTHR>
__device__ __forceinline__ void tile_r2l(lbf16* lds, const TileRegs<ROWS, D, NTHR>& t, int tid) {
#pragma unroll
  for (int u = 0; u < ROWS * D / 8 / NTHR; ++u) {
    const int c = tid + NTHR * u;
    const int row = c / (D / 8), col = (c % (D / 8)) * 8;
    lds_st16(lds + row * (D + 16) + col, t.r[u]);
  }
}

// ==========================================================================================
// state pass, two levels
// ==========================================================================================
// The slot recurrence is sequential over the chunks of a sequence, so it is cut into segments of
// SEG chunks.  Level 1 (mfma_state_local_kernel, one workgroup per (segment, kv-head), one wave
// per 16-slot block) runs the recurrence of chunk_fused.py:30-113 from a ZERO state over its
// segment and stores, per chunk, the local chunk-start states, the gate cumsum table and the
// decay accumulated since the segment start; per segment, the local end state and total decay.
// Level 2 carries the true state across segments element-wise, h_seg[s+1] = h_seg[s] * dtot[s] + hend[s],
// in one of two forms.  The forward turns every chunk-start state into the true one, h_loc + h_seg * dcum,
// rounded to bf16 in place, so that the output pass reads plain operand tiles (state_final_kernel inside the
// scan, or state_scan_kernel followed by state_apply_kernel).  The backward (state_scan_kernel) keeps the
// segment-local states and writes the segment-start states h_seg beside them: it needs the sum in fp32.
// Both states are kept as C[d][m] accumulators (slot m = lane % 16).

// DW: columns of the state one workgroup carries (D, or D/2: twice the workgroups with half the
// tile, which this latency-bound kernel turns into bandwidth; the gates are then read once more).
template <int D, int DW>
__global__ __launch_bounds__(256) void mfma_state_local_kernel(const MP p) {
  constexpr int LDT = DW + 16;
  constexpr int NB = DW / 16;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* Xt = (lbf16*)smem;
  lbf16* St = Xt + BT * LDT;
  lbf16* Gt = St + BT * SLD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H;
  // One-dimensional grid, blockIdx.x = (state and column range z, kv-head h) + H Z k with k counting the segments of
  // the call one sequence after the other, without gaps: the workgroups that find k past the last segment (the grid
  // is sized for the most segments NT chunks in N sequences can have) are the last of the launch.  A workgroup
  // holds its CU slot for the whole chain of its segment and two fit a CU: were workgroups that leave at once
  // strewn over the launch order, the shader engines' shares of the working ones would differ, some CUs would
  // get a third one after their first two and others only one -- a second round for a tenth of the chip (49 us
  // against 32 us per launch at 512 segments x heads x states on 256 CUs).
  // z picks the state: even = k-state (rows of k_gsa; it also writes the gate tables), odd = v-state (rows of v).
  // The two recurrences share nothing but the gates, and twice the workgroups of half the size fill the chip better.
  constexpr int Z = 2 * (D / DW);
  const int hz = blockIdx.x % (H * Z), k = blockIdx.x / (H * Z);
  const int h = hz % H, z = hz / H;
  const bool isv = (z & 1) != 0;
  const int dcol0 = (z >> 1) * DW;             // first state column of this workgroup
  const bool lead = dcol0 == 0;                // writes what does not depend on the column range
  const bf16_t* xsrc = (isv ? p.v : p.k_gsa) + dcol0;
  bf16_t* hloc = isv ? p.hvc : p.hkT;
  float* hend = isv ? p.hend_v : p.hend_k;
  // segment k of the call -> (sequence n, segment kseg of it): a running count of ceil(chunks / SEG) over the
  // sequences, 256 at a time (one per thread, prefix over the workgroup)
  __shared__ int seg_wave[4], seg_hit[2];
  int n = 0, kseg = 0;
  {
    int base = 0;
    for (int n0 = 0; n0 < p.N; n0 += 256) {
      const int i = n0 + tid;
      const int segs = i < p.N ? (p.coff[i + 1] - p.coff[i] + SEG - 1) / SEG : 0;
      int incl = segs;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(incl, o, 64);
        if (lane >= o) incl += t;
      }
      if (lane == 63) seg_wave[wave] = incl;
      __syncthreads();
      int before = base;
      for (int w = 0; w < wave; ++w) before += seg_wave[w];
      const int first = before + incl - segs;
      if (k >= first && k < first + segs) {
        seg_hit[0] = i;
        seg_hit[1] = k - first;
      }
      base += seg_wave[0] + seg_wave[1] + seg_wave[2] + seg_wave[3];
      __syncthreads();
      if (k < base) break;
    }
    if (k >= base) return;   // past the last segment of the call
    n = seg_hit[0];
    kseg = seg_hit[1];
  }
  const int it0 = kseg * SEG;
  const int chunk0 = p.coff[n] + it0;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int L = eos - bos;
  const int nchunks = (L + BT - 1) / BT;
  const int nloc = (nchunks - it0) < SEG ? (nchunks - it0) : SEG;
  const int m = wave * 16 + l16;   // this lane's slot

  f32x4 hx[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) hx[b] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float gsum = 0.f;   // sum of the chunk-end gate cumsums since the segment start, this lane's slot

  TileRegs<BT, DW, 256> rx;
  uint4 rs[2], rg[2];
  auto issue = [&](int it) {
    const int rows = (L - it * BT) < BT ? (L - it * BT) : BT;
    const int64_t grow0 = (int64_t)bos + it * BT - p.shift;
    int vlo = p.shift - it * BT;
    vlo = vlo < 0 ? 0 : vlo;
    tile_g2r<BT, DW, 256>(rx, xsrc + (int64_t)h * D, (int64_t)H * D, grow0, vlo, rows, tid);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c8 = tid + 256 * u;
      const int j = c8 >> 3, m8 = (c8 & 7) * 8;
      uint4 xs = make_uint4(0, 0, 0, 0), xg = xs;
      if (j >= vlo && j < rows) {
        xs = *reinterpret_cast<const uint4*>(p.s + ((grow0 + j) * H + h) * MS + m8);
        xg = *reinterpret_cast<const uint4*>(p.g + ((grow0 + j) * H + h) * MS + m8);
      }
      rs[u] = xs;
      rg[u] = xg;
    }
  };

  issue(it0);
  for (int jc = 0; jc < nloc; ++jc) {
    const int it = it0 + jc;
    const int chunk = chunk0 + jc;
    const int rows = (L - it * BT) < BT ? (L - it * BT) : BT;
    if (jc > 0) __syncthreads();   // everyone is done reading the previous chunk's tiles
    tile_r2l<BT, DW, 256>(Xt, rx, tid);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c8 = tid + 256 * u;
      const int j = c8 >> 3, m8 = (c8 & 7) * 8;
      lds_st16(St + j * SLD + m8, rs[u]);
      lds_st16(Gt + j * SLD + m8, rg[u]);
    }
    if (jc + 1 < nloc) issue(it + 1);
    __syncthreads();
    // this lane's rows: element e = 4*q + r is row t = 16*q + 4*kb + r
    // (the sixteen gate and s values of a lane are a column of their tiles: four transposing reads each
    // instead of sixteen 2-byte reads)
    float gcv[16], sg[16];
    const bf16x8 gq01 = lds_frag_tr(Gt, SLD, 0, 16, 16 * wave, lane), gq23 = lds_frag_tr(Gt, SLD, 32, 48, 16 * wave, lane);
    const bf16x8 sq01 = lds_frag_tr(St, SLD, 0, 16, 16 * wave, lane), sq23 = lds_frag_tr(St, SLD, 32, 48, 16 * wave, lane);
    {
      float run[4], base = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float a = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          a += (float)(q < 2 ? gq01[4 * q + r] : gq23[4 * (q - 2) + r]);
          gcv[4 * q + r] = a;
        }
        run[q] = a;
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float off = base;
#pragma unroll
        for (int k2 = 0; k2 < 4; ++k2) {
          const float a = __shfl(run[q], l16 + 16 * k2, 64);
          base += a;
          if (k2 < kb) off += a;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) gcv[4 * q + r] += off;
      }
    }
    float glast;
    {
      const int tl = rows - 1;
      const int src_kb = (tl & 15) >> 2, e = 4 * (tl >> 4) + (tl & 3);
      float cand = 0.f;
#pragma unroll
      for (int x = 0; x < 16; ++x)
        if (x == e) cand = gcv[x];
      glast = __shfl(cand, l16 + 16 * src_kb, 64);
    }
    const int64_t cg = (int64_t)chunk * H + h;
    if (lead) {
      // the gate table: rows 0..31 from the k-state workgroup, rows 32..63 from the v-state one (both hold it)
      float* gout = p.gc + cg * BT * MS + m;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int ee = isv ? e + 8 : e;
        gout[(16 * (ee >> 2) + 4 * kb + (ee & 3)) * MS] = isv ? gcv[e + 8] : gcv[e];
      }
    }
    if (!isv && lead) {
      if (kb == 0) p.dcum[cg * MS + m] = fexp(gsum);
      // 16-row sub-blocks over which some slot decays by more than exp(DECAY_CLAMP): the output
      // pass cannot factor their intra-block decay; mfma_repair_kernel recomputes their rows
      int bits = 0;
      if (kb == 3) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float ref = q > 0 ? gcv[4 * q - 1] : 0.f;
          if (ref - gcv[4 * q + 3] > DECAY_CLAMP) bits |= 1 << q;
        }
      }
#pragma unroll
      for (int x = 32; x >= 1; x >>= 1) bits |= __shfl_xor(bits, x, 64);
      if (lane == 0) p.flags[cg * 4 + wave] = bits;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int t = 16 * (e >> 2) + 4 * kb + (e & 3);
      sg[e] = (t < rows) ? (float)(e < 8 ? sq01[e] : sq23[e - 8]) * fexp(glast - gcv[e]) : 0.f;
    }
    bf16x8 sg0, sg1;   // contraction steps over rows [0,32) and [32,64)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sg0[e] = (__bf16)sg[e];
      sg1[e] = (__bf16)sg[8 + e];
    }
    // local chunk-start states (bf16), before the update: rows m.  A lane holds 4 consecutive d of every 16-column
    // block; the lanes of an even 16-lane row keep block b, those of the odd row block b + 1, and the two trade their
    // halves, so that a lane stores 16 bytes and a row of the state 64 consecutive bytes per instruction
#pragma unroll
    for (int b = 0; b < NB; b += 2) {
      bf16x4 pa, pb;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pa[r] = (__bf16)hx[b][r];
        pb[r] = (__bf16)hx[b + 1][r];
      }
      uint2 ua = __builtin_bit_cast(uint2, pa), ub = __builtin_bit_cast(uint2, pb);
      const auto s0 = __builtin_amdgcn_permlane16_swap(ua.x, ub.x, false, false);
      const auto s1 = __builtin_amdgcn_permlane16_swap(ua.y, ub.y, false, false);
      const int dcol = 16 * (b + (kb & 1)) + 8 * (kb >> 1);
      *reinterpret_cast<uint4*>(hloc + (cg * MS + m) * D + dcol0 + dcol) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
    }
    const float dk = fexp(glast);
    gsum += glast;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int r = 0; r < 4; ++r) hx[b][r] *= dk;
      // h[d][m] += sum_t x[t][d] sg[t][m]     A = x^T (transposed LDS read), B = sg
      hx[b] = mfma16(lds_frag_tr(Xt, LDT, 0, 16, 16 * b, lane), sg0, hx[b]);
      hx[b] = mfma16(lds_frag_tr(Xt, LDT, 32, 48, 16 * b, lane), sg1, hx[b]);
    }
  }
  // segment end: local state (fp32, [m][d]) and total decay
  const int64_t sl = (int64_t)seg_slot(p.coff, n, it0) * H + h;
#pragma unroll
  for (int b = 0; b < NB; ++b)
    *reinterpret_cast<float4*>(hend + (sl * MS + m) * D + dcol0 + 16 * b + 4 * kb) = make_float4(hx[b][0], hx[b][1], hx[b][2], hx[b][3]);
  if (kb == 0 && !isv && lead) p.dtot[sl * MS + m] = fexp(gsum);
}

// Level 2, the scan: four consecutive d of one slot per thread, sequential over the segments of its sequence;
// writes the true segment-start states h_seg and the final states.  The loads do not depend on the chain, so the
// end states and decays of SCAN_AHEAD segments are requested together, one group ahead of the group that is
// being combined: a thread waits for memory once per group, not once per segment.
// grid (N*H, 2*MS*D/1024): the first MS*D/4 groups are the k-state ([m][d]), the rest the v-state.
constexpr int SCAN_AHEAD = 4;

template <int D>
__global__ __launch_bounds__(256) void state_scan_kernel(const MP p) {
  const int H = p.H;
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const int e4 = blockIdx.y * 256 + threadIdx.x;
  const bool isv = e4 >= MS * D / 4;
  const int em = (isv ? e4 - MS * D / 4 : e4) * 4;
  const int m = em / D, d = em % D;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int nchunks = (eos - bos + BT - 1) / BT;
  const int nseg = (nchunks + SEG - 1) / SEG;
  float4 hcur = make_float4(0.f, 0.f, 0.f, 0.f);
  if (p.h0k) {
    if (isv) {
      hcur = *reinterpret_cast<const float4*>(p.h0v + (((int64_t)n * H + h) * MS + m) * D + d);
    } else {
      const float* src = p.h0k + (((int64_t)n * H + h) * D + d) * MS + m;
      hcur = make_float4(src[0], src[MS], src[2 * MS], src[3 * MS]);
    }
  }
  const float* __restrict__ hend = isv ? p.hend_v : p.hend_k;
  float* __restrict__ hseg = isv ? p.hseg_v : p.hseg_k;
  const float* __restrict__ dtot = p.dtot;
  const int slot0 = p.coff[n] / SEG + n;
  struct Grp {
    float4 he[SCAN_AHEAD];
    float dt[SCAN_AHEAD];
  };
  auto request = [&](Grp& g, int sg0) {
#pragma unroll
    for (int i = 0; i < SCAN_AHEAD; ++i) {
      g.he[i] = make_float4(0.f, 0.f, 0.f, 0.f);
      g.dt[i] = 0.f;
      if (sg0 + i < nseg) {
        const int64_t sl = (int64_t)(slot0 + sg0 + i) * H + h;
        g.he[i] = *reinterpret_cast<const float4*>(hend + (sl * MS + m) * D + d);
        g.dt[i] = dtot[sl * MS + m];
      }
    }
  };
  Grp cur, nxt;
  request(cur, 0);
  for (int sg0 = 0; sg0 < nseg; sg0 += SCAN_AHEAD) {
    if (sg0 + SCAN_AHEAD < nseg) request(nxt, sg0 + SCAN_AHEAD);
#pragma unroll
    for (int i = 0; i < SCAN_AHEAD; ++i) {
      if (sg0 + i < nseg) {
        const int64_t sl = (int64_t)(slot0 + sg0 + i) * H + h;
        *reinterpret_cast<float4*>(hseg + (sl * MS + m) * D + d) = hcur;
        hcur.x = hcur.x * cur.dt[i] + cur.he[i].x;
        hcur.y = hcur.y * cur.dt[i] + cur.he[i].y;
        hcur.z = hcur.z * cur.dt[i] + cur.he[i].z;
        hcur.w = hcur.w * cur.dt[i] + cur.he[i].w;
      }
    }
    cur = nxt;
  }
  if (p.hkt) {
    if (isv) {
      *reinterpret_cast<float4*>(p.hvt + (((int64_t)n * H + h) * MS + m) * D + d) = hcur;
    } else {
      float* dst = p.hkt + (((int64_t)n * H + h) * D + d) * MS + m;
      dst[0] = hcur.x; dst[MS] = hcur.y; dst[2 * MS] = hcur.z; dst[3 * MS] = hcur.w;
    }
  }
}

// Level 2, forward form: every chunk-start state becomes the true one, h_loc + h_seg * dcum, rounded to bf16 in
// place, so that the output pass reads plain operand tiles.
//
// Where the carried part h_seg * dcum is below CARRY_FLOOR in absolute value for all four elements of a thread,
// the local state is left as it is -- neither read nor written: the sum would be the local state again to within
// 2^-100, fifty binary orders below anything bf16 tensors of representable magnitude can show.  Gates that forget
// quickly (log-gates of about -1 per token: e^-80 per chunk) leave only the first chunk of a segment to rewrite;
// with slow gates (the layers' logsigmoid / 8: e^-5 per chunk) every chunk is rewritten.
//
// Two forms.  state_final_kernel does it inside the scan (no h_seg round trip through memory; a thread's chain
// costs about a memory latency per segment): for sequences of a few segments.  state_apply_kernel runs after
// state_scan_kernel, one thread per (segment, slot, four d) with no chain: for long sequences.
constexpr float CARRY_FLOOR = 0x1p-100f;

// Four consecutive d of one slot per thread, sequential over the segments of its sequence; the small loads of
// segment sg + 2 (decays, end state) and the local states of segment sg + 1 that need rewriting are requested
// before segment sg is combined.
// grid (N*H, 2*MS*D/1024): the first MS*D/4 groups are the k-state ([m][d]), the rest the v-state.
template <int D>
__global__ __launch_bounds__(256) void state_final_kernel(const MP p) {
  const int H = p.H;
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const int e4 = blockIdx.y * 256 + threadIdx.x;
  const bool isv = e4 >= MS * D / 4;
  const int em = (isv ? e4 - MS * D / 4 : e4) * 4;
  const int m = em / D, d = em % D;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int nchunks = (eos - bos + BT - 1) / BT;
  const int nseg = (nchunks + SEG - 1) / SEG;
  float hcur[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.h0k) {
    if (isv) {
      const float4 x = *reinterpret_cast<const float4*>(p.h0v + (((int64_t)n * H + h) * MS + m) * D + d);
      hcur[0] = x.x; hcur[1] = x.y; hcur[2] = x.z; hcur[3] = x.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) hcur[i] = p.h0k[(((int64_t)n * H + h) * D + d + i) * MS + m];
    }
  }
  const float* hend = isv ? p.hend_v : p.hend_k;
  bf16_t* hloc = isv ? p.hvc : p.hkT;
  const int chunk0 = p.coff[n];
  const int slot0 = chunk0 / SEG + n;
  struct Small {      // what the chain itself needs of a segment
    float dc[SEG];
    float dt;
    float4 he;
  };
  struct Loc {        // local chunk-start states of a segment (those that are rewritten)
    uint2 v[SEG];
    unsigned need;
  };
  auto request_small = [&](Small& r, int sg) {
    const int64_t sl = (int64_t)(slot0 + sg) * H + h;
#pragma unroll
    for (int jc = 0; jc < SEG; ++jc) {
      r.dc[jc] = 0.f;
      if (sg * SEG + jc < nchunks) r.dc[jc] = p.dcum[((int64_t)(chunk0 + sg * SEG + jc) * H + h) * MS + m];
    }
    r.dt = p.dtot[sl * MS + m];
    r.he = *reinterpret_cast<const float4*>(hend + (sl * MS + m) * D + d);
  };
  // hs: the state that enters segment sg
  auto request_loc = [&](Loc& r, const Small& sm, int sg, const float (&hs)[4]) {
    const float amax = fmaxf(fmaxf(fabsf(hs[0]), fabsf(hs[1])), fmaxf(fabsf(hs[2]), fabsf(hs[3])));
    r.need = 0;
#pragma unroll
    for (int jc = 0; jc < SEG; ++jc) {
      r.v[jc] = make_uint2(0, 0);
      if (sg * SEG + jc < nchunks && amax * sm.dc[jc] >= CARRY_FLOOR) {
        r.need |= 1u << jc;
        r.v[jc] = *reinterpret_cast<const uint2*>(hloc + (((int64_t)(chunk0 + sg * SEG + jc) * H + h) * MS + m) * D + d);
      }
    }
  };
  Small s_cur, s_nxt, s_nn;
  Loc l_cur, l_nxt;
  request_small(s_cur, 0);
  if (nseg > 1) request_small(s_nxt, 1);
  request_loc(l_cur, s_cur, 0, hcur);
  for (int sg = 0; sg < nseg; ++sg) {
    float hn[4];
    hn[0] = hcur[0] * s_cur.dt + s_cur.he.x;
    hn[1] = hcur[1] * s_cur.dt + s_cur.he.y;
    hn[2] = hcur[2] * s_cur.dt + s_cur.he.z;
    hn[3] = hcur[3] * s_cur.dt + s_cur.he.w;
    if (sg + 2 < nseg) request_small(s_nn, sg + 2);
    if (sg + 1 < nseg) request_loc(l_nxt, s_nxt, sg + 1, hn);
#pragma unroll
    for (int jc = 0; jc < SEG; ++jc) {
      if (l_cur.need & (1u << jc)) {
        const int64_t cg = (int64_t)(chunk0 + sg * SEG + jc) * H + h;
        const uint32_t w[2] = {l_cur.v[jc].x, l_cur.v[jc].y};
        bf16x4 o4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float a0 = __uint_as_float((i & 1) ? (w[i >> 1] & 0xffff0000u) : (w[i >> 1] << 16));
          o4[i] = (__bf16)(a0 + hcur[i] * s_cur.dc[jc]);
        }
        *reinterpret_cast<bf16x4*>(hloc + (cg * MS + m) * D + d) = o4;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) hcur[i] = hn[i];
    s_cur = s_nxt;
    s_nxt = s_nn;
    l_cur = l_nxt;
  }
  if (p.hkt) {
    if (isv) {
      *reinterpret_cast<float4*>(p.hvt + (((int64_t)n * H + h) * MS + m) * D + d) = make_float4(hcur[0], hcur[1], hcur[2], hcur[3]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) p.hkt[(((int64_t)n * H + h) * D + d + i) * MS + m] = hcur[i];
    }
  }
}

// After state_scan_kernel: one thread per (segment, kv-head, slot, four consecutive d), every segment at once.
// grid (segment slots, H, 2*MS*D/1024): the first MS*D/4 groups of z are the k-state ([m][d]), the rest the v-state.
template <int D>
__global__ __launch_bounds__(256) void state_apply_kernel(const MP p) {
  const int H = p.H;
  const int slot = blockIdx.x, h = blockIdx.y;
  int n = 0;
  {
    int lo = 0, hi = p.N - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p.coff[mid] / SEG + mid <= slot) lo = mid; else hi = mid - 1;
    }
    n = lo;
  }
  const int it0 = (slot - (p.coff[n] / SEG + n)) * SEG;
  const int nchunks = p.coff[n + 1] - p.coff[n];
  if (it0 >= nchunks) return;
  const int nloc = (nchunks - it0) < SEG ? (nchunks - it0) : SEG;
  const int e4 = blockIdx.z * 256 + threadIdx.x;
  const bool isv = e4 >= MS * D / 4;
  const int em = (isv ? e4 - MS * D / 4 : e4) * 4;
  const int m = em / D, d = em % D;
  const int64_t sl = (int64_t)slot * H + h;
  const float4 hs = *reinterpret_cast<const float4*>((isv ? p.hseg_v : p.hseg_k) + (sl * MS + m) * D + d);
  const float amax = fmaxf(fmaxf(fabsf(hs.x), fabsf(hs.y)), fmaxf(fabsf(hs.z), fabsf(hs.w)));
  if (!(amax >= CARRY_FLOOR)) return;      // nothing is carried into this segment (its first, without initial state)
  bf16_t* hloc = isv ? p.hvc : p.hkT;
  const int64_t cg0 = (int64_t)(p.coff[n] + it0) * H + h;
  float dc[SEG];
#pragma unroll
  for (int jc = 0; jc < SEG; ++jc) dc[jc] = jc < nloc ? p.dcum[(cg0 + (int64_t)jc * H) * MS + m] : 0.f;
  uint2 loc[SEG];
  unsigned need = 0;
#pragma unroll
  for (int jc = 0; jc < SEG; ++jc) {
    loc[jc] = make_uint2(0, 0);
    if (amax * dc[jc] >= CARRY_FLOOR) {
      need |= 1u << jc;
      loc[jc] = *reinterpret_cast<const uint2*>(hloc + ((cg0 + (int64_t)jc * H) * MS + m) * D + d);
    }
  }
  const float hv4[4] = {hs.x, hs.y, hs.z, hs.w};
#pragma unroll
  for (int jc = 0; jc < SEG; ++jc) {
    if (need & (1u << jc)) {
      const uint32_t w[2] = {loc[jc].x, loc[jc].y};
      bf16x4 o4;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a0 = __uint_as_float((i & 1) ? (w[i >> 1] & 0xffff0000u) : (w[i >> 1] << 16));
        o4[i] = (__bf16)(a0 + hv4[i] * dc[jc]);
      }
      *reinterpret_cast<bf16x4*>(hloc + ((cg0 + (int64_t)jc * H) * MS + m) * D + d) = o4;
    }
  }
}

// ==========================================================================================
// output pass
// ==========================================================================================
// One workgroup = one 64-row chunk x G query heads of one kv-head; its NW waves split the
// 64 x G query rows into RQB blocks of 16 rows per wave.  Window K/V stream through four LDS
// buffers of TK keys (two K, two V, double buffered); TK = 64 for D <= 128, 32 for D = 256.
// The slot branch runs first on the same buffers: its four 64-row operand tiles (transposed
// chunk-start k-state, k_gsa rows, chunk-start v-state, v rows) fit at once when TK = 64 and
// in two stages when TK = 32.  The decay factors s_j[m] exp(gr[m] - gc_j[m]) that every wave
// needs are computed once per workgroup into LDS, already in MFMA fragment order.

template <int D, int TK>
struct OutSmem {
  static constexpr int LDT = D + 16;
  static constexpr size_t tile_bytes = (size_t)TK * LDT * 2;
  static constexpr size_t bytes =
      4 * tile_bytes + (size_t)BT * GLD * 4 + (size_t)BT * SLD * 2 + (size_t)(NSEA + NSEB) * 512 * 2;
};


template <int D, int G, int NW, int TK>
__global__ __launch_bounds__(64 * NW, 1) void mfma_out_kernel(const MP p) {
  constexpr int NTHR = 64 * NW;      // threads per workgroup
  constexpr int WPU = NW / G;        // waves per (chunk, head)
  constexpr int RQB = 4 / WPU;       // 16-row query blocks per wave
  static_assert(WPU >= 1 && WPU <= 4 && RQB * WPU == 4, "bad wave split");
  static_assert(TK == 64 || TK == 32, "bad tile size");
  constexpr int KS = D / 32;
  constexpr int DB = D / 16;
  constexpr int LDT = D + 16;
  constexpr int NH = TK / 32;        // 32-key halves per tile
  constexpr int TILE = TK * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const tiles = (lbf16*)smem;           // K0, K1, V0, V1
  lbf16* const Kb0 = tiles;
  lbf16* const Kb1 = tiles + TILE;
  lbf16* const Vb0 = tiles + 2 * TILE;
  lbf16* const Vb1 = tiles + 3 * TILE;
  lfloat* const gcR = (lfloat*)(tiles + 4 * TILE);   // gate cumsum [row j][slot m]
  lbf16* const sR = (lbf16*)(gcR + BT * GLD);        // s [row j][slot m]
  lbf16* const SEa = sR + BT * SLD;                  // NSEA fragments of 64 lanes x 8
  lbf16* const SEb = SEa + NSEA * 512;               // NSEB fragments
  // 64-row slot-branch tiles: TK = 64 -> four buffers; TK = 32 -> two double-height buffers
  lbf16* const tA = Kb0;                                 // hkT, then (TK = 32) hv
  lbf16* const tB = TK == 64 ? Kb1 : Vb0;                // k_gsa rows, then (TK = 32) v rows
  lbf16* const tC = TK == 64 ? Vb0 : Kb0;                // hv
  lbf16* const tD = TK == 64 ? Vb1 : Vb0;                // v rows

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  // grid = (kv-head x head-group, chunk), tiles dealt so that an XCD (workgroup id % 8) streams neighbouring
  // chunks of ONE kv-head and the window tiles its resident workgroups share stay in that XCD's L2 (xcd_tile;
  // with 8 (kv-head, group) pairs that is the launch order itself).  Chunks are taken from
  // the last to the first: the chunks at the start of a sequence have the shortest windows, and
  // short workgroups at the end of the launch leave the smallest tail.
  const int ngrp = NG / G;
  int vx, vy;
  xcd_tile(ngrp, p.NT, vx, vy);
  const int chunk = p.NT - 1 - vy;
  const int h = vx / ngrp, grp = vx % ngrp;
  const int hq = h * NG + grp * G + wave / WPU;
  const int qb0 = (wave % WPU) * RQB;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  const float cs = p.scale * LOG2E;   // logits are kept unscaled; p = exp2(cs * (s - m))
  const int64_t cg = (int64_t)chunk * H + h;

  // ---- window tile schedule: tile i covers keys [c0 + 64 - TK (i+1), c0 + 64 - TK i) ----------
  int lowest = bos;
  if (p.wl >= 0 && c0 - p.wl > bos) lowest = c0 - p.wl;
  const int ntiles = (c0 + 64 - lowest + TK - 1) / TK;
  TileRegs<TK, D, NTHR> rk, rv;
  // Tile boundaries are multiples of TK away from bos, so a window tile never starts before its
  // sequence; only the tiles over the chunk's own rows can run past eos.  Every tile that ends at
  // or before eos is loaded unconditionally from a wave-uniform base plus per-thread 32-bit
  // offsets that never change (one scalar subtraction per tile instead of per-load 64-bit
  // address arithmetic); the others take the row-checked path.
  constexpr int NPC = TK * D / 8 / NTHR;   // 16-byte pieces per thread and tile
  uint32_t goff[NPC], loff[NPC];
#pragma unroll
  for (int u = 0; u < NPC; ++u) {
    const int c = tid + NTHR * u;
    const int row = c / (D / 8), col = (c % (D / 8)) * 8;
    goff[u] = (uint32_t)row * (uint32_t)(H * D) + col;
    loff[u] = row * (D + 16) + col;
  }
  auto issue_window_fast = [&](int i) {
    const int64_t grow0 = (int64_t)c0 + 64 - TK * (i + 1);
    const bf16_t* kb_ = p.k_swa + (grow0 * H + h) * D;
    const bf16_t* vb_ = p.v + (grow0 * H + h) * D;
#pragma unroll
    for (int u = 0; u < NPC; ++u) {
      rk.r[u] = *reinterpret_cast<const uint4*>(kb_ + goff[u]);
      rv.r[u] = *reinterpret_cast<const uint4*>(vb_ + goff[u]);
    }
  };
  // tiles 0 and 1 (issued before the loop) may cover rows of the chunk itself, i.e. run past eos
  auto issue_window = [&](int i) {
    const int64_t grow0 = (int64_t)c0 + 64 - TK * (i + 1);
    if (grow0 + TK > eos) {
      int vhi = eos - (int)grow0;
      vhi = vhi < 0 ? 0 : (vhi > TK ? TK : vhi);
      tile_g2r<TK, D, NTHR>(rk, p.k_swa + (int64_t)h * D, (int64_t)H * D, grow0, 0, vhi, tid);
      tile_g2r<TK, D, NTHR>(rv, p.v + (int64_t)h * D, (int64_t)H * D, grow0, 0, vhi, tid);
    } else {
      issue_window_fast(i);
    }
  };
  auto stage_window = [&](lbf16* kdst, lbf16* vdst) {
#pragma unroll
    for (int u = 0; u < NPC; ++u) {
      lds_st16(kdst + loff[u], rk.r[u]);
      lds_st16(vdst + loff[u], rv.r[u]);
    }
  };
  // ---- phase 0: slot-branch operands -> LDS --------------------------------------------------
  int vlo = p.shift - it * BT;
  vlo = vlo < 0 ? 0 : vlo;
  const int64_t grow_s = (int64_t)c0 - p.shift;
  // Every global load of this phase is issued before the first result is used, so the phase costs
  // one memory latency, not one per tile.
  // chunk-start states are plain [m][d] bf16 tiles (the state pass leaves the true states)
  auto issue_state = [&](TileRegs<BT, D, NTHR>& r, const bf16_t* hst) {
    tile_g2r<BT, D, NTHR>(r, hst + cg * MS * D, (int64_t)D, 0, 0, BT, tid);
  };
  auto load_state_tile = [&](lbf16* dst, const bf16_t* hst) {
    TileRegs<BT, D, NTHR> r;
    issue_state(r, hst);
    tile_r2l<BT, D, NTHR>(dst, r, tid);
  };
  auto load_rows_tile = [&](lbf16* dst, const bf16_t* src) {
    TileRegs<BT, D, NTHR> t;
    tile_g2r<BT, D, NTHR>(t, src + (int64_t)h * D, (int64_t)H * D, grow_s, vlo, rows, tid);
    tile_r2l<BT, D, NTHR>(dst, t, tid);
  };
  {
    TileRegs<BT, D, NTHR> ra, rc, tb, td;
    constexpr int NG4 = 1024 / NTHR, NS8 = (512 + NTHR - 1) / NTHR;
    float4 gx[NG4];
    uint4 sx[NS8];
    issue_state(ra, p.hkT);
    tile_g2r<BT, D, NTHR>(tb, p.k_gsa + (int64_t)h * D, (int64_t)H * D, grow_s, vlo, rows, tid);
    if (TK == 64) {
      issue_state(rc, p.hvc);
      tile_g2r<BT, D, NTHR>(td, p.v + (int64_t)h * D, (int64_t)H * D, grow_s, vlo, rows, tid);
    }
    // gate cumsum table (fp32 [64][64]); rows past the sequence end are zero
    const float* gsrc = p.gc + cg * BT * MS;
#pragma unroll
    for (int u = 0; u < NG4; ++u) {
      const int c4 = tid + NTHR * u;
      const int j = c4 >> 4, m4 = (c4 & 15) * 4;
      gx[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (j < rows) gx[u] = *reinterpret_cast<const float4*>(gsrc + j * MS + m4);
    }
    // s rows of the slot branch (shifted)
#pragma unroll
    for (int u = 0; u < NS8; ++u) {
      const int c8 = tid + NTHR * u;
      const int j = c8 >> 3, m8 = (c8 & 7) * 8;
      sx[u] = make_uint4(0, 0, 0, 0);
      if (c8 < 512 && j >= vlo && j < rows) sx[u] = *reinterpret_cast<const uint4*>(p.s + ((grow_s + j) * H + h) * MS + m8);
    }
    issue_window(0);
    __builtin_amdgcn_sched_barrier(0);
    tile_r2l<BT, D, NTHR>(tA, ra, tid);
    tile_r2l<BT, D, NTHR>(tB, tb, tid);
    if (TK == 64) {
      tile_r2l<BT, D, NTHR>(tC, rc, tid);
      tile_r2l<BT, D, NTHR>(tD, td, tid);
    }
#pragma unroll
    for (int u = 0; u < NG4; ++u) {
      const int c4 = tid + NTHR * u;
      const int j = c4 >> 4, m4 = (c4 & 15) * 4;
      *reinterpret_cast<NHA_LDS f32x4*>(gcR + j * GLD + m4) = (f32x4){gx[u].x, gx[u].y, gx[u].z, gx[u].w};
    }
#pragma unroll
    for (int u = 0; u < NS8; ++u) {
      const int c8 = tid + NTHR * u;
      const int j = c8 >> 3, m8 = (c8 & 7) * 8;
      if (c8 < 512) lds_st16(sR + j * SLD + m8, sx[u]);
    }
  }
  __syncthreads();
  // decay-factor fragments, one (fragment, lane) item = 8 values.  Sub-block Q (16 query rows)
  // references the gate cumsum gr of the row before it: exponent gr[m] - gc_j[m] <= 0 for rows
  // j of earlier sub-blocks, and bounded by the sub-block's own decay for its diagonal rows.
  // All LDS reads of an item are issued before the first exponential waits for one: read one at a
  // time, the 8 values of an item cost 24 LDS latencies in sequence.
  for (int item = tid; item < (NSEA + NSEB) * 64; item += NTHR) {
    const int f = item >> 6, ln = item & 63;
    const int fl16 = ln & 15, fkb = ln >> 4;
    bf16x8 out;
    if (f < NSEA) {
      const int Q = f < 4 ? 0 : f < 8 ? 1 : f < 16 ? 2 : 3;
      const int rem = f - sea_base(Q);
      const int pr = rem >> 2, mb = rem & 3;
      const int m = 16 * mb + fl16;
      const float gr = Q > 0 ? gcR[(16 * Q - 1) * GLD + m] : 0.f;
      float gv[8];
      bf16_t sv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = 16 * (2 * pr + (e >> 2)) + 4 * fkb + (e & 3);   // j < 64 for every fragment
        gv[e] = gcR[j * GLD + m];
        sv[e] = sR[j * SLD + m];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int jb = 2 * pr + (e >> 2);
        const float val = bf16_to_f32(sv[e]) * fexp(fminf(gr - gv[e], DECAY_CLAMP));
        out[e] = (__bf16)(jb <= Q ? val : 0.f);
      }
      *reinterpret_cast<NHA_LDS bf16x8*>(SEa + f * 512 + ln * 8) = out;
    } else {
      const int g2 = f - NSEA;
      const int Q = g2 < 2 ? 0 : g2 < 6 ? 1 : g2 < 12 ? 2 : 3;
      const int rem = g2 - seb_base(Q);
      const int jb = rem >> 1, pr = rem & 1;
      const int j = 16 * jb + fl16;
      f32x4 gv[2], gr[2];
      bf16x4 sv[2];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int m0 = 32 * pr + 16 * hh + 4 * fkb;   // the lane's 4 consecutive slots of this half
        gv[hh] = *reinterpret_cast<const NHA_LDS f32x4*>(gcR + j * GLD + m0);
        gr[hh] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (Q > 0) gr[hh] = *reinterpret_cast<const NHA_LDS f32x4*>(gcR + (16 * Q - 1) * GLD + m0);
        sv[hh] = *reinterpret_cast<const NHA_LDS bf16x4*>(sR + j * SLD + m0);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        out[e] = (__bf16)((float)sv[e >> 2][e & 3] * fexp(fminf(gr[e >> 2][e & 3] - gv[e >> 2][e & 3], DECAY_CLAMP)));
      *reinterpret_cast<NHA_LDS bf16x8*>(SEb + g2 * 512 + ln * 8) = out;
    }
  }
  __syncthreads();

  // per-lane softmax state for the RQB queries (l16 + 16*(qb0+qb)) this lane serves
  float mrun[RQB], lg[RQB];
  f32x4 O[DB][RQB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) O[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  bf16x8 bp[RQB][2], bpr[RQB][2];   // slot probabilities x exp(gc_i) and x exp(gc_i - gr), B operands

  // window-query fragments: requested here so that they land during the slot branch
  bf16x8 qs[RQB][KS];
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    const bf16_t* qp = p.q_swa + ((int64_t)(c0 + irow) * HQ + hq) * D + 8 * kb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 x = make_uint4(0, 0, 0, 0);
      if (irow < rows) x = *reinterpret_cast<const uint4*>(qp + 32 * ks);
      qs[qb][ks] = as_bf16x8(x);
    }
  }
  // ---- phase 1a: slot logits and the slot "tile" of the softmax, one 16-row block at a time ----
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int Q = qb0 + qb;                // sub-block index inside the chunk
    const int irow = 16 * Q + l16;         // this lane's query row inside the chunk
    bf16x8 qf[KS];
    {
      const bf16_t* qp = p.q_gsa + ((int64_t)(c0 + irow) * HQ + hq) * D + 8 * kb;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        uint4 x = make_uint4(0, 0, 0, 0);
        if (irow < rows) x = *reinterpret_cast<const uint4*>(qp + 32 * ks);
        qf[ks] = as_bf16x8(x);
      }
    }
    // inter-chunk slot logits: okT[m][i] = sum_d hkT[m][d] q[i][d]
    f32x4 ok[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) ok[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) ok[mb] = mfma16(lds_frag(tA, LDT, 16 * mb + l16, 32 * ks + 8 * kb), qf[ks], ok[mb]);
    // intra-chunk scores AT[j][i] = sum_d k_gsa[j][d] q[i][d] for row blocks jb <= Q, masked j <= i
    bf16x8 bA[2];
    {
      f32x4 at[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) at[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int jb = 0; jb < 4; ++jb)
          if (jb <= Q) at[jb] = mfma16(lds_frag(tB, LDT, 16 * jb + l16, 32 * ks + 8 * kb), qf[ks], at[jb]);
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
        if (jb == Q) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (4 * kb + r > l16) at[jb][r] = 0.f;
        }
      bA[0] = pack8(at[0], at[1]);
      bA[1] = pack8(at[2], at[3]);
    }
    // okT_intra[m][i] = sum_j s_j[m] exp(gr[m] - gc_j[m]) AT[j][i]
    f32x4 oki[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      oki[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int pr = 0; pr < 2; ++pr)
        if (2 * pr <= Q) {
          const bf16x8 se = *reinterpret_cast<const NHA_LDS bf16x8*>(SEa + (sea_base(Q) + 4 * pr + mb) * 512 + lane * 8);
          oki[mb] = mfma16(se, bA[pr], oki[mb]);
        }
    }
    // combine, then the slot "tile" of the online softmax (logits unscaled, exponent scale cs)
    const int rref = 16 * Q - 1;
    float rmax = -INFINITY;
    f32x4 egi[4], egr[4];   // exp(gc_i[m]) and exp(gc_i[m] - gr[m]) in accumulator layout
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      const float4 gi = lds_ld_f4(gcR + irow * GLD + 16 * mb + 4 * kb);
      float4 gr4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (Q > 0) gr4 = lds_ld_f4(gcR + rref * GLD + 16 * mb + 4 * kb);
      const float giv[4] = {gi.x, gi.y, gi.z, gi.w};
      const float grv[4] = {gr4.x, gr4.y, gr4.z, gr4.w};
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        egi[mb][r] = fexp(giv[r]);
        egr[mb][r] = fexp(giv[r] - grv[r]);
        ok[mb][r] = ok[mb][r] * egi[mb][r] + oki[mb][r] * egr[mb][r];
        rmax = fmaxf(rmax, ok[mb][r]);
      }
    }
    rmax = max_over_rows(rmax);
    mrun[qb] = rmax;
    float psum = 0.f;
    const float mc = rmax * cs;
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        ok[mb][r] = fexp2(ok[mb][r] * cs - mc);   // unnormalised slot probabilities
        psum += ok[mb][r];
      }
    lg[qb] = psum;   // partial over this lane's 16 slots
    if (p.lse_gsa) {
      float tot = psum + __shfl_xor(psum, 16, 64);
      tot += __shfl_xor(tot, 32, 64);
      if (kb == 0 && irow < rows) p.lse_gsa[(int64_t)(c0 + irow) * HQ + hq] = (mc + __builtin_amdgcn_logf(tot)) * LN2;
    }
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      f32x4 x0, x1, y0, y1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        x0[r] = ok[2 * pr][r] * egi[2 * pr][r];
        x1[r] = ok[2 * pr + 1][r] * egi[2 * pr + 1][r];
        y0[r] = ok[2 * pr][r] * egr[2 * pr][r];
        y1[r] = ok[2 * pr + 1][r] * egr[2 * pr + 1][r];
      }
      bp[qb][pr] = pack8(x0, x1);
      bpr[qb][pr] = pack8(y0, y1);
    }
  }
  if (TK == 32) {
    // second stage of the slot-branch tiles: the state / row tiles of the value side
    __syncthreads();
    load_state_tile(tC, p.hvc);
    load_rows_tile(tD, p.v);
    __syncthreads();
  }
  // ---- phase 1b: slot read ----------------------------------------------------------------------
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int Q = qb0 + qb;
    // inter-chunk part: O^T[d][i] += sum_m hv[m][d] (p[i][m] exp(gc_i[m]))
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
      for (int db = 0; db < DB; ++db)
        O[db][qb] = mfma16(lds_frag_tr(tC, LDT, 32 * pr, 32 * pr + 16, 16 * db, lane), bp[qb][pr], O[db][qb]);
    // intra-chunk part: AvT[j][i] = sum_m s_j[m] exp(gr[m]-gc_j[m]) (p[i][m] exp(gc_i[m]-gr[m])), j <= i
    bf16x8 bAv[2];
    {
      f32x4 av[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        av[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (jb <= Q) {
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            const bf16x8 se = *reinterpret_cast<const NHA_LDS bf16x8*>(SEb + (seb_base(Q) + 2 * jb + pr) * 512 + lane * 8);
            av[jb] = mfma16(se, bpr[qb][pr], av[jb]);
          }
          if (jb == Q) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (4 * kb + r > l16) av[jb][r] = 0.f;
          }
        }
      }
      bAv[0] = pack8(av[0], av[1]);
      bAv[1] = pack8(av[2], av[3]);
    }
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
      if (2 * pr <= Q) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
          O[db][qb] = mfma16(lds_frag_tr(tD, LDT, 32 * pr, 32 * pr + 16, 16 * db, lane), bAv[pr], O[db][qb]);
      }
  }
  // ---- phase 2: sliding window, streamed in TK-key tiles --------------------------------------
  lds_barrier();   // every wave is done with the slot-branch tiles
  stage_window(Kb0, Vb0);
  if (ntiles > 1) issue_window(1);
  lds_barrier();

  // lazy rescaling: the running reference max only moves when a half tile exceeds it by more than
  // 2^RESCALE_LOG2 in probability units, so O is rescaled a handful of times per chunk
  constexpr float RESCALE_LOG2 = 8.f;
  const float thr = RESCALE_LOG2 / cs;
  f32x4 Lw[RQB];
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) Lw[qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (__bf16)1.0f;
  // every load issued before the prefetch of tile 1 (queries, tile 0) has landed here, so inside
  // the loop only the tile prefetch of the previous iteration is ever outstanding
  __builtin_amdgcn_s_waitcnt(0x0f70 | (2 * NPC));   // vmcnt(2 * NPC), other counters untouched
  for (int i = 0; i < ntiles; ++i) {
    const int cur = i & 1;
    const lbf16* Kt = cur ? Kb1 : Kb0;
    const lbf16* Vt = cur ? Vb1 : Vb0;
    const int xbase = 64 - TK * (i + 1);   // key offset of the tile's first key relative to the chunk start
    const bool edge = (xbase + TK - 1 > 0) || (p.wl >= 0 && p.wl < TK * (i + 1) - 1);
#pragma unroll
    for (int hf = 0; hf < NH; ++hf) {
      // S^T[key][q] for the 32 keys of this half: 2 key blocks x RQB query blocks, the
      // 2 * RQB accumulators advance together so consecutive MFMAs are independent
      f32x4 S[2][RQB];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) S[kk][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 a0 = lds_frag(Kt, LDT, 32 * hf + l16, 32 * ks + 8 * kb);
        const bf16x8 a1 = lds_frag(Kt, LDT, 32 * hf + 16 + l16, 32 * ks + 8 * kb);
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) {
          S[0][qb] = mfma16(a0, qs[qb][ks], S[0][qb]);
          S[1][qb] = mfma16(a1, qs[qb][ks], S[1][qb]);
        }
      }
      if (edge) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int qb = 0; qb < RQB; ++qb) {
            const int y = 16 * (qb0 + qb) + l16;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int x = xbase + 32 * hf + 16 * kk + 4 * kb + r;
              const bool ok = (x <= y) && (p.wl < 0 || x >= y - p.wl);
              if (!ok) S[kk][qb][r] = -INFINITY;
            }
          }
      }
      // online softmax per query column
      bf16x8 P[RQB];
      bool need = false;
      float rmax[RQB];
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) {
        float x = fmaxf(fmaxf(S[0][qb][0], S[0][qb][1]), fmaxf(S[0][qb][2], S[0][qb][3]));
        x = fmaxf(x, fmaxf(fmaxf(S[1][qb][0], S[1][qb][1]), fmaxf(S[1][qb][2], S[1][qb][3])));
        // the lane's own 8 keys suffice to decide (some lane exceeds the threshold iff the column
        // maximum does); the cross-lane maximum is only formed on the rare rescale path
        rmax[qb] = x;
        need |= x > mrun[qb] + thr;
      }
      if (__any(need)) {
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) {
          const float mnew = fmaxf(mrun[qb], max_over_rows(rmax[qb]));
          const float alpha = fexp2((mrun[qb] - mnew) * cs);
          mrun[qb] = mnew;
          lg[qb] *= alpha;
#pragma unroll
          for (int r = 0; r < 4; ++r) Lw[qb][r] *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) O[db][qb][r] *= alpha;
        }
      }
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) {
        const float mc = mrun[qb] * cs;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int r = 0; r < 4; ++r) S[kk][qb][r] = fexp2(S[kk][qb][r] * cs - mc);
        P[qb] = pack8(S[0][qb], S[1][qb]);
        // window row sums on the matrix core: every row of ones^T P is the sum over the 32 keys
        Lw[qb] = mfma16(ones, P[qb], Lw[qb]);
      }
      // O^T[d][q] += V^T P^T over the 32 keys of this half
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x8 a = lds_frag_tr(Vt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane);
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) O[db][qb] = mfma16(a, P[qb], O[db][qb]);
      }
    }
    if (i + 1 < ntiles) {
      stage_window(cur ? Kb0 : Kb1, cur ? Vb0 : Vb1);
      if (i + 2 < ntiles) issue_window_fast(i + 2);   // tiles >= 2 lie wholly before the chunk
    }
    lds_barrier();
  }

  // ---- epilogue -------------------------------------------------------------------------------
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    const float lwt = Lw[qb][0];
    float lgt = lg[qb] + __shfl_xor(lg[qb], 16, 64);
    lgt += __shfl_xor(lgt, 32, 64);
    const float inv = 1.f / (lwt + lgt);
    if (irow < rows) {
      bf16_t* op = p.o + ((int64_t)(c0 + irow) * HQ + hq) * D + 4 * kb;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        bf16x4 pk;
#pragma unroll
        for (int r = 0; r < 4; ++r) pk[r] = (__bf16)(O[db][qb][r] * inv);
        *reinterpret_cast<bf16x4*>(op + 16 * db) = pk;
      }
      if (p.lse_swa && kb == 0)
        p.lse_swa[(int64_t)(c0 + irow) * HQ + hq] = (mrun[qb] * cs + __builtin_amdgcn_logf(lwt)) * LN2;
    }
  }
}

// ==========================================================================================
// exact recomputation of rows the output pass cannot factor
// ==========================================================================================
// The output pass writes the intra-chunk decay exp(gc_i - gc_j) as exp(gc_i - gr) * exp(gr - gc_j)
// with gr the gate cumsum at the start of j's 16-row sub-block, and caps the second exponent at
// DECAY_CLAMP.  Where a slot forgets faster than that (flags from the state pass), the rows of
// that sub-block are recomputed here token by token with the unfactored decay (<= 1), in fp32
// VALU arithmetic, from the same chunk-start states and gate table: slot logits
// (nha_fla/ops/nha/chunk_fused.py:186-222), window logits, one softmax (:233-240), both reads
// (:242-283) and the branch LSEs (nha_fla/ops/nha/chunk.py:459-470).  grid (chunk, kv-head), the
// q-heads of the group in turn; workgroups of unflagged chunks leave at once.
template <int D>
struct RepairSmem {
  static constexpr int LDH = D + 1;
  static constexpr size_t floats = (size_t)MS * LDH + (size_t)MS * D + (size_t)BT * MS + 2 * D + 2 * MS + 2 * BT + 256 + 4 + BT;
};

template <int D>
__global__ __launch_bounds__(256) void mfma_repair_kernel(const MP p) {
  constexpr int LDH = RepairSmem<D>::LDH;
  const int chunk = blockIdx.x, h = blockIdx.y;
  const int H = p.H, HQ = p.HQ;
  const int64_t cg = (int64_t)chunk * H + h;
  const int* fl = p.flags + cg * 4;
  const int bits = fl[0] | fl[1] | fl[2] | fl[3];
  if (bits == 0) return;
  extern __shared__ __align__(16) float rsm[];
  float* hk = rsm;                // [MS][LDH] true chunk-start k-state, transposed
  float* hv = hk + MS * LDH;      // [MS][D]   true chunk-start v-state
  float* gcl = hv + MS * D;       // [BT][MS]  gate cumsum
  float* qg = gcl + BT * MS;      // [D] scaled slot-branch query
  float* qs = qg + D;             // [D] scaled window query
  float* okl = qs + D;            // [MS] slot logits -> probabilities
  float* gct = okl + MS;          // [MS] gate cumsum of the row
  float* Aj = gct + MS;           // [BT]
  float* Avj = Aj + BT;           // [BT]
  float* pw = Avj + BT;           // [256]
  float* red = pw + 256;          // [4]
  int* src = (int*)(red + 4);     // [BT]
  const int tid = threadIdx.x;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  for (int e = tid; e < MS * D; e += 256) {
    const int m = e / D, d = e % D;
    hk[m * LDH + d] = bf16_to_f32(p.hkT[(cg * MS + m) * D + d]);
    hv[m * D + d] = bf16_to_f32(p.hvc[(cg * MS + m) * D + d]);
  }
  for (int e = tid; e < BT * MS; e += 256) gcl[e] = p.gc[cg * BT * MS + e];

  for (int hq = h * p.NG; hq < (h + 1) * p.NG; ++hq)
  for (int r = 0; r < rows; ++r) {
    if (!((bits >> (r >> 4)) & 1)) continue;
    const int t = c0 + r;
    __syncthreads();   // state tables are in place; the previous row is finished
    const bf16_t* qsw = p.q_swa + ((int64_t)t * HQ + hq) * D;
    const bf16_t* qgs = p.q_gsa + ((int64_t)t * HQ + hq) * D;
    for (int i = tid; i < D; i += 256) {
      qg[i] = bf16_to_f32(qgs[i]) * p.scale;
      qs[i] = bf16_to_f32(qsw[i]) * p.scale;
    }
    if (tid < MS) gct[tid] = gcl[r * MS + tid];
    if (tid < BT) {
      const int tl = it * BT + tid - p.shift;
      src[tid] = (tid <= r && tl >= 0) ? bos + tl : -1;
    }
    __syncthreads();
    if (tid < BT) {
      const int sj = src[tid];
      Aj[tid] = sj >= 0 ? dot_row<bf16_t>(qg, p.k_gsa + ((int64_t)sj * H + h) * D, D) : 0.f;
    }
    __syncthreads();
    float lmax = -INFINITY;
    if (tid < MS) {
      const int m = tid;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += qg[d] * hk[m * LDH + d];
      acc *= expf(gct[m]);
      for (int j = 0; j <= r; ++j) {
        const int sj = src[j];
        if (sj >= 0) acc += Aj[j] * bf16_to_f32(p.s[((int64_t)sj * H + h) * MS + m]) * expf(gct[m] - gcl[j * MS + m]);
      }
      okl[m] = acc;
      lmax = acc;
    }
    const float mg = block_max(lmax, red);
    const float lg = block_sum(tid < MS ? expf(okl[tid] - mg) : 0.f, red);
    const int lo = p.wl < 0 ? bos : (t - p.wl > bos ? t - p.wl : bos);
    float wm = -INFINITY, wsum = 0.f;
    for (int j = lo + tid; j <= t; j += 256) {
      const float d = dot_row<bf16_t>(qs, p.k_swa + ((int64_t)j * H + h) * D, D);
      if (d > wm) {
        wsum = wsum * expf(wm - d) + 1.f;
        wm = d;
      } else {
        wsum += expf(d - wm);
      }
    }
    const float mw = block_max(wm, red);
    const float lw = block_sum(wm == -INFINITY ? 0.f : wsum * expf(wm - mw), red);
    if (tid == 0) {
      if (p.lse_gsa) p.lse_gsa[(int64_t)t * HQ + hq] = mg + logf(lg);
      if (p.lse_swa) p.lse_swa[(int64_t)t * HQ + hq] = mw + logf(lw);
    }
    const float mt = fmaxf(mg, mw);
    const float inv = 1.f / (lg * expf(mg - mt) + lw * expf(mw - mt));
    __syncthreads();
    if (tid < MS) okl[tid] = expf(okl[tid] - mt) * inv;
    __syncthreads();
    if (tid < BT) {
      const int sj = src[tid];
      float acc = 0.f;
      if (sj >= 0) {
        const bf16_t* srow = p.s + ((int64_t)sj * H + h) * MS;
        for (int m = 0; m < MS; ++m) acc += okl[m] * bf16_to_f32(srow[m]) * expf(gct[m] - gcl[tid * MS + m]);
      }
      Avj[tid] = acc;
    }
    __syncthreads();
    float acc = 0.f;   // value column tid (D <= 256 == threads)
    if (tid < D) {
      for (int m = 0; m < MS; ++m) acc += okl[m] * expf(gct[m]) * hv[m * D + tid];
      for (int j = 0; j <= r; ++j) {
        const int sj = src[j];
        if (sj >= 0) acc += Avj[j] * bf16_to_f32(p.v[((int64_t)sj * H + h) * D + tid]);
      }
    }
    for (int jb = lo; jb <= t; jb += 256) {
      const int j = jb + tid;
      __syncthreads();
      pw[tid] = j <= t ? expf(dot_row<bf16_t>(qs, p.k_swa + ((int64_t)j * H + h) * D, D) - mt) * inv : 0.f;
      __syncthreads();
      const int cnt = (t - jb + 1) < 256 ? (t - jb + 1) : 256;
      if (tid < D)
        for (int x = 0; x < cnt; ++x) acc += pw[x] * bf16_to_f32(p.v[((int64_t)(jb + x) * H + h) * D + tid]);
    }
    if (tid < D) p.o[((int64_t)t * HQ + hq) * D + tid] = f32_to_bf16(acc);
  }
}

template <int D>
int launch_repair(const MP& p, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  const size_t lds = RepairSmem<D>::floats * 4;
  std::call_once(once, [&] { attr_err = hipFuncSetAttribute((const void*)mfma_repair_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_fwd(mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((mfma_repair_kernel<D>), dim3(p.NT, p.H), dim3(256), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma repair pass)");
  return NHA_OK;
}

// ==========================================================================================
// fp32 copies of what the state pass left in the scratch for the backward pass: true chunk-start
// states as hk [K][M] and transposed hk^T [M][K], hv^T [V][M], plus bf16 copies hk^T [M][K] and
// hv [M][V] as matrix-core operands; gate cumsums per row token
// ==========================================================================================
template <int D>
__global__ __launch_bounds__(256) void export_states_kernel(const MP p, float* gc, float* hkc, float* hkct, float* hvct, bf16_t* hkb, bf16_t* hvb, bf16_t* hkl,
                                                          bf16_t* hvl, int* big) {
  const int chunk = blockIdx.x, h = blockIdx.y, H = p.H;
  const int tid = threadIdx.x;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const int64_t cg = (int64_t)chunk * H + h;
  const int64_t sl = (int64_t)seg_slot(p.coff, n, it) * H + h;
  // eight consecutive d of one slot per thread and trip: 16-byte reads of the bf16 local states, 32-byte
  // reads of the fp32 segment states, 16-byte writes of the four bf16 copies
  for (int e8 = tid; e8 < MS * D / 8; e8 += 256) {
    const int m = e8 / (D / 8), d = (e8 % (D / 8)) * 8;
    const float dc = p.dcum[cg * MS + m];
    const int64_t li = (cg * MS + m) * D + d, si = (sl * MS + m) * D + d;
    float lk[8], lv[8], sk[8], sv[8], hk[8], hv[8];
    Elem<bf16_t>::ld8(p.hkT + li, lk);
    Elem<bf16_t>::ld8(p.hvc + li, lv);
    Elem<float>::ld8(p.hseg_k + si, sk);
    Elem<float>::ld8(p.hseg_v + si, sv);
    uint32_t kh[4], vh[4], kl[4], vl[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      hk[j] = lk[j] + sk[j] * dc;
      hv[j] = lv[j] + sv[j] * dc;
    }
    // bf16 pairs hi + lo: the backward multiplies by hi and by lo
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bf16_t k0 = f32_to_bf16(hk[2 * j]), k1 = f32_to_bf16(hk[2 * j + 1]);
      const bf16_t v0 = f32_to_bf16(hv[2 * j]), v1 = f32_to_bf16(hv[2 * j + 1]);
      kh[j] = (uint32_t)k0 | ((uint32_t)k1 << 16);
      vh[j] = (uint32_t)v0 | ((uint32_t)v1 << 16);
      kl[j] = (uint32_t)f32_to_bf16(hk[2 * j] - bf16_to_f32(k0)) | ((uint32_t)f32_to_bf16(hk[2 * j + 1] - bf16_to_f32(k1)) << 16);
      vl[j] = (uint32_t)f32_to_bf16(hv[2 * j] - bf16_to_f32(v0)) | ((uint32_t)f32_to_bf16(hv[2 * j + 1] - bf16_to_f32(v1)) << 16);
    }
    *reinterpret_cast<uint4*>(hkb + li) = make_uint4(kh[0], kh[1], kh[2], kh[3]);
    *reinterpret_cast<uint4*>(hvb + li) = make_uint4(vh[0], vh[1], vh[2], vh[3]);
    *reinterpret_cast<uint4*>(hkl + li) = make_uint4(kl[0], kl[1], kl[2], kl[3]);
    *reinterpret_cast<uint4*>(hvl + li) = make_uint4(vl[0], vl[1], vl[2], vl[3]);
    if (hkc) {   // fp32 copies: only the VALU kernels of the backward read them
      Elem<float>::st8(hkct + li, hk);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        hkc[(cg * D + d + j) * MS + m] = hk[j];
        hvct[(cg * D + d + j) * MS + m] = hv[j];
      }
    }
  }
  for (int e4 = tid; e4 < R * MS / 4; e4 += 256) {
    const int r = e4 / (MS / 4), m4 = (e4 % (MS / 4)) * 4;
    *reinterpret_cast<float4*>(gc + ((int64_t)(c0 + r) * H + h) * MS + m4) = *reinterpret_cast<const float4*>(p.gc + cg * BT * MS + r * MS + m4);
  }
  // chunks in which some slot decays by more than e^-BWD_DECAY_CLAMP over one of the two 32-row halves: the
  // backward's factored products (e^(gc_i - ref) e^(ref - gc_j) as two operands, ref = the start of
  // j's half) leave the bf16 / fp32 range there.  One slot per lane of the first wave.
  if (tid < 64) {
    const float* g = p.gc + cg * BT * MS;
    const int m = tid;
    const float g31 = g[(R > 32 ? 31 : R - 1) * MS + m];
    const bool b = (g31 < -BWD_DECAY_CLAMP) | (g[(R - 1) * MS + m] - g31 < -BWD_DECAY_CLAMP);
    const bool any = __any(b);
    if (tid == 0) big[cg] = any ? 1 : 0;
  }
}

template <int D, int G, int NW, int TK>
int launch_out(const MP& p, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  const size_t lds = OutSmem<D, TK>::bytes;
  std::call_once(once, [&] { attr_err = hipFuncSetAttribute((const void*)mfma_out_kernel<D, G, NW, TK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_fwd(mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL((mfma_out_kernel<D, G, NW, TK>), dim3(p.H * (p.NG / G), p.NT), dim3(64 * NW), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma output pass)");
  return NHA_OK;
}

// state pass: level 1, then level 2 in the forward form (true chunk-start states in place) or, for
// the backward's state export, in the segment form (segment-start states beside the local ones)
template <int D>
int run_state_pass(const MP& p, bool segment_form, hipStream_t st) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  constexpr int DW = D >= 256 ? D / 2 : D;   // measured: 96 -> 88 us at B=8 T=2048 H=4 D=256; no gain at D = 128
  const size_t lds = (size_t)BT * (DW + 16) * 2 + (size_t)2 * BT * SLD * 2;
  std::call_once(once, [&] { attr_err = hipFuncSetAttribute((const void*)mfma_state_local_kernel<D, DW>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_fwd(mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  // at most NT / SEG + N segments: every sequence but for its last segment fills SEG chunks
  const int64_t l1_grid = (int64_t)(p.NT / SEG + p.N) * p.H * 2 * (D / DW);
  if (l1_grid > 0x7fffffff) {
    set_error("nha_prefill_fwd(mfma): too many segments for one launch (%lld workgroups)", (long long)l1_grid);
    return NHA_ERR_UNSUPPORTED;
  }
  hipLaunchKernelGGL((mfma_state_local_kernel<D, DW>), dim3((unsigned)l1_grid), dim3(256), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma state pass, level 1)");
  // the forward's chunk states: inside the scan while a sequence has about eight segments or fewer (a thread's
  // chain there costs a memory latency per segment: 15 us at 4 segments, 21 us at 16 on one box), after it beyond
  // (two launches without a chain: 16-18 us whatever the length)
  const bool in_scan = !segment_form && (int64_t)p.NT <= (int64_t)8 * SEG * p.N;
  if (in_scan) {
    hipLaunchKernelGGL((state_final_kernel<D>), dim3(p.N * p.H, 2 * MS * D / 1024), dim3(256), 0, st, p);
  } else {
    hipLaunchKernelGGL((state_scan_kernel<D>), dim3(p.N * p.H, 2 * MS * D / 1024), dim3(256), 0, st, p);
    if (!segment_form) hipLaunchKernelGGL((state_apply_kernel<D>), dim3(p.NT / SEG + p.N + 1, p.H, 2 * MS * D / 1024), dim3(256), 0, st, p);
  }
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma state pass, level 2)");
  return NHA_OK;
}

template <int D>
int run_mfma(const MP& p, int phases, hipStream_t st) {
  if (p.NT > 65535) {
    set_error("nha_prefill_fwd(mfma): more than 65535 chunks (%d) in one call", p.NT);
    return NHA_ERR_UNSUPPORTED;
  }
  if (phases != 2) {
    const int rc = run_state_pass<D>(p, false, st);
    if (rc != NHA_OK) return rc;
  }
  if (phases != 1) {
    // G query heads of one kv-head share a workgroup.  D <= 128: 64-key tiles, 8 waves of 32 (G = 4)
    // or 16 (G = 2) query rows, two per SIMD; D = 256: 32-key tiles and 16-row waves to fit the
    // register file and LDS
    int rc;
#ifdef NHA_AB_SWITCHES   // measurement builds only (-DNHA_AB_SWITCHES): run the kernels the LDS-direct ones replaced
    static const bool ring_off = getenv("NHA_PREFILL_NO_RING") != nullptr;
#else
    constexpr bool ring_off = false;
#endif
    if (!ring_off && prefill_ring_supported(p, D)) {
      rc = prefill_ring_launch(p, D, st);
    } else if (!ring_off && prefill_ring256_supported(p, D)) {
      rc = prefill_ring256_launch(p, st);
    } else if constexpr (D <= 128) {
      if (p.NG % 4 == 0) rc = launch_out<D, 4, 8, 64>(p, st);
      else if (p.NG % 2 == 0) rc = launch_out<D, 2, 8, 64>(p, st);
      else rc = launch_out<D, 1, 4, 64>(p, st);
    } else {
      if (p.NG % 2 == 0) rc = launch_out<D, 2, 8, 32>(p, st);
      else rc = launch_out<D, 1, 4, 32>(p, st);
    }
    if (rc != NHA_OK) return rc;
    return launch_repair<D>(p, st);
  }
  return NHA_OK;
}

static size_t aligned(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

bool prefill_mfma_supported(const NhaPrefillArgs* a) {
  return a->dtype == NHA_DTYPE_BF16 && a->K == a->V && (a->K == 64 || a->K == 128 || a->K == 256) && a->M == MS;
}

namespace {
struct ScratchPlan {
  size_t hkT, hvc, gc, dcum, hend_k, hend_v, hseg_k, hseg_v, dtot, flags, total;
};
ScratchPlan plan_scratch(const NhaPrefillArgs* a) {
  const size_t per = (size_t)a->NT * a->H;
  const size_t nslot = (size_t)a->NT / SEG + a->N + 1;
  const size_t seg = aligned(nslot * a->H * MS * a->K * 4);
  ScratchPlan s;
  size_t off = 0;
  s.hkT = off; off += aligned(per * MS * a->K * 2);
  s.hvc = off; off += aligned(per * MS * a->V * 2);
  s.gc = off; off += aligned(per * BT * MS * 4);
  s.dcum = off; off += aligned(per * MS * 4);
  s.hend_k = off; off += seg;
  s.hend_v = off; off += seg;
  s.hseg_k = off; off += seg;
  s.hseg_v = off; off += seg;
  s.dtot = off; off += aligned(nslot * a->H * MS * 4);
  s.flags = off; off += aligned(per * 4 * 4);
  s.total = off;
  return s;
}
}  // namespace

size_t prefill_mfma_scratch_bytes(const NhaPrefillArgs* a) { return plan_scratch(a).total; }

namespace {
MP make_mp(const NhaPrefillArgs* a) {
  MP p;
  p.q_swa = (const bf16_t*)a->q_swa; p.k_swa = (const bf16_t*)a->k_swa;
  p.q_gsa = (const bf16_t*)a->q_gsa; p.k_gsa = (const bf16_t*)a->k_gsa;
  p.v = (const bf16_t*)a->v; p.s = (const bf16_t*)a->s; p.g = (const bf16_t*)a->g;
  p.o = (bf16_t*)a->o;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa;
  p.h0k = a->h0k; p.h0v = a->h0v; p.hkt = a->hkt; p.hvt = a->hvt;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices; p.coff = a->chunk_offsets;
  const ScratchPlan sp = plan_scratch(a);
  char* sc = (char*)a->scratch;
  p.hkT = (bf16_t*)(sc + sp.hkT);
  p.hvc = (bf16_t*)(sc + sp.hvc);
  p.gc = (float*)(sc + sp.gc);
  p.dcum = (float*)(sc + sp.dcum);
  p.hend_k = (float*)(sc + sp.hend_k);
  p.hend_v = (float*)(sc + sp.hend_v);
  p.hseg_k = (float*)(sc + sp.hseg_k);
  p.hseg_v = (float*)(sc + sp.hseg_v);
  p.dtot = (float*)(sc + sp.dtot);
  p.flags = (int*)(sc + sp.flags);
  p.T_tot = a->T_tot; p.N = a->N; p.NT = a->NT; p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H;
  p.wl = a->wl; p.shift = a->shift; p.scale = a->scale;
  return p;
}
}  // namespace

int prefill_mfma_impl(const NhaPrefillArgs* a, int phase) {
  const MP p = make_mp(a);
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return run_mfma<64>(p, phase, st);
  if (a->K == 128) return run_mfma<128>(p, phase, st);
  return run_mfma<256>(p, phase, st);
}

// Runs the state pass of `a` in the segment form and exports it; gc [T_tot][H][M], hkc
// [NT][H][K][M], hkct [NT][H][M][K], hvct [NT][H][V][M] receive fp32 copies, hkb [NT][H][M][K] and
// hvb [NT][H][M][V] bf16 copies with their low parts hkl, hvl (hkc, hkct, hvct may be NULL together), big [NT][H] the flag of
// chunks with a decay beyond e^-80
int prefill_mfma_export_states(const NhaPrefillArgs* a, float* gc, float* hkc, float* hkct, float* hvct, void* hkb, void* hvb,
                               void* hkl, void* hvl, int* big) {
  const MP p = make_mp(a);
  hipStream_t st = (hipStream_t)a->stream;
  if (p.NT > 65535) {
    set_error("nha_prefill_bwd(mfma): more than 65535 chunks (%d) in one call", p.NT);
    return NHA_ERR_UNSUPPORTED;
  }
  const int rcs = a->K == 64 ? run_state_pass<64>(p, true, st) : a->K == 128 ? run_state_pass<128>(p, true, st) : run_state_pass<256>(p, true, st);
  if (rcs != NHA_OK) return rcs;
  const dim3 grid(a->NT, a->H);
  if (a->K == 64) hipLaunchKernelGGL((export_states_kernel<64>), grid, dim3(256), 0, st, p, gc, hkc, hkct, hvct, (bf16_t*)hkb, (bf16_t*)hvb, (bf16_t*)hkl, (bf16_t*)hvl, big);
  else if (a->K == 128) hipLaunchKernelGGL((export_states_kernel<128>), grid, dim3(256), 0, st, p, gc, hkc, hkct, hvct, (bf16_t*)hkb, (bf16_t*)hvb, (bf16_t*)hkl, (bf16_t*)hvl, big);
  else hipLaunchKernelGGL((export_states_kernel<256>), grid, dim3(256), 0, st, p, gc, hkc, hkct, hvct, (bf16_t*)hkb, (bf16_t*)hvb, (bf16_t*)hkl, (bf16_t*)hvl, big);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(state export)");
  return NHA_OK;
}

}  // namespace nha
