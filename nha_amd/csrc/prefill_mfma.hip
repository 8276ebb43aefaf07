// bf16 MFMA prefill for gfx950 (K == V == D in {64,128}, M == 64 slots), fp32 accumulation.
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
#include "common.h"

namespace nha {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int BT = 64;        // chunk rows == window tile keys
constexpr int MS = 64;        // slots
constexpr int GLD = 68;       // LDS row stride (floats) of the gate-cumsum tables
constexpr int SLD = 72;       // LDS row stride (bf16) of the s tables
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float DECAY_CLAMP = 80.f;   // largest positive decay exponent formed on the MFMA path

struct MP {
  const bf16_t *q_swa, *k_swa, *q_gsa, *k_gsa, *v, *s, *g;
  bf16_t* o;
  float *lse_swa, *lse_gsa;
  const float *h0k, *h0v;
  float *hkt, *hvt;
  const int32_t *cu, *cidx, *coff;
  bf16_t* hkT;   // [NT][H][MS][D]   chunk-start k-state, transposed
  bf16_t* hvc;   // [NT][H][MS][D]   chunk-start v-state
  float* gc;     // [NT][H][BT][MS]  chunk-local inclusive gate cumsum
  int T_tot, N, NT, HQ, H, NG, wl, shift;
  float scale;
};

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 u) { return __builtin_bit_cast(bf16x8, u); }
__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fexp(float x) { return __builtin_amdgcn_exp2f(x * LOG2E); }

__device__ __forceinline__ bf16x8 pack8(f32x4 a, f32x4 b) {
  bf16x8 r;
  r[0] = (__bf16)a[0]; r[1] = (__bf16)a[1]; r[2] = (__bf16)a[2]; r[3] = (__bf16)a[3];
  r[4] = (__bf16)b[0]; r[5] = (__bf16)b[1]; r[6] = (__bf16)b[2]; r[7] = (__bf16)b[3];
  return r;
}

// A/B fragment of a row-major LDS tile: 8 consecutive elements of row `row` starting at `col`.
__device__ __forceinline__ bf16x8 lds_frag(const bf16_t* tile, int ld, int row, int col) {
  return as_bf16x8(*reinterpret_cast<const uint4*>(tile + row * ld + col));
}

// Transposed fragment of a row-major [rows][ld] bf16 LDS tile: the lane (c = l%16, kb = l/16)
// receives X[r0a + 4*kb + e][col0 + c] for e = 0..3 and X[r0b + 4*kb + e][col0 + c] for e = 4..7.
__device__ __forceinline__ bf16x8 lds_frag_tr(const bf16_t* tile, int ld, int r0a, int r0b, int col0, int lane) {
  const int l16 = lane & 15, kb = lane >> 4;
  const bf16_t* pa = tile + (r0a + 4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  const bf16_t* pb = tile + (r0b + 4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  struct { s16x4 a, b; } t;
  t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)pa);
  t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)pb);
  return __builtin_bit_cast(bf16x8, t);
}

// ------------------------------------------------------------------------------------------
// cooperative 64-row tile copy, global -> registers -> LDS (16-byte pieces, zero fill)
// ------------------------------------------------------------------------------------------
template <int D>
struct TileRegs {
  uint4 r[D / 32];
};

// rows of the tile map to global rows grow0 + j; rows outside [vlo, vhi) are zero
template <int D>
__device__ __forceinline__ void tile_g2r(TileRegs<D>& t, const bf16_t* base, int64_t row_stride, int64_t grow0,
                                         int vlo, int vhi, int tid) {
#pragma unroll
  for (int u = 0; u < D / 32; ++u) {
    const int c = tid + 256 * u;
    const int row = c / (D / 8), col = (c % (D / 8)) * 8;
    uint4 x = make_uint4(0, 0, 0, 0);
    if (row >= vlo && row < vhi) x = *reinterpret_cast<const uint4*>(base + (grow0 + row) * row_stride + col);
    t.r[u] = x;
  }
}
template <int D>
__device__ __forceinline__ void tile_r2l(bf16_t* lds, const TileRegs<D>& t, int tid) {
#pragma unroll
  for (int u = 0; u < D / 32; ++u) {
    const int c = tid + 256 * u;
    const int row = c / (D / 8), col = (c % (D / 8)) * 8;
    *reinterpret_cast<uint4*>(lds + row * (D + 16) + col) = t.r[u];
  }
}

// ==========================================================================================
// state pass
// ==========================================================================================
template <int D>
__global__ __launch_bounds__(256) void mfma_state_kernel(const MP p) {
  constexpr int LDT = D + 16;
  constexpr int BPW = D / 64;   // 16-wide blocks of the head dim per wave
  __shared__ __align__(16) bf16_t Kt[2][BT * LDT];
  __shared__ __align__(16) bf16_t Vt[2][BT * LDT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H;
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const int mb = blockIdx.y * 16;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int L = eos - bos;
  const int nchunks = (L + BT - 1) / BT;
  const int c0g = p.coff[n];
  const int m = mb + l16;   // this lane's slot in the B/A fragments and in hk's accumulator columns

  // accumulators: hk[kk block][.] : C[kk = 4*kb + r][m = l16];  hv[.][vv block] : C[m = 4*kb + r][vv = l16]
  f32x4 hk[BPW], hv[BPW];
#pragma unroll
  for (int b = 0; b < BPW; ++b) {
    const int d0 = (wave * BPW + b) * 16;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      hk[b][r] = p.h0k ? p.h0k[(((int64_t)n * H + h) * D + d0 + 4 * kb + r) * MS + m] : 0.f;
      hv[b][r] = p.h0v ? p.h0v[(((int64_t)n * H + h) * MS + mb + 4 * kb + r) * D + d0 + l16] : 0.f;
    }
  }

  TileRegs<D> rk, rv;
  // this lane's g / s values: element e = 4*q + r is row t = 16*q + 4*kb + r of the chunk
  float gq[16], sq[16];
  auto issue = [&](int it) {
    const int rows = (L - it * BT) < BT ? (L - it * BT) : BT;
    const int64_t grow0 = (int64_t)bos + it * BT - p.shift;
    int vlo = p.shift - it * BT;
    vlo = vlo < 0 ? 0 : vlo;
    tile_g2r<D>(rk, p.k_gsa + (int64_t)h * D, (int64_t)H * D, grow0, vlo, rows, tid);
    tile_g2r<D>(rv, p.v + (int64_t)h * D, (int64_t)H * D, grow0, vlo, rows, tid);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int t = 16 * (e >> 2) + 4 * kb + (e & 3);
      float gv = 0.f, sv = 0.f;
      if (t >= vlo && t < rows) {
        const int64_t off = ((grow0 + t) * H + h) * MS + m;
        gv = bf16_to_f32(p.g[off]);
        sv = bf16_to_f32(p.s[off]);
      }
      gq[e] = gv;
      sq[e] = sv;
    }
  };

  if (nchunks > 0) issue(0);
  for (int it = 0; it < nchunks; ++it) {
    const int cur = it & 1;
    const int rows = (L - it * BT) < BT ? (L - it * BT) : BT;
    tile_r2l<D>(Kt[cur], rk, tid);
    tile_r2l<D>(Vt[cur], rv, tid);
    // inclusive cumsum over t for this lane's slot: four runs of 4 rows per lane, 16 runs per slot
    float gcv[16], sg[16];
    {
      float run[4], base = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float a = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          a += gq[4 * q + r];
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
    // gc of the chunk's last valid row, for this lane's slot
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
    if (wave == 0) {
      float* gout = p.gc + (((int64_t)(c0g + it) * H + h) * BT) * MS + m;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int t = 16 * (e >> 2) + 4 * kb + (e & 3);
        gout[(int64_t)t * MS] = gcv[e];
      }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int t = 16 * (e >> 2) + 4 * kb + (e & 3);
      sg[e] = (t < rows) ? sq[e] * fexp(glast - gcv[e]) : 0.f;
    }
    bf16x8 sg0, sg1;   // contraction steps over rows [0,32) and [32,64)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sg0[e] = (__bf16)sg[e];
      sg1[e] = (__bf16)sg[8 + e];
    }
    // chunk-start states (bf16), before the update
    {
      const int64_t cg = (int64_t)(c0g + it) * H + h;
#pragma unroll
      for (int b = 0; b < BPW; ++b) {
        const int d0 = (wave * BPW + b) * 16;
        bf16x4 pk;
#pragma unroll
        for (int r = 0; r < 4; ++r) pk[r] = (__bf16)hk[b][r];
        *reinterpret_cast<bf16x4*>(p.hkT + (cg * MS + m) * D + d0 + 4 * kb) = pk;
#pragma unroll
        for (int r = 0; r < 4; ++r) p.hvc[(cg * MS + mb + 4 * kb + r) * D + d0 + l16] = f32_to_bf16(hv[b][r]);
      }
    }
    if (it + 1 < nchunks) issue(it + 1);
    __syncthreads();
    // decay, then accumulate this chunk
    const float dk = fexp(glast);
    float dv[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) dv[r] = __shfl(dk, 4 * kb + r, 64);
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
      const int d0 = (wave * BPW + b) * 16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        hk[b][r] *= dk;
        hv[b][r] *= dv[r];
      }
      // hk[kk][m] += sum_t k[t][kk] sg[t][m]      A = k^T (transposed read), B = sg
      hk[b] = mfma16(lds_frag_tr(Kt[cur], LDT, 0, 16, d0, lane), sg0, hk[b]);
      hk[b] = mfma16(lds_frag_tr(Kt[cur], LDT, 32, 48, d0, lane), sg1, hk[b]);
      // hv[m][vv] += sum_t sg[t][m] v[t][vv]      A = sg^T (same registers), B = v (transposed read)
      hv[b] = mfma16(sg0, lds_frag_tr(Vt[cur], LDT, 0, 16, d0, lane), hv[b]);
      hv[b] = mfma16(sg1, lds_frag_tr(Vt[cur], LDT, 32, 48, d0, lane), hv[b]);
    }
  }
  if (p.hkt) {
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
      const int d0 = (wave * BPW + b) * 16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p.hkt[(((int64_t)n * H + h) * D + d0 + 4 * kb + r) * MS + m] = hk[b][r];
        p.hvt[(((int64_t)n * H + h) * MS + mb + 4 * kb + r) * D + d0 + l16] = hv[b][r];
      }
    }
  }
}


// ==========================================================================================
// output pass
// ==========================================================================================
// One workgroup = one 64-row chunk x G query heads of one kv-head (G in {1,2,4}); wave w owns
// RQB = G blocks of 16 query rows of head w / (4/G).  LDS: two K-tile and two V-tile buffers
// (double buffered window stream; they first hold hkT, k_gsa rows, hv, v rows of the slot branch)
// plus the chunk's gate-cumsum / s tables in both orientations.
template <int D>
struct OutSmem {
  static constexpr int LDT = D + 16;
  static constexpr size_t tile_bytes = (size_t)BT * LDT * 2;
  static constexpr size_t bytes = 4 * tile_bytes + 2 * (size_t)BT * GLD * 4 + 2 * (size_t)BT * SLD * 2;
};

template <int D, int G>
__global__ __launch_bounds__(256, 1) void mfma_out_kernel(const MP p) {
  constexpr int RQB = G;
  constexpr int WPU = 4 / G;
  constexpr int KS = D / 32;
  constexpr int DB = D / 16;
  constexpr int LDT = D + 16;
  extern __shared__ __align__(16) unsigned char smem[];
  bf16_t* Kb[2];
  bf16_t* Vb[2];
  Kb[0] = (bf16_t*)smem;
  Kb[1] = Kb[0] + BT * LDT;
  Vb[0] = Kb[1] + BT * LDT;
  Vb[1] = Vb[0] + BT * LDT;
  float* gcR = (float*)(Vb[1] + BT * LDT);   // [row j][slot m]
  float* gcT = gcR + BT * GLD;               // [slot m][row j]
  bf16_t* sR = (bf16_t*)(gcT + BT * GLD);    // [row j][slot m]
  bf16_t* sT = sR + BT * SLD;                // [slot m][row j]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  const int chunk = blockIdx.x;
  const int ngrp = NG / G;
  const int h = blockIdx.y / ngrp, grp = blockIdx.y % ngrp;
  const int hq = h * NG + grp * G + wave / WPU;
  const int qb0 = (wave % WPU) * RQB;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  const float cs = p.scale * LOG2E;   // logits are kept unscaled; p = exp2(cs * (s - m))

  // ---- window tile schedule: tile i covers keys [c0 - 64 i, c0 - 64 i + 63] -----------------
  int n_last = it;   // tiles may not start before bos
  if (p.wl >= 0) {
    const int w = (p.wl + 63) / 64;
    n_last = w < n_last ? w : n_last;
  }
  const int ntiles = n_last + 1;
  TileRegs<D> rk, rv;
  auto issue_window = [&](int i) {
    const int64_t grow0 = (int64_t)c0 - 64 * i;
    const int vhi = i == 0 ? rows : BT;
    tile_g2r<D>(rk, p.k_swa + (int64_t)h * D, (int64_t)H * D, grow0, 0, vhi, tid);
    tile_g2r<D>(rv, p.v + (int64_t)h * D, (int64_t)H * D, grow0, 0, vhi, tid);
  };

  // ---- phase 0: slot-branch operands -> LDS --------------------------------------------------
  {
    const int64_t cg = (int64_t)chunk * H + h;
    int vlo = p.shift - it * BT;
    vlo = vlo < 0 ? 0 : vlo;
    const int64_t grow0 = (int64_t)c0 - p.shift;
    TileRegs<D> a, b, c, d;
    tile_g2r<D>(a, p.hkT + cg * MS * D, D, 0, 0, BT, tid);
    tile_g2r<D>(b, p.k_gsa + (int64_t)h * D, (int64_t)H * D, grow0, vlo, rows, tid);
    tile_g2r<D>(c, p.hvc + cg * MS * D, D, 0, 0, BT, tid);
    tile_g2r<D>(d, p.v + (int64_t)h * D, (int64_t)H * D, grow0, vlo, rows, tid);
    tile_r2l<D>(Kb[0], a, tid);
    tile_r2l<D>(Kb[1], b, tid);
    tile_r2l<D>(Vb[0], c, tid);
    tile_r2l<D>(Vb[1], d, tid);
    // gate cumsum table (fp32 [64][64]) in both orientations; rows past the sequence end are zero
    const float* gsrc = p.gc + cg * BT * MS;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int cidx4 = tid + 256 * u;
      const int j = cidx4 >> 4, m4 = (cidx4 & 15) * 4;
      float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
      if (j < rows) x = *reinterpret_cast<const float4*>(gsrc + j * MS + m4);
      *reinterpret_cast<float4*>(gcR + j * GLD + m4) = x;
      gcT[(m4 + 0) * GLD + j] = x.x;
      gcT[(m4 + 1) * GLD + j] = x.y;
      gcT[(m4 + 2) * GLD + j] = x.z;
      gcT[(m4 + 3) * GLD + j] = x.w;
    }
    // s rows of the slot branch (shifted), both orientations
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c8 = tid + 256 * u;
      const int j = c8 >> 3, m8 = (c8 & 7) * 8;
      uint4 x = make_uint4(0, 0, 0, 0);
      if (j >= vlo && j < rows) x = *reinterpret_cast<const uint4*>(p.s + ((grow0 + j) * H + h) * MS + m8);
      *reinterpret_cast<uint4*>(sR + j * SLD + m8) = x;
      const uint32_t w4[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) sT[(m8 + e) * SLD + j] = (bf16_t)(w4[e >> 1] >> (16 * (e & 1)));
    }
  }
  issue_window(0);
  __syncthreads();

  // per-lane softmax state for the RQB queries (l16 + 16*(qb0+qb)) this lane serves
  float mrun[RQB], lg[RQB], lw[RQB];
  f32x4 O[DB][RQB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) O[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // ---- phase 1: slot branch, one 16-row query block at a time --------------------------------
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
    for (int mb = 0; mb < 4; ++mb) {
      ok[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ok[mb] = mfma16(lds_frag(Kb[0], LDT, 16 * mb + l16, 32 * ks + 8 * kb), qf[ks], ok[mb]);
    }
    // intra-chunk scores AT[j][i] = sum_d k_gsa[j][d] q[i][d] for row blocks jb <= Q, masked j <= i
    bf16x8 bA[2];
    {
      f32x4 at[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        at[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (jb <= Q) {
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            at[jb] = mfma16(lds_frag(Kb[1], LDT, 16 * jb + l16, 32 * ks + 8 * kb), qf[ks], at[jb]);
          if (jb == Q) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (4 * kb + r > l16) at[jb][r] = 0.f;
          }
        }
      }
      bA[0] = pack8(at[0], at[1]);
      bA[1] = pack8(at[2], at[3]);
    }
    // decay reference of this sub-block: gc at the row before it (0 for the first sub-block)
    const int rref = 16 * Q - 1;
    // okT_intra[m][i] = sum_j s_j[m] exp(gr[m] - gc_j[m]) AT[j][i]
    f32x4 oki[4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      oki[mb] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const int mrow = 16 * mb + l16;
      const float gr = Q > 0 ? gcT[mrow * GLD + rref] : 0.f;
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        if (2 * pr <= Q) {
          bf16x8 se;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int jb = 2 * pr + half;
            const int j0 = 16 * jb + 4 * kb;
            const float4 gj = *reinterpret_cast<const float4*>(gcT + mrow * GLD + j0);
            const bf16x4 sj = *reinterpret_cast<const bf16x4*>(sT + mrow * SLD + j0);
            const float gv[4] = {gj.x, gj.y, gj.z, gj.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float val = 0.f;
              if (jb <= Q) val = (float)sj[e] * fexp(fminf(gr - gv[e], DECAY_CLAMP));
              se[4 * half + e] = (__bf16)val;
            }
          }
          oki[mb] = mfma16(se, bA[pr], oki[mb]);
        }
      }
    }
    // combine, then the slot "tile" of the online softmax (logits unscaled, exponent scale cs)
    float rmax = -INFINITY;
    f32x4 egi[4], egr[4];   // exp(gc_i[m]) and exp(gc_i[m] - gr[m]) in accumulator layout
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) {
      const float4 gi = *reinterpret_cast<const float4*>(gcR + irow * GLD + 16 * mb + 4 * kb);
      float4 gr4 = make_float4(0.f, 0.f, 0.f, 0.f);
      if (Q > 0) gr4 = *reinterpret_cast<const float4*>(gcR + rref * GLD + 16 * mb + 4 * kb);
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
    rmax = fmaxf(rmax, __shfl_xor(rmax, 16, 64));
    rmax = fmaxf(rmax, __shfl_xor(rmax, 32, 64));
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
    lw[qb] = 0.f;
    if (p.lse_gsa) {
      float tot = psum + __shfl_xor(psum, 16, 64);
      tot += __shfl_xor(tot, 32, 64);
      if (kb == 0 && irow < rows) p.lse_gsa[(int64_t)(c0 + irow) * HQ + hq] = (mc + __builtin_amdgcn_logf(tot)) * LN2;
    }
    // slot read, inter-chunk part: O^T[d][i] += sum_m hv[m][d] (p[i][m] exp(gc_i[m]))
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      f32x4 x0, x1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        x0[r] = ok[2 * pr][r] * egi[2 * pr][r];
        x1[r] = ok[2 * pr + 1][r] * egi[2 * pr + 1][r];
      }
      const bf16x8 bp = pack8(x0, x1);
#pragma unroll
      for (int db = 0; db < DB; ++db)
        O[db][qb] = mfma16(lds_frag_tr(Vb[0], LDT, 32 * pr, 32 * pr + 16, 16 * db, lane), bp, O[db][qb]);
    }
    // slot read, intra-chunk part: AvT[j][i] = sum_m s_j[m] exp(gr[m]-gc_j[m]) (p[i][m] exp(gc_i[m]-gr[m]))
    bf16x8 bpr[2];
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      f32x4 x0, x1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        x0[r] = ok[2 * pr][r] * egr[2 * pr][r];
        x1[r] = ok[2 * pr + 1][r] * egr[2 * pr + 1][r];
      }
      bpr[pr] = pack8(x0, x1);
    }
    bf16x8 bAv[2];
    {
      f32x4 av[4];
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        av[jb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        if (jb <= Q) {
          const int jrow = 16 * jb + l16;
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            bf16x8 se;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              const int m0 = 32 * pr + 16 * half + 4 * kb;
              const float4 gj = *reinterpret_cast<const float4*>(gcR + jrow * GLD + m0);
              float4 gr4 = make_float4(0.f, 0.f, 0.f, 0.f);
              if (Q > 0) gr4 = *reinterpret_cast<const float4*>(gcR + rref * GLD + m0);
              const bf16x4 sj = *reinterpret_cast<const bf16x4*>(sR + jrow * SLD + m0);
              const float gv[4] = {gj.x, gj.y, gj.z, gj.w};
              const float grv[4] = {gr4.x, gr4.y, gr4.z, gr4.w};
#pragma unroll
              for (int e = 0; e < 4; ++e)
                se[4 * half + e] = (__bf16)((float)sj[e] * fexp(fminf(grv[e] - gv[e], DECAY_CLAMP)));
            }
            av[jb] = mfma16(se, bpr[pr], av[jb]);
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
    for (int pr = 0; pr < 2; ++pr) {
      if (2 * pr <= Q) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
          O[db][qb] = mfma16(lds_frag_tr(Vb[1], LDT, 32 * pr, 32 * pr + 16, 16 * db, lane), bAv[pr], O[db][qb]);
      }
    }
  }

  // ---- phase 2: sliding window, streamed in 64-key tiles --------------------------------------
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
  __syncthreads();   // every wave is done with the slot-branch tiles
  tile_r2l<D>(Kb[0], rk, tid);
  tile_r2l<D>(Vb[0], rv, tid);
  if (ntiles > 1) issue_window(1);
  __syncthreads();

  for (int i = 0; i < ntiles; ++i) {
    const int cur = i & 1;
    const bf16_t* Kt = Kb[cur];
    const bf16_t* Vt = Vb[cur];
    // S^T[key][q] for 4 key blocks x RQB query blocks
    f32x4 S[4][RQB];
#pragma unroll
    for (int kblk = 0; kblk < 4; ++kblk) {
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) S[kblk][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 a = lds_frag(Kt, LDT, 16 * kblk + l16, 32 * ks + 8 * kb);
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) S[kblk][qb] = mfma16(a, qs[qb][ks], S[kblk][qb]);
      }
    }
    const bool edge = (i == 0) || (p.wl >= 0 && 64 * i + 63 > p.wl);
    if (edge) {
#pragma unroll
      for (int kblk = 0; kblk < 4; ++kblk)
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) {
          const int y = 16 * (qb0 + qb) + l16;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int x = 16 * kblk + 4 * kb + r - 64 * i;   // key offset relative to the chunk start
            const bool ok = (x <= y) && (p.wl < 0 || x >= y - p.wl);
            if (!ok) S[kblk][qb][r] = -INFINITY;
          }
        }
    }
    // online softmax per query column
    bf16x8 P[2][RQB];
    bool any_rescale = false;
    float alpha[RQB];
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      float rmax = S[0][qb][0];
#pragma unroll
      for (int kblk = 0; kblk < 4; ++kblk)
#pragma unroll
        for (int r = 0; r < 4; ++r) rmax = fmaxf(rmax, S[kblk][qb][r]);
      rmax = fmaxf(rmax, __shfl_xor(rmax, 16, 64));
      rmax = fmaxf(rmax, __shfl_xor(rmax, 32, 64));
      const float mnew = fmaxf(mrun[qb], rmax);
      alpha[qb] = fexp2((mrun[qb] - mnew) * cs);
      any_rescale |= (mnew != mrun[qb]);
      mrun[qb] = mnew;
      const float mc = mnew * cs;
      float psum = 0.f;
#pragma unroll
      for (int kblk = 0; kblk < 4; ++kblk)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float e = fexp2(S[kblk][qb][r] * cs - mc);
          S[kblk][qb][r] = e;
          psum += e;
        }
      lw[qb] = lw[qb] * alpha[qb] + psum;
      lg[qb] *= alpha[qb];
      P[0][qb] = pack8(S[0][qb], S[1][qb]);
      P[1][qb] = pack8(S[2][qb], S[3][qb]);
    }
    if (__any(any_rescale)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb)
#pragma unroll
          for (int r = 0; r < 4; ++r) O[db][qb][r] *= alpha[qb];
    }
    // O^T[d][q] += V^T P^T
#pragma unroll
    for (int pr = 0; pr < 2; ++pr)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x8 a = lds_frag_tr(Vt, LDT, 32 * pr, 32 * pr + 16, 16 * db, lane);
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) O[db][qb] = mfma16(a, P[pr][qb], O[db][qb]);
      }
    if (i + 1 < ntiles) {
      tile_r2l<D>(Kb[cur ^ 1], rk, tid);
      tile_r2l<D>(Vb[cur ^ 1], rv, tid);
      if (i + 2 < ntiles) issue_window(i + 2);
    }
    __syncthreads();
  }

  // ---- epilogue -------------------------------------------------------------------------------
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    float lwt = lw[qb] + __shfl_xor(lw[qb], 16, 64);
    lwt += __shfl_xor(lwt, 32, 64);
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

template <int D, int G>
int launch_out(const MP& p, hipStream_t st) {
  static bool configured = false;
  const size_t lds = OutSmem<D>::bytes;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)mfma_out_kernel<D, G>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("nha_prefill_fwd(mfma): cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((mfma_out_kernel<D, G>), dim3(p.NT, p.H * (p.NG / G)), dim3(256), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma output pass)");
  return NHA_OK;
}

template <int D>
int run_mfma(const MP& p, int phases, hipStream_t st) {
  if (phases != 2) {
    hipLaunchKernelGGL((mfma_state_kernel<D>), dim3(p.N * p.H, MS / 16), dim3(256), 0, st, p);
    NHA_CHECK_LAUNCH("nha_prefill_fwd(mfma state pass)");
  }
  if (phases != 1) {
    const int G = (p.NG % 4 == 0) ? 4 : (p.NG % 2 == 0) ? 2 : 1;
    if (G == 4) return launch_out<D, 4>(p, st);
    if (G == 2) return launch_out<D, 2>(p, st);
    return launch_out<D, 1>(p, st);
  }
  return NHA_OK;
}

static size_t aligned(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

bool prefill_mfma_supported(const NhaPrefillArgs* a) {
  return a->dtype == NHA_DTYPE_BF16 && a->K == a->V && (a->K == 64 || a->K == 128) && a->M == MS;
}

size_t prefill_mfma_scratch_bytes(const NhaPrefillArgs* a) {
  const size_t per = (size_t)a->NT * a->H;
  return aligned(per * MS * a->K * 2) + aligned(per * MS * a->V * 2) + aligned(per * BT * MS * 4);
}

int prefill_mfma_impl(const NhaPrefillArgs* a) {
  MP p;
  p.q_swa = (const bf16_t*)a->q_swa; p.k_swa = (const bf16_t*)a->k_swa;
  p.q_gsa = (const bf16_t*)a->q_gsa; p.k_gsa = (const bf16_t*)a->k_gsa;
  p.v = (const bf16_t*)a->v; p.s = (const bf16_t*)a->s; p.g = (const bf16_t*)a->g;
  p.o = (bf16_t*)a->o;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa;
  p.h0k = a->h0k; p.h0v = a->h0v; p.hkt = a->hkt; p.hvt = a->hvt;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices; p.coff = a->chunk_offsets;
  const size_t per = (size_t)a->NT * a->H;
  char* sc = (char*)a->scratch;
  p.hkT = (bf16_t*)sc;
  sc += aligned(per * MS * a->K * 2);
  p.hvc = (bf16_t*)sc;
  sc += aligned(per * MS * a->V * 2);
  p.gc = (float*)sc;
  p.T_tot = a->T_tot; p.N = a->N; p.NT = a->NT; p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H;
  p.wl = a->wl; p.shift = a->shift; p.scale = a->scale;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return run_mfma<64>(p, a->phases, st);
  return run_mfma<128>(p, a->phases, st);
}

}  // namespace nha
