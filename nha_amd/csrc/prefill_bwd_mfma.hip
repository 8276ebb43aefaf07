// Matrix-core kernels for the window branch of the NHA prefill backward on gfx950
// (bf16, K == V == D in {64,128,256}; the part nha_fla/ops/nha/chunk.py:499-511 hands to
// flash-attn's backward).  With the merged-softmax quantities of the whole op per (token, q-head)
//   lse = log(sum_m e^u + sum_j e^w),   delta = do . o,
// the window logits w[q][j] = scale q_swa_q . k_swa_j (j in [max(bos, q - wl), q]) give
//   pi = e^(w - lse),  dpi = do_q . v_j,  dw = pi (dpi - delta),
//   dq_swa_q = scale sum_j dw k_swa_j,   dk_swa_j = scale sum_q dw q_swa_q,   dv_j += sum_q pi do_q.
// Two kernels, each in the orientation whose accumulator layout feeds its next MFMA without moving
// data between lanes (v_mfma_f32_16x16x32_bf16: A[i][8(l/16)+e], B[8(l/16)+e][j], C[4(l/16)+r][l%16]):
//   bwd_dq_kernel   one workgroup per (64 queries, q-head); K/V tiles stream through LDS;
//                   S^T = K Q^T and dP^T = V dO^T put a query per lane, dQ^T += K^T dS^T
//   bwd_dkv_kernel  one workgroup per (64 keys, kv-head); Q/dO tiles of every q-head of the group
//                   stream through LDS; S = Q K^T and dP = dO V^T put a key per lane,
//                   dV^T += dO^T P and dK^T += Q^T dS
#include "common.h"

namespace nha {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define NHA_LDS __attribute__((address_space(3)))
typedef NHA_LDS bf16_t lbf16;
typedef NHA_LDS float lfloat;

constexpr int BT = 64;
constexpr float LOG2E = 1.4426950408889634f;

struct WP {
  const bf16_t *q, *k, *v, *dout;          // q_swa [T,HQ,D]; k_swa, v [T,H,D]; dout [T,HQ,D]
  const float *lse_swa, *lse_gsa, *delta;  // [T,HQ]
  const float* dvs;                        // [T,H,D] slot-branch part of dv
  bf16_t *dq, *dk, *dv;
  const int32_t *cu, *cidx;
  int HQ, H, NG, wl;
  float scale;
};

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ void lds_st16(lbf16* p, uint4 v) { *reinterpret_cast<NHA_LDS u32x4*>(p) = (u32x4){v.x, v.y, v.z, v.w}; }
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ bf16x8 pack8(f32x4 a, f32x4 b) {
  bf16x8 r;
  r[0] = (__bf16)a[0]; r[1] = (__bf16)a[1]; r[2] = (__bf16)a[2]; r[3] = (__bf16)a[3];
  r[4] = (__bf16)b[0]; r[5] = (__bf16)b[1]; r[6] = (__bf16)b[2]; r[7] = (__bf16)b[3];
  return r;
}
// 8 consecutive elements of row `row` of a row-major LDS tile, starting at `col`
__device__ __forceinline__ bf16x8 lds_frag(const lbf16* tile, int ld, int row, int col) {
  return *reinterpret_cast<const NHA_LDS bf16x8*>(tile + row * ld + col);
}
// transposed fragment: lane (c = l%16, kb = l/16) receives X[r0a + 4 kb + e][col0 + c], e = 0..3,
// and X[r0b + 4 kb + e][col0 + c] as elements 4..7
__device__ __forceinline__ bf16x8 lds_frag_tr(const lbf16* tile, int ld, int r0a, int r0b, int col0, int lane) {
  const int l16 = lane & 15, kb = lane >> 4;
  const lbf16* pa = tile + (r0a + 4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  const lbf16* pb = tile + (r0b + 4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  struct { s16x4 a, b; } t;
  t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
  t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pb);
  return __builtin_bit_cast(bf16x8, t);
}
// Query head of workgroup x in a launch whose rows hold one workgroup per query head.  Workgroups are dealt
// to the 8 XCDs in launch order, so x runs on XCD x % 8: the heads are numbered so that an XCD gets
// consecutive heads, and the query heads of one kv-head fetch its states and rows through one L2.
__device__ __forceinline__ int head_of_workgroup(int x, int HQ) { return (HQ & 7) == 0 ? (x & 7) * (HQ >> 3) + (x >> 3) : x; }
// (head, row of the launch) of a workgroup of the window kernels, grid (heads, chunks).  With 8 heads or a multiple
// the launch order already keeps a head on one XCD (head_of_workgroup).  With fewer -- the 340M layers have four -- the
// chunks of a head would alternate between XCDs (workgroup L runs on XCD L % 8 and L = row * heads + head), and the
// window rows that neighbouring chunks share would be fetched into two L2s, each holding twice the span of chunks:
// there XCD k takes the k-th eighth of the (head, row) sequence, consecutive rows of one head.
__device__ __forceinline__ void window_tile(int heads, int& head, int& row) {
  const int total = gridDim.x * gridDim.y;
  if ((heads & 7) == 0) {
    head = head_of_workgroup(blockIdx.x, heads);
    row = blockIdx.y;
  } else {
    // the first 8 * (total / 8) workgroups are dealt as said, the up to seven left over keep their place
    const int L = blockIdx.y * gridDim.x + blockIdx.x, per = total >> 3;
    const int v = L < 8 * per ? (L & 7) * per + (L >> 3) : L;
    head = v / (int)gridDim.y;
    row = v % (int)gridDim.y;
  }
}
__device__ __forceinline__ float logaddexp_f(float a, float b) {
  const float mx = fmaxf(a, b);
  return mx + logf(expf(a - mx) + expf(b - mx));
}

// rows [0, vhi) of a ROWS x D tile whose row r is global row grow0 + r of a [*, heads, D] tensor
template <int ROWS, int D>
struct Tile {
  static constexpr int NPC = ROWS * D / 8 / 256;
  uint4 r[NPC];
  __device__ __forceinline__ void load(const bf16_t* base, int64_t row_stride, int64_t grow0, int vhi, int tid) {
#pragma unroll
    for (int u = 0; u < NPC; ++u) {
      const int c = tid + 256 * u;
      const int row = c / (D / 8), col = (c % (D / 8)) * 8;
      uint4 x = make_uint4(0, 0, 0, 0);
      if (row < vhi) x = *reinterpret_cast<const uint4*>(base + (grow0 + row) * row_stride + col);
      r[u] = x;
    }
  }
  __device__ __forceinline__ void store(lbf16* lds, int tid) const {
#pragma unroll
    for (int u = 0; u < NPC; ++u) {
      const int c = tid + 256 * u;
      const int row = c / (D / 8), col = (c % (D / 8)) * 8;
      lds_st16(lds + row * (D + 16) + col, r[u]);
    }
  }
};

// ------------------------------------------------------------------------------------------
// dq_swa: grid (HQ, NT), 4 waves x 16 query rows
// ------------------------------------------------------------------------------------------
template <int D, int TK>
__global__ __launch_bounds__(256) void bwd_dq_kernel(const WP p) {
  constexpr int KS = D / 32, DB = D / 16, LDT = D + 16, NH = TK / 32, TILE = TK * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const tiles = (lbf16*)smem;   // K0, K1, V0, V1
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ;
  int hq, wrow;
  window_tile(p.HQ, hq, wrow);
  const int h = hq / p.NG;
  // last chunk first: the chunks at the start of a sequence see the fewest keys, and short
  // workgroups at the end of the launch leave the smallest tail
  const int chunk = gridDim.y - 1 - wrow;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  const int y = 16 * wave + l16;   // this lane's query, relative to the chunk
  const bool valid = y < rows;
  const int64_t tq = (int64_t)(c0 + (valid ? y : 0)) * HQ + hq;
  bf16x8 qf[KS], df[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (valid) {
      a = *reinterpret_cast<const uint4*>(p.q + tq * D + 32 * ks + 8 * kb);
      b = *reinterpret_cast<const uint4*>(p.dout + tq * D + 32 * ks + 8 * kb);
    }
    qf[ks] = __builtin_bit_cast(bf16x8, a);
    df[ks] = __builtin_bit_cast(bf16x8, b);
  }
  const float lse2 = valid ? logaddexp_f(p.lse_swa[tq], p.lse_gsa[tq]) * LOG2E : 0.f;
  const float dl = valid ? p.delta[tq] : 0.f;
  const float cs = p.scale * LOG2E;
  f32x4 dQ[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) dQ[db] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // key tile i covers keys [c0 + 64 - TK (i+1), c0 + 64 - TK i); boundaries are multiples of TK
  // away from bos, so no tile starts before its sequence
  int lowest = bos;
  if (p.wl >= 0 && c0 - p.wl > bos) lowest = c0 - p.wl;
  const int ntiles = (c0 + 64 - lowest + TK - 1) / TK;
  Tile<TK, D> rk, rv;
  auto issue = [&](int i) {
    const int64_t grow0 = (int64_t)c0 + 64 - TK * (i + 1);
    int vhi = eos - (int)grow0;
    vhi = vhi < 0 ? 0 : (vhi > TK ? TK : vhi);
    rk.load(p.k + (int64_t)h * D, (int64_t)H * D, grow0, vhi, tid);
    rv.load(p.v + (int64_t)h * D, (int64_t)H * D, grow0, vhi, tid);
  };
  issue(0);
  rk.store(tiles, tid);
  rv.store(tiles + 2 * TILE, tid);
  if (ntiles > 1) issue(1);
  lds_barrier();
  for (int i = 0; i < ntiles; ++i) {
    const int cur = i & 1;
    const lbf16* Kt = tiles + cur * TILE;
    const lbf16* Vt = tiles + (2 + cur) * TILE;
    const int xbase = 64 - TK * (i + 1);
    const bool edge = (xbase + TK - 1 > 0) || (p.wl >= 0 && p.wl < TK * (i + 1) - 1);
#pragma unroll
    for (int hf = 0; hf < NH; ++hf) {
      f32x4 S[2], dP[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        S[kk] = (f32x4){0.f, 0.f, 0.f, 0.f};
        dP[kk] = (f32x4){0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          S[kk] = mfma16(lds_frag(Kt, LDT, 32 * hf + 16 * kk + l16, 32 * ks + 8 * kb), qf[ks], S[kk]);
          dP[kk] = mfma16(lds_frag(Vt, LDT, 32 * hf + 16 * kk + l16, 32 * ks + 8 * kb), df[ks], dP[kk]);
        }
      }
      f32x4 dS[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int x = xbase + 32 * hf + 16 * kk + 4 * kb + r;
          const bool ok = !edge || ((x <= y) && (p.wl < 0 || x >= y - p.wl));
          const float pr = ok ? fexp2(S[kk][r] * cs - lse2) : 0.f;
          dS[kk][r] = pr * (dP[kk][r] - dl) * p.scale;
        }
      const bf16x8 dSb = pack8(dS[0], dS[1]);
      // dQ^T[d][q] += K^T[d][key] dS^T[key][q]
#pragma unroll
      for (int db = 0; db < DB; ++db) dQ[db] = mfma16(lds_frag_tr(Kt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane), dSb, dQ[db]);
    }
    if (i + 1 < ntiles) {
      rk.store(tiles + (cur ^ 1) * TILE, tid);
      rv.store(tiles + (2 + (cur ^ 1)) * TILE, tid);
      if (i + 2 < ntiles) issue(i + 2);
    }
    lds_barrier();
  }
  if (valid) {
    bf16_t* op = p.dq + tq * D + 4 * kb;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 pk;
#pragma unroll
      for (int r = 0; r < 4; ++r) pk[r] = (__bf16)dQ[db][r];
      *reinterpret_cast<bf16x4*>(op + 16 * db) = pk;
    }
  }
}

// ------------------------------------------------------------------------------------------
// dk_swa, dv: grid (H, NT), 4 waves x 16 keys.  MODE 0: both; 1: dk only; 2: dv only (D = 256
// runs 1 and 2 as two launches: both accumulators do not fit the register file)
// ------------------------------------------------------------------------------------------
template <int D, int TQ, int MODE>
__global__ __launch_bounds__(256) void bwd_dkv_kernel(const WP p) {
  constexpr int KS = D / 32, DB = D / 16, LDT = D + 16, NH = TQ / 32, TILE = TQ * LDT;
  constexpr bool DO_K = MODE != 2, DO_V = MODE != 1;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const tiles = (lbf16*)smem;                 // Q0, Q1, dO0, dO1
  lfloat* const lsb = (lfloat*)(tiles + 4 * TILE);   // [2][TQ] lse * log2(e)
  lfloat* const dlb = lsb + 2 * TQ;                  // [2][TQ] delta
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  int h, chunk;
  window_tile(H, h, chunk);
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int j0 = bos + it * BT;
  const int krows = (eos - j0) < BT ? (eos - j0) : BT;
  const int x = 16 * wave + l16;   // this lane's key, relative to j0
  const bool valid = x < krows;
  const int64_t jk = (int64_t)(j0 + (valid ? x : 0)) * H + h;
  bf16x8 kf[KS], vf[DO_K ? KS : 1];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (valid) {
      a = *reinterpret_cast<const uint4*>(p.k + jk * D + 32 * ks + 8 * kb);
      if (DO_K) b = *reinterpret_cast<const uint4*>(p.v + jk * D + 32 * ks + 8 * kb);
    }
    kf[ks] = __builtin_bit_cast(bf16x8, a);
    if (DO_K) vf[ks] = __builtin_bit_cast(bf16x8, b);
  }
  const float cs = p.scale * LOG2E;
  f32x4 dK[DO_K ? DB : 1], dV[DO_V ? DB : 1];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    if (DO_K) dK[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (DO_V) dV[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  // queries that see any of these keys: [j0, qend); tiles of TQ queries x the NG heads of the group
  int qend = eos;
  if (p.wl >= 0 && j0 + 64 + p.wl < eos) qend = j0 + 64 + p.wl;
  const int nqt = (qend - j0 + TQ - 1) / TQ;
  const int niter = nqt * NG;
  Tile<TQ, D> rq, ro;
  float rls = 0.f, rlg = 0.f, rd = 0.f;
  // iteration i = (q-head of the group, query tile), tiles innermost: the workgroup of the next
  // chunk (same XCD, started together) reads the same tile one iteration earlier, so the tile is
  // still in that XCD's L2; with the heads innermost the reuse distance was four iterations of
  // every resident workgroup, more than the L2 holds.
  auto issue = [&](int i) {
    const int qt = i % nqt, hq = h * NG + i / nqt;
    const int64_t grow0 = (int64_t)j0 + TQ * qt;
    int vhi = eos - (int)grow0;
    vhi = vhi < 0 ? 0 : (vhi > TQ ? TQ : vhi);
    rq.load(p.q + (int64_t)hq * D, (int64_t)HQ * D, grow0, vhi, tid);
    ro.load(p.dout + (int64_t)hq * D, (int64_t)HQ * D, grow0, vhi, tid);
    // only requested here: the merge of the two log-sum-exps waits until the values are staged, a
    // tile later (used at once, it stalled the first wave for a memory latency in every iteration
    // and the other waves behind it at the barrier)
    rls = rlg = rd = 0.f;
    if (tid < TQ && tid < vhi) {
      const int64_t tq = (grow0 + tid) * HQ + hq;
      rls = p.lse_swa[tq];
      rlg = p.lse_gsa[tq];
      rd = p.delta[tq];
    }
  };
  auto stage = [&](int buf) {
    rq.store(tiles + buf * TILE, tid);
    ro.store(tiles + (2 + buf) * TILE, tid);
    if (tid < TQ) {
      lsb[buf * TQ + tid] = logaddexp_f(rls, rlg) * LOG2E;
      dlb[buf * TQ + tid] = rd;
    }
  };
  issue(0);
  stage(0);
  if (niter > 1) issue(1);
  lds_barrier();
  for (int i = 0; i < niter; ++i) {
    const int cur = i & 1;
    const lbf16* Qt = tiles + cur * TILE;
    const lbf16* Ot = tiles + (2 + cur) * TILE;
    const lfloat* ls = lsb + cur * TQ;
    const lfloat* dl = dlb + cur * TQ;
    const int ybase = TQ * (i % nqt);   // first query of the tile, relative to j0
    const bool edge = (ybase < 63) || (p.wl >= 0 && ybase + TQ - 1 > p.wl) || (j0 + ybase + TQ > eos);
#pragma unroll
    for (int hf = 0; hf < NH; ++hf) {
      f32x4 S[2], dP[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        S[kk] = (f32x4){0.f, 0.f, 0.f, 0.f};
        dP[kk] = (f32x4){0.f, 0.f, 0.f, 0.f};
      }
      // the fragments of a 16-query block are requested together, then multiplied: one LDS
      // latency per block instead of one per MFMA
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        constexpr int KH = KS > 4 ? 4 : KS;   // fragments in flight per tensor
#pragma unroll
        for (int k0 = 0; k0 < KS; k0 += KH) {
          bf16x8 qa[KH], oa[DO_K ? KH : 1];
#pragma unroll
          for (int u = 0; u < KH; ++u) {
            qa[u] = lds_frag(Qt, LDT, 32 * hf + 16 * kk + l16, 32 * (k0 + u) + 8 * kb);
            if (DO_K) oa[u] = lds_frag(Ot, LDT, 32 * hf + 16 * kk + l16, 32 * (k0 + u) + 8 * kb);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int u = 0; u < KH; ++u) {
            S[kk] = mfma16(qa[u], kf[k0 + u], S[kk]);
            if (DO_K) dP[kk] = mfma16(oa[u], vf[k0 + u], dP[kk]);
          }
        }
      }
      f32x4 P[2], dS[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int yr0 = 32 * hf + 16 * kk + 4 * kb;   // first of this lane's 4 query rows in the tile
        const f32x4 l4 = *reinterpret_cast<const NHA_LDS f32x4*>(ls + yr0);
        const f32x4 d4 = *reinterpret_cast<const NHA_LDS f32x4*>(dl + yr0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int yy = ybase + yr0 + r;
          const bool ok = !edge || ((x <= yy) && (p.wl < 0 || x >= yy - p.wl) && (j0 + yy < eos));
          const float pr = ok ? fexp2(S[kk][r] * cs - l4[r]) : 0.f;
          P[kk][r] = pr;
          dS[kk][r] = pr * (dP[kk][r] - d4[r]) * p.scale;
        }
      }
      const bf16x8 Pb = pack8(P[0], P[1]);
      const bf16x8 dSb = pack8(dS[0], dS[1]);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        // dV^T[d][key] += dO^T[d][q] P[q][key];  dK^T[d][key] += Q^T[d][q] dS[q][key]
        if (DO_V) dV[db] = mfma16(lds_frag_tr(Ot, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane), Pb, dV[db]);
        if (DO_K) dK[db] = mfma16(lds_frag_tr(Qt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane), dSb, dK[db]);
      }
    }
    if (i + 1 < niter) {
      stage(cur ^ 1);
      if (i + 2 < niter) issue(i + 2);
    }
    lds_barrier();
  }
  if (valid) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int64_t off = jk * D + 16 * db + 4 * kb;
      bf16x4 pk;
      if (DO_K) {
#pragma unroll
        for (int r = 0; r < 4; ++r) pk[r] = (__bf16)dK[db][r];
        *reinterpret_cast<bf16x4*>(p.dk + off) = pk;
      }
      if (DO_V) {
        const float4 sv = *reinterpret_cast<const float4*>(p.dvs + off);
        pk[0] = (__bf16)(dV[db][0] + sv.x);
        pk[1] = (__bf16)(dV[db][1] + sv.y);
        pk[2] = (__bf16)(dV[db][2] + sv.z);
        pk[3] = (__bf16)(dV[db][3] + sv.w);
        *reinterpret_cast<bf16x4*>(p.dv + off) = pk;
      }
    }
  }
}


// ------------------------------------------------------------------------------------------
// Slot branch, products that do not involve the decay: per (chunk, q-head)
//   A[i][j] = q_gsa_i . k'_j      B[i][j] = do_i . v'_j          (rows i, j of the chunk; k', v' read at
//   U0[i][m] = q_gsa_i . hk0[:,m]  P0[i][m] = do_i . hv0[m,:]      the source token of row j)
// all of the form X Y^T with X in {q_gsa, do} (64 rows through LDS) and Y in {k', hk0^T, v', hv0}
// (64 rows as register fragments, 16 per wave).  grid (HQ, NT), 4 waves.
// ------------------------------------------------------------------------------------------
struct SP1 {
  const bf16_t *q, *dout, *kg, *v;   // q_gsa [T,HQ,D], dout [T,HQ,D], k_gsa [T,H,D], v [T,H,D]
  const bf16_t *hkb, *hvb;           // [NT][H][64][D] chunk-start states, hk transposed (high parts)
  const bf16_t *hkl, *hvl;           // their low parts
  bf16_t *ap, *bp;                   // [NT][HQ][64][64] bf16: every consumer takes them as matrix-core operands
  float *ust, *dpst;                 // [T][HQ][64]
  const bf16_t* o;                   // [T,HQ,D]
  float* delta;                      // [T][HQ]  do . o
  const int32_t *cu, *cidx;
  int HQ, H, NG, shift;
};

// ------------------------------------------------------------------------------------------
// Slot branch, products over the rows of a chunk (bf16 operands, fp32 accumulation).
//
// bwd_slot_state_kernel, grid (H, NT, 2 D / DW): per (chunk, kv-head), state and column range (z even: k-state with
// X = q_gsa, weights scale*du, matrix ck; z = 1: v-state with X = do, weights p, matrix cv), summed
// over the q-heads of the group:
//   N[x][m]  = sum_i X_i[x] w_i[m] e^(gc_i[m])        inhomogeneous term of the state-gradient recurrence
//   out[r][x] = sum_(i>=r) c[i][r] X_i[x]              intra-chunk part of dk' / dv'
// Both are X^T times a 64-row table, so they share the transposed X fragments (A operand); the
// tables are staged transposed ([column][row i], bf16) so that a B fragment is two 8-byte reads.
//
// bwd_slot_dq_kernel, grid (HQ, NT): per (chunk, q-head)
//   dq_gsa[i][d] = sum_m (scale du_i[m] e^(gc_i[m])) hk0[d][m] + sum_(j<=i) ck[i][j] k'_j[d]
// as dQ^T = hk0 W^T + K'^T C^T with the state and the k' rows as transposed A fragments.
// ------------------------------------------------------------------------------------------
constexpr int TLD = 72;   // bf16 row stride of the 64 x 64 tables in LDS

struct SP2 {
  const bf16_t *q, *dout, *kg, *s;   // q_gsa, dout [T,HQ,D]; k_gsa [T,H,D]
  const bf16_t* hkb;                 // [NT][H][64][D]
  const float *dus, *pp, *ck, *cv;   // [T][HQ][64] x2, [NT][HQ][64][64] x2
  const float* gc;                   // [T][H][64]
  float *ek, *ev;                    // [NT][H][D][64] x2
  float *dks, *dvs;                  // [T][H][D] x2 (source-token index)
  float* dsp;                        // [2 * slabs][T][H][64] inter-chunk part of ds per state and column range
  const bf16_t* v;                   // [T,H,D]
  bf16_t* dkg;                       // dk_gsa [T,H,D]
  int T_tot;
  bf16_t* dq;                        // dq_gsa [T,HQ,D]
  const int32_t *cu, *cidx;
  int HQ, H, NG, shift;
};

// B fragment from a transposed table tab[n][i] (row stride TLD): rows of the contraction
// i = 32 hf + 4 kb + e (e < 4) and 32 hf + 16 + 4 kb + (e - 4), column n
__device__ __forceinline__ bf16x8 table_frag(const lbf16* tab, int n, int hf, int kb) {
  struct { bf16x4 a, b; } t;
  t.a = *reinterpret_cast<const NHA_LDS bf16x4*>(tab + n * TLD + 32 * hf + 4 * kb);
  t.b = *reinterpret_cast<const NHA_LDS bf16x4*>(tab + n * TLD + 32 * hf + 16 + 4 * kb);
  return __builtin_bit_cast(bf16x8, t);
}

// x as a bf16 pair hi + lo (16 mantissa bits): the tables built from fp32 intermediates are kept
// this way and multiplied as hi*b + lo*b, so that their rounding stays below that of the bf16 inputs.
// Four consecutive elements at once: two 8-byte LDS writes (idx a multiple of 4)
__device__ __forceinline__ void split4_bf16(const float4 x, lbf16* hi, lbf16* lo, int idx) {
  const float v[4] = {x.x, x.y, x.z, x.w};
  bf16x4 h, l;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    h[e] = (__bf16)v[e];
    l[e] = (__bf16)(v[e] - (float)h[e]);
  }
  *reinterpret_cast<NHA_LDS bf16x4*>(hi + idx) = h;
  *reinterpret_cast<NHA_LDS bf16x4*>(lo + idx) = l;
}

// DW: the columns x a workgroup takes (blockIdx.z / 2 picks them); launched with DW = D
template <int D, int DW>
__global__ __launch_bounds__(256) void bwd_slot_state_kernel(const SP2 p) {
  constexpr int DB = DW / 16, LDT = DW + 16, TILE = BT * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const Xt = (lbf16*)smem;        // [64 rows i][DW]
  // the two tables lie as they are read from memory, row i by row i (8-byte LDS writes); the transposing LDS
  // read turns them into B operands (2-byte writes of the transposed tables cost four times the instructions)
  lbf16* const Wt = Xt + TILE;           // [64 i][TLD]  w_i[m] e^(gc_i[m]), high part
  lbf16* const Wl = Wt + BT * TLD;       //              low part
  lbf16* const Ct = Wl + BT * TLD;       // [64 i][TLD]  c[i][r], zero for i < r, high part
  lbf16* const Cl = Ct + BT * TLD;       //              low part
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  const int h = blockIdx.x, chunk = blockIdx.y;
  const bool isv = (blockIdx.z & 1) != 0;
  const int x0 = (blockIdx.z >> 1) * DW;   // this workgroup's columns
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const bf16_t* xsrc = isv ? p.dout : p.q;
  const float* wsrc = isv ? p.pp : p.dus;
  const float* csrc = isv ? p.cv : p.ck;
  f32x4 accN[DB], accO[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    accN[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    accO[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const int col = 16 * wave + l16;   // this lane's column: slot m of N, row r of out
  // The X tile and the tables of a q-head are requested together (coalesced 16-byte reads over c, all
  // issued before the first use); at head sizes up to 128 those of the next head are requested before the
  // products of this one, so that only the first head of a workgroup waits out a memory latency.
  constexpr int NS = BT * BT / 4 / 256;
  constexpr bool AHEAD = DW <= 128;
  Tile<BT, DW> rx;
  float4 wv[NS], cv[NS];
  auto load_head = [&](int hq) {
    rx.load(xsrc + (int64_t)hq * D + x0, (int64_t)HQ * D, c0, R, tid);
    const float* cp = csrc + ((int64_t)chunk * HQ + hq) * BT * BT;
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), i = e >> 6, c = e & 63;
      wv[u] = cv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < R) {
        wv[u] = *reinterpret_cast<const float4*>(wsrc + ((int64_t)(c0 + i) * HQ + hq) * BT + c);
        if (c <= i) cv[u] = *reinterpret_cast<const float4*>(cp + i * BT + c);
      }
    }
  };
  if (AHEAD) load_head(h * NG);
  // e^(gc) of this thread's elements: the same for every q-head of the group, read and formed once
  float4 eg[NS];
#pragma unroll
  for (int u = 0; u < NS; ++u) {
    const int e = 4 * (tid + 256 * u), i = e >> 6, c = e & 63;
    eg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < R) {
      const float4 g = *reinterpret_cast<const float4*>(p.gc + ((int64_t)(c0 + i) * H + h) * BT + c);
      eg[u] = make_float4(__expf(g.x), __expf(g.y), __expf(g.z), __expf(g.w));
    }
  }
  for (int a = 0; a < NG; ++a) {
    const int hq = h * NG + a;
    if (!AHEAD) load_head(hq);
    if (a > 0) lds_barrier();   // everyone is done with the previous head's tiles
    rx.store(Xt, tid);
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), i = e >> 6, c = e & 63;
      // rows i >= R were not read: wv, cv and eg are zero there
      split4_bf16(make_float4(wv[u].x * eg[u].x, wv[u].y * eg[u].y, wv[u].z * eg[u].z, wv[u].w * eg[u].w), Wt, Wl, i * TLD + c);
      split4_bf16(make_float4(c <= i ? cv[u].x : 0.f, c + 1 <= i ? cv[u].y : 0.f, c + 2 <= i ? cv[u].z : 0.f,
                              c + 3 <= i ? cv[u].w : 0.f), Ct, Cl, i * TLD + c);
    }
    lds_barrier();
    if (AHEAD && a + 1 < NG) load_head(hq + 1);
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const bf16x8 bw = lds_frag_tr(Wt, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 bwl = lds_frag_tr(Wl, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 bc = lds_frag_tr(Ct, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 bcl = lds_frag_tr(Cl, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x8 xa = lds_frag_tr(Xt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane);   // X^T[x][i]
        accN[db] = mfma16(xa, bw, mfma16(xa, bwl, accN[db]));
        accO[db] = mfma16(xa, bc, mfma16(xa, bcl, accO[db]));
      }
    }
  }
  // N[x = 16 db + 4 kb + r][m = col];  out^T[x][row = col]
  float* ep = (isv ? p.ev : p.ek) + (((int64_t)chunk * H + h) * D + x0) * BT;
  const int tl = it * BT + col - p.shift;
  const bool has = col < R && tl >= 0;
  float* op = (isv ? p.dvs : p.dks) + (((int64_t)bos + (has ? tl : 0)) * H + h) * D + x0;
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int r = 0; r < 4; ++r) ep[(16 * db + 4 * kb + r) * BT + col] = accN[db][r];
    if (has) *reinterpret_cast<float4*>(op + 16 * db + 4 * kb) = make_float4(accO[db][0], accO[db][1], accO[db][2], accO[db][3]);
  }
}

template <int D>
__global__ __launch_bounds__(256) void bwd_slot_dq_kernel(const SP2 p) {
  constexpr int DB = D / 16, LDT = D + 16, TILE = BT * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  // The two products run one after the other through the same LDS (a tile and one table as a high and a low
  // part: 36 KB, four workgroups per CU; with both sets resident, 72 KB, two); the operands of the second are
  // requested with those of the first and wait in registers.
  lbf16* const Ht = (lbf16*)smem;        // [64 m][D]  hk0^T
  lbf16* const Kt = Ht;                  // [64 j][D]  k' rows (second product)
  lbf16* const Wt = Ht + TILE;           // [64 i][TLD]  scale du_i[m] e^(gc_i[m]), high part
  lbf16* const Wl = Wt + BT * TLD;       //              low part
  lbf16* const Ct = Wt;                  // [64 i][TLD]  ck[i][j], zero for j > i, high part (second product)
  lbf16* const Cl = Wl;                  //              low part
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ;
  const int hq = head_of_workgroup(blockIdx.x, p.HQ), h = hq / p.NG, chunk = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  Tile<BT, D> rk;
  constexpr int NS = BT * BT / 4 / 256;
  float4 cv[NS];
  {
    Tile<BT, D> rh;
    rh.load(p.hkb + ((int64_t)chunk * H + h) * BT * D, D, 0, BT, tid);
    // k' row j is the k_gsa row of source token c0 + j - shift: rows before the sequence are zero
    int vlo = p.shift - it * BT;
    vlo = vlo < 0 ? 0 : vlo;
#pragma unroll
    for (int u = 0; u < Tile<BT, D>::NPC; ++u) {
      const int c = tid + 256 * u;
      const int row = c / (D / 8), cc = (c % (D / 8)) * 8;
      uint4 x = make_uint4(0, 0, 0, 0);
      if (row >= vlo && row < R) x = *reinterpret_cast<const uint4*>(p.kg + (((int64_t)c0 + row - p.shift) * H + h) * D + cc);
      rk.r[u] = x;
    }
    // the tables are requested before the tiles are stored: one memory latency for both
    const float* cp = p.ck + ((int64_t)chunk * HQ + hq) * BT * BT;
    float4 wv[NS], gv[NS];
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), i = e >> 6, c = e & 63;
      wv[u] = gv[u] = cv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < R) {
        wv[u] = *reinterpret_cast<const float4*>(p.dus + ((int64_t)(c0 + i) * HQ + hq) * BT + c);
        gv[u] = *reinterpret_cast<const float4*>(p.gc + ((int64_t)(c0 + i) * H + h) * BT + c);
        if (c <= i) cv[u] = *reinterpret_cast<const float4*>(cp + i * BT + c);
      }
    }
    rh.store(Ht, tid);
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), i = e >> 6, c = e & 63;
      float4 w;
      w.x = i < R ? wv[u].x * __expf(gv[u].x) : 0.f;
      w.y = i < R ? wv[u].y * __expf(gv[u].y) : 0.f;
      w.z = i < R ? wv[u].z * __expf(gv[u].z) : 0.f;
      w.w = i < R ? wv[u].w * __expf(gv[u].w) : 0.f;
      split4_bf16(w, Wt, Wl, i * TLD + c);
    }
  }
  lds_barrier();
  const int i = 16 * wave + l16;   // this lane's row of the chunk
  f32x4 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const bf16x8 bw = table_frag(Wt, i, hf, kb), bwl = table_frag(Wl, i, hf, kb);   // contraction over m
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x8 ha = lds_frag_tr(Ht, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane);   // hk0[d][m]
      acc[db] = mfma16(ha, bw, mfma16(ha, bwl, acc[db]));
    }
  }
  lds_barrier();   // everyone has read the first product's operands
  rk.store(Kt, tid);
#pragma unroll
  for (int u = 0; u < NS; ++u) {
    const int e = 4 * (tid + 256 * u), i2 = e >> 6, c = e & 63;
    float4 cc;
    cc.x = c <= i2 ? cv[u].x : 0.f;
    cc.y = c + 1 <= i2 ? cv[u].y : 0.f;
    cc.z = c + 2 <= i2 ? cv[u].z : 0.f;
    cc.w = c + 3 <= i2 ? cv[u].w : 0.f;
    split4_bf16(cc, Ct, Cl, i2 * TLD + c);
  }
  lds_barrier();
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    if (hf == 1 && wave < 2) continue;   // ck[i][j] is zero for j > i: rows below 32 have no second half
    const bf16x8 bc = table_frag(Ct, i, hf, kb), bcl = table_frag(Cl, i, hf, kb);   // contraction over j
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x8 ka = lds_frag_tr(Kt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane);   // k'_j[d]
      acc[db] = mfma16(ka, bc, mfma16(ka, bcl, acc[db]));
    }
  }
  if (i < R) {
    bf16_t* op = p.dq + ((int64_t)(c0 + i) * HQ + hq) * D + 4 * kb;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 pk;
#pragma unroll
      for (int r = 0; r < 4; ++r) pk[r] = (__bf16)acc[db][r];
      *reinterpret_cast<bf16x4*>(op + 16 * db) = pk;
    }
  }
}

// bwd_slot_inter_kernel, grid (H, NT, 2 D / DW): the parts that involve E_c, the state gradient carried
// into the END of chunk c (z even: k-state, rows k', output dk_gsa; z odd: v-state, rows v', output
// dvs), with dec_r[m] = e^(gl[m] - gc_r[m]):
//   out[r][x] = intra part + sum_m (s_r[m] dec_r[m]) E[x][m]         as out^T = E sE^T
//   dsp[r][m] = dec_r[m] sum_x y_r[x] E[x][m]                         as Y E
// A workgroup takes DW of the D columns x (z / 2 picks them): at head size 256 two workgroups of half the
// columns fit a CU where one of all columns does not, and each writes its own partial of dsp (one slab per
// state and column range; the gate kernel adds the slabs).
template <int D, int DW>
__global__ __launch_bounds__(256) void bwd_slot_inter_kernel(const SP2 p) {
  constexpr int DB = DW / 16, LDT = DW + 16, TILE = BT * LDT, ELD = BT + 8, NH = D / DW;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const Yt = (lbf16*)smem;        // [64 rows r][DW]  k' / v'
  lbf16* const Et = Yt + TILE;           // [DW x][ELD]      E[x][m], high part
  lbf16* const El = Et + DW * ELD;       //                  low part
  lbf16* const St = El + DW * ELD;        // [64 r][TLD]      s_r[m] dec_r[m], high part
  lbf16* const Sl = St + BT * TLD;       //                  low part
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H;
  const int h = blockIdx.x, chunk = blockIdx.y;
  const bool isv = (blockIdx.z & 1) != 0;
  const int xh = blockIdx.z >> 1, x0 = xh * DW;   // this workgroup's columns
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const bf16_t* ysrc = isv ? p.v : p.kg;
  int vlo = p.shift - it * BT;
  vlo = vlo < 0 ? 0 : vlo;
  Tile<BT, DW> ry;
#pragma unroll
  for (int u = 0; u < Tile<BT, DW>::NPC; ++u) {
    const int c = tid + 256 * u;
    const int row = c / (DW / 8), cc = (c % (DW / 8)) * 8;
    uint4 x = make_uint4(0, 0, 0, 0);
    if (row >= vlo && row < R) x = *reinterpret_cast<const uint4*>(ysrc + (((int64_t)c0 + row - p.shift) * H + h) * D + x0 + cc);
    ry.r[u] = x;
  }
  const float* ep = (isv ? p.ev : p.ek) + (((int64_t)chunk * H + h) * D + x0) * BT;
  const float* gcb = p.gc + ((int64_t)c0 * H + h) * BT;
  {
    // all global loads of a batch are issued before the first conversion waits for one; the first batch
    // of E and the gate rows are requested before the Y tile is stored
    constexpr int NE = DW * BT / 4 / 256, EB = NE < 8 ? NE : 8;
    const float4* ep4 = reinterpret_cast<const float4*>(ep);
    constexpr int NS = BT * BT / 4 / 256;
    float4 gl[NS], gr[NS];
    uint2 sr[NS];
#pragma unroll
    for (int b0 = 0; b0 < NE; b0 += EB) {
      float4 buf[EB];
#pragma unroll
      for (int u = 0; u < EB; ++u) buf[u] = ep4[tid + 256 * (b0 + u)];
      if (b0 == 0) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const int e = 4 * (tid + 256 * u), r = e >> 6, m = e & 63;
          gl[u] = gr[u] = make_float4(0.f, 0.f, 0.f, 0.f);
          sr[u] = make_uint2(0, 0);
          if (r >= vlo && r < R) {
            sr[u] = *reinterpret_cast<const uint2*>(p.s + (((int64_t)c0 + r - p.shift) * H + h) * BT + m);
            gl[u] = *reinterpret_cast<const float4*>(gcb + (int64_t)(R - 1) * H * BT + m);
            gr[u] = *reinterpret_cast<const float4*>(gcb + (int64_t)r * H * BT + m);
          }
        }
        ry.store(Yt, tid);
      }
#pragma unroll
      for (int u = 0; u < EB; ++u) {
        const int e = 4 * (tid + 256 * (b0 + u));
        split4_bf16(buf[u], Et, El, (e >> 6) * ELD + (e & 63));
      }
    }
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), r = e >> 6, m = e & 63;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r >= vlo && r < R) {
        v.x = __uint_as_float(sr[u].x << 16) * __expf(gl[u].x - gr[u].x);
        v.y = __uint_as_float(sr[u].x & 0xffff0000u) * __expf(gl[u].y - gr[u].y);
        v.z = __uint_as_float(sr[u].y << 16) * __expf(gl[u].z - gr[u].z);
        v.w = __uint_as_float(sr[u].y & 0xffff0000u) * __expf(gl[u].w - gr[u].w);
      }
      split4_bf16(v, St, Sl, r * TLD + m);
    }
  }
  lds_barrier();
  const int col = 16 * wave + l16;
  // the gate rows of the last products' decay, requested before the products
  const float glast = gcb[(int64_t)(R - 1) * H * BT + col];
  float grow[4][4];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 16 * rb + 4 * kb + q;
      grow[rb][q] = r < R ? gcb[(int64_t)r * H * BT + col] : 0.f;
    }
  // the partial sums the first products are added to: requested before the products where the registers
  // allow (head sizes up to 128)
  const bool has = col >= vlo && col < R;
  const int64_t oi = (((int64_t)c0 + col - p.shift) * H + h) * D + x0;
  const float* const part = isv ? p.dvs : p.dks;
  constexpr bool EARLY = DW <= 128;
  float4 pve[EARLY ? DB : 1];
  if (EARLY && has) {
#pragma unroll
    for (int db = 0; db < DB; ++db) pve[EARLY ? db : 0] = *reinterpret_cast<const float4*>(part + oi + 16 * db + 4 * kb);
  }
  // out^T[x][r = col] = sum_m E[x][m] sE[r][m]: A = E rows (plain), B = sE rows (plain), contraction m in 2 steps
  f32x4 accO[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) accO[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const bf16x8 bs = lds_frag(St, TLD, col, 32 * ks + 8 * kb), bsl = lds_frag(Sl, TLD, col, 32 * ks + 8 * kb);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x8 eh = lds_frag(Et, ELD, 16 * db + l16, 32 * ks + 8 * kb);
      accO[db] = mfma16(eh, bs, mfma16(eh, bsl, mfma16(lds_frag(El, ELD, 16 * db + l16, 32 * ks + 8 * kb), bs, accO[db])));
    }
  }
  if (has) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const float4 pv = EARLY ? pve[EARLY ? db : 0] : *reinterpret_cast<const float4*>(part + oi + 16 * db + 4 * kb);
      const float o0 = accO[db][0] + pv.x, o1 = accO[db][1] + pv.y, o2 = accO[db][2] + pv.z, o3 = accO[db][3] + pv.w;
      if (isv) {
        *reinterpret_cast<float4*>(p.dvs + oi + 16 * db + 4 * kb) = make_float4(o0, o1, o2, o3);
      } else {
        bf16x4 pk;
        pk[0] = (__bf16)o0; pk[1] = (__bf16)o1; pk[2] = (__bf16)o2; pk[3] = (__bf16)o3;
        *reinterpret_cast<bf16x4*>(p.dkg + oi + 16 * db + 4 * kb) = pk;
      }
    }
  }
  // dsp[r][m = col] = dec_r[m] sum_x y_r[x] E[x][m]: A = y rows (two 8-byte reads, contraction index
  // permuted like the transposing read), B = E via the transposing read
#pragma unroll
  for (int rb = 0; rb < 4; ++rb) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int xs = 0; xs < DW / 32; ++xs) {
      struct { bf16x4 a, b; } t;
      t.a = *reinterpret_cast<const NHA_LDS bf16x4*>(Yt + (16 * rb + l16) * LDT + 32 * xs + 4 * kb);
      t.b = *reinterpret_cast<const NHA_LDS bf16x4*>(Yt + (16 * rb + l16) * LDT + 32 * xs + 16 + 4 * kb);
      const bf16x8 ya = __builtin_bit_cast(bf16x8, t);
      acc = mfma16(ya, lds_frag_tr(Et, ELD, 32 * xs, 32 * xs + 16, 16 * wave, lane),
                   mfma16(ya, lds_frag_tr(El, ELD, 32 * xs, 32 * xs + 16, 16 * wave, lane), acc));
    }
    // C[r = 16 rb + 4 kb + q][m = col]
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 16 * rb + 4 * kb + q;
      if (r < R) {
        const float dec = __expf(glast - grow[rb][q]);
        p.dsp[(((int64_t)((isv ? NH : 0) + xh) * p.T_tot + c0 + r) * H + h) * BT + col] = acc[q] * dec;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Slot branch, the intra-chunk terms that couple rows through the decay e^(gc_i[m] - gc_j[m]), j <= i.
// With a reference point per 32-row half of the chunk (ref_0 = 0, ref_1 = gc_31) the decay splits
// into e^(gc_i - ref) <= 1 for the later row and e^(ref - gc_j) >= 1 for the earlier one, ref taken
// at the start of j's half, and the terms become plain products of 64 x 64 tables
//   X^(b) = scale du o e^(gc - ref_b), Xp^(b) = p o e^(gc - ref_b) (rows i), Y = s o e^(ref - gc) (rows j)
// as long as no slot decays by more than e^-70 within a half (bf16 and fp32 share the exponent
// range); chunks beyond that are flagged by the state export and take the fp32 VALU kernels.
//
// bwd_slot_q_kernel, grid (HQ, NT): u = scale (E o q.hk0 + sum_b e^(gc - ref_b) o (A_masked Y)_b),
//   dp likewise with do.hv0 and B; then p, du and the per-token vectors scale*du, p, du*u + p*dp,
//   element-wise in the accumulators.
// bwd_slot_intra_kernel, grid (H, NT): ck = X Y^T, cv = Xp Y^T (i >= r) per q-head, and
//   ds_intra[r][m] = e^(ref - gc_r[m]) sum_a sum_(i>=r) (A[i][r] X_i[m] + B[i][r] Xp_i[m]),
//   X and ref of r's half.
// ------------------------------------------------------------------------------------------
struct SP3 {
  const bf16_t* s;                                 // [T,H,64]
  const bf16_t *ap, *bp;                           // see bwd_slot_products
  const float *ust, *dpst, *gc, *delta;
  const float *lse_swa, *lse_gsa, *dlse_gsa;
  float *dus, *pp, *xg;                            // [T][HQ][64]
  float *ck, *cv;                                  // [NT][HQ][64][64]
  float* dsi;                                      // [T][H][64]
  const int* big;                                  // [NT][H]
  const int32_t *cu, *cidx;
  int HQ, H, NG, shift;
  float scale;
};

// gate cumsum of the chunk's row r and the reference of its half (0 for rows 0..31, gc_31 after)
__device__ __forceinline__ float gc_at(const SP3& p, int c0, int h, int r, int m) {
  return p.gc[((int64_t)(c0 + r) * p.H + h) * BT + m];
}
__device__ __forceinline__ float ref_of(const SP3& p, int c0, int h, int r, int m) {
  return r < 32 ? 0.f : gc_at(p, c0, h, 31, m);
}

// The decay-scaled tables enter the gate gradient through a difference of nearly equal sums (dg is
// a telescoping sum), so they are bf16 pairs (split4_bf16) and their products hi*hi + hi*lo + lo*hi.
// rows of Y = s_j[m] e^(ref - gc_j[m]) (zero for rows without a source token)
struct StageY {
  // 16-byte reads, all issued before the first conversion waits for one
  static constexpr int NS = BT * BT / 4 / 256;
  float4 gj[NS], gr[NS];
  uint2 sr[NS];
  __device__ __forceinline__ void load(const SP3& p, int c0, int h, int R, int vlo, int tid) {
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), j = e >> 6, m = e & 63;
      gj[u] = gr[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      sr[u] = make_uint2(0, 0);
      if (j >= vlo && j < R) {
        sr[u] = *reinterpret_cast<const uint2*>(p.s + (((int64_t)c0 + j - p.shift) * p.H + h) * BT + m);
        gj[u] = *reinterpret_cast<const float4*>(p.gc + ((int64_t)(c0 + j) * p.H + h) * BT + m);
        if (j >= 32) gr[u] = *reinterpret_cast<const float4*>(p.gc + ((int64_t)(c0 + 31) * p.H + h) * BT + m);
      }
    }
  }
  __device__ __forceinline__ void store(lbf16* Yh, lbf16* Yl, int R, int vlo, int tid) const {
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), j = e >> 6, m = e & 63;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (j >= vlo && j < R) {
        v.x = __uint_as_float(sr[u].x << 16) * __expf(gr[u].x - gj[u].x);
        v.y = __uint_as_float(sr[u].x & 0xffff0000u) * __expf(gr[u].y - gj[u].y);
        v.z = __uint_as_float(sr[u].y << 16) * __expf(gr[u].z - gj[u].z);
        v.w = __uint_as_float(sr[u].y & 0xffff0000u) * __expf(gr[u].w - gj[u].w);
      }
      split4_bf16(v, Yh, Yl, j * TLD + m);
    }
  }
};
__device__ __forceinline__ void stage_y(lbf16* Yh, lbf16* Yl, const SP3& p, int c0, int h, int R, int vlo, int tid) {
  StageY y;
  y.load(p, c0, h, R, vlo, tid);
  y.store(Yh, Yl, R, vlo, tid);
}

// per-row operands of the per-token stage for the rows 16 blk + 4 kb + q of a lane (slot m): requested
// together, ahead of the stage, so that no block of rows waits out a memory latency of its own
struct RowOps {
  float gi[4][4], ls[4][4], lg[4][4], g31;
  __device__ __forceinline__ void load(const SP3& p, int c0, int R, int h, int hq, int m, int kb) {
    g31 = R > 32 ? p.gc[((int64_t)(c0 + 31) * p.H + h) * BT + m] : 0.f;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = 16 * blk + 4 * kb + q;
        gi[blk][q] = ls[blk][q] = lg[blk][q] = 0.f;
        if (i < R) {
          const int64_t tq = (int64_t)(c0 + i) * p.HQ + hq;
          gi[blk][q] = p.gc[((int64_t)(c0 + i) * p.H + h) * BT + m];
          ls[blk][q] = p.lse_swa[tq];
          lg[blk][q] = p.lse_gsa[tq];
        }
      }
  }
};

// u, dp, p and du of the chunk's rows from the tables in LDS (A, B masked to j <= i; Y high and low
// parts); the lane's values of q.hk0 and do.hv0 come either from the products kernel's accumulators
// (cU, cP: rows 16 blk + 4 kb + q, slot 16 wave + l16, the same mapping as here) or from scratch.
template <bool FROM_REGS>
__device__ __forceinline__ void slot_q_rows(const SP3& p, const lbf16* At, const lbf16* Bt, const lbf16* Yh, const lbf16* Yl,
                                            int c0, int R, int h, int hq, int wave, int lane, const f32x4* cU,
                                            const f32x4* cP, const lfloat* dl, const RowOps& ro) {
  const int l16 = lane & 15, kb = lane >> 4;
  const int HQ = p.HQ;
  const int m = 16 * wave + l16;
  const float g31 = ro.g31;
#pragma unroll
  for (int blk = 0; blk < 4; ++blk) {
    f32x4 cu_[2], cd_[2];   // one accumulator per half of the contraction (= per reference)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const bf16x8 yh = lds_frag_tr(Yh, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);   // Y[j][m]
      const bf16x8 yl = lds_frag_tr(Yl, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 af = table_frag(At, 16 * blk + l16, hf, kb), bf = table_frag(Bt, 16 * blk + l16, hf, kb);
      cu_[hf] = mfma16(af, yh, mfma16(af, yl, (f32x4){0.f, 0.f, 0.f, 0.f}));
      cd_[hf] = mfma16(bf, yh, mfma16(bf, yl, (f32x4){0.f, 0.f, 0.f, 0.f}));
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i = 16 * blk + 4 * kb + q;
      if (i >= R) continue;
      const int64_t tq = (int64_t)(c0 + i) * HQ + hq;
      const float gi = ro.gi[blk][q];
      const float e0 = __expf(gi);
      const float e1 = blk >= 2 ? __expf(gi - g31) : 0.f;   // rows before the second half see none of it
      const float au = p.scale * (e0 * ((FROM_REGS ? cU[blk][q] : p.ust[tq * BT + m]) + cu_[0][q]) + e1 * cu_[1][q]);
      const float ad = e0 * ((FROM_REGS ? cP[blk][q] : p.dpst[tq * BT + m]) + cd_[0][q]) + e1 * cd_[1][q];
      const float ls = ro.ls[blk][q], lg = ro.lg[blk][q];
      const float lt = logaddexp_f(ls, lg);
      const float pm = __expf(au - lt);
      float du = pm * (ad - (FROM_REGS ? dl[i] : p.delta[tq]));
      if (p.dlse_gsa) du += p.dlse_gsa[tq] * __expf(au - lg);
      p.dus[tq * BT + m] = p.scale * du;
      p.pp[tq * BT + m] = pm;
      p.xg[tq * BT + m] = du * au + pm * ad;
    }
  }
}

__global__ __launch_bounds__(256) void bwd_slot_q_kernel(const SP3 p) {
  __shared__ __align__(16) bf16_t sm[4 * BT * TLD];
  lbf16* const At = (lbf16*)sm;          // [64 i][TLD]  A[i][j], zero for j > i
  lbf16* const Bt = At + BT * TLD;       // [64 i][TLD]  B[i][j], zero for j > i
  lbf16* const Yh = Bt + BT * TLD;       // [64 j][TLD]  Y, high and low parts
  lbf16* const Yl = Yh + BT * TLD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ;
  const int hq = head_of_workgroup(blockIdx.x, p.HQ), h = hq / p.NG, chunk = blockIdx.y;
  if (p.big[(int64_t)chunk * H + h]) return;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  int vlo = p.shift - it * BT;
  vlo = vlo < 0 ? 0 : vlo;
  const bf16_t* ap = p.ap + ((int64_t)chunk * HQ + hq) * BT * BT;
  const bf16_t* bp = p.bp + ((int64_t)chunk * HQ + hq) * BT * BT;
  {
    constexpr int NS = BT * BT / 4 / 256;
    uint2 av[NS], bv[NS];
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), i = e >> 6, j = e & 63;
      av[u] = bv[u] = make_uint2(0, 0);
      if (j <= i && i < R) {
        av[u] = *reinterpret_cast<const uint2*>(ap + e);
        bv[u] = *reinterpret_cast<const uint2*>(bp + e);
      }
    }
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int e = 4 * (tid + 256 * u), i = e >> 6, j = e & 63;
      const uint16_t a4[4] = {(uint16_t)av[u].x, (uint16_t)(av[u].x >> 16), (uint16_t)av[u].y, (uint16_t)(av[u].y >> 16)};
      const uint16_t b4[4] = {(uint16_t)bv[u].x, (uint16_t)(bv[u].x >> 16), (uint16_t)bv[u].y, (uint16_t)(bv[u].y >> 16)};
      uint16_t pa[4], pb[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool in = j + q <= i && i < R;
        pa[q] = in ? a4[q] : (uint16_t)0;
        pb[q] = in ? b4[q] : (uint16_t)0;
      }
      typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
      *reinterpret_cast<NHA_LDS u32x2_t*>(At + i * TLD + j) = (u32x2_t){pa[0] | ((uint32_t)pa[1] << 16), pa[2] | ((uint32_t)pa[3] << 16)};
      *reinterpret_cast<NHA_LDS u32x2_t*>(Bt + i * TLD + j) = (u32x2_t){pb[0] | ((uint32_t)pb[1] << 16), pb[2] | ((uint32_t)pb[3] << 16)};
    }
  }
  RowOps rops;
  rops.load(p, c0, R, h, hq, 16 * wave + l16, kb);
  stage_y(Yh, Yl, p, c0, h, R, vlo, tid);
  lds_barrier();
  slot_q_rows<false>(p, At, Bt, Yh, Yl, c0, R, h, hq, wave, lane, nullptr, nullptr, nullptr, rops);
}

// FUSE: the per-token stage of bwd_slot_q_kernel runs in the same workgroup (same grid, same
// lane-to-element mapping), so q.hk0 and do.hv0 never leave the registers; chunks flagged for the
// fp32 fallback, and every chunk without FUSE, get them in scratch instead.
template <int D, bool FUSE>
__global__ __launch_bounds__(256) void bwd_slot_products_kernel(const SP1 p, const SP3 pq) {
  constexpr int KS = D / 32, LDT = D + 16, TILE = BT * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const Qt = (lbf16*)smem;
  lbf16* const Ot = Qt + TILE;
  lbf16* const At = Ot + TILE;           // FUSE only: the four tables of the per-token stage
  lbf16* const Bt = At + BT * TLD;
  lbf16* const Yh = Bt + BT * TLD;
  lbf16* const Yl = Yh + BT * TLD;
  lfloat* const dlt = (lfloat*)(Yl + BT * TLD);   // [64] delta of the chunk's rows
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ;
  const int hq = head_of_workgroup(blockIdx.x, p.HQ), h = hq / p.NG;
  const int chunk = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  // Every global read of the workgroup is requested ahead of the stage that consumes it, in the order
  // of use, so that the stages do not each wait out a memory latency: q / do tiles, the Y rows, the o
  // rows of delta and the rows of the Y table here; the per-row operands of the per-token stage before
  // the products.
  const bool fused = FUSE && !pq.big[(int64_t)chunk * H + h];
  int vlo = pq.shift - it * BT;
  vlo = vlo < 0 ? 0 : vlo;
  // (at head size 256 the Y rows alone are 192 registers: there the tiles are stored before the Y rows
  // are requested and the o rows are requested last)
  constexpr bool EARLY = D <= 128;
  Tile<BT, D> rq, ro;
  rq.load(p.q + (int64_t)hq * D, (int64_t)HQ * D, c0, R, tid);
  ro.load(p.dout + (int64_t)hq * D, (int64_t)HQ * D, c0, R, tid);
  if (!EARLY) {
    rq.store(Qt, tid);
    ro.store(Ot, tid);
  }
  // this lane's Y rows: row j = 16 wave + l16 of the chunk (source token c0 + j - shift), slot m = j
  const int j = 16 * wave + l16;
  const int tl = it * BT + j - p.shift;
  const bool has = j < R && tl >= 0;
  const int64_t sj = ((int64_t)bos + (has ? tl : 0)) * H + h;
  const int64_t cg = ((int64_t)chunk * H + h) * BT + j;
  bf16x8 yk[KS], yv[KS], yhk[KS], yhv[KS], yhkl[KS], yhvl[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (has) {
      a = *reinterpret_cast<const uint4*>(p.kg + sj * D + 32 * ks + 8 * kb);
      b = *reinterpret_cast<const uint4*>(p.v + sj * D + 32 * ks + 8 * kb);
    }
    yk[ks] = __builtin_bit_cast(bf16x8, a);
    yv[ks] = __builtin_bit_cast(bf16x8, b);
    yhk[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p.hkb + cg * D + 32 * ks + 8 * kb));
    yhv[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p.hvb + cg * D + 32 * ks + 8 * kb));
    yhkl[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p.hkl + cg * D + 32 * ks + 8 * kb));
    yhvl[ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p.hvl + cg * D + 32 * ks + 8 * kb));
  }
  // o rows of delta: row i = 16 wave + l16, the four lanes sharing l16 split the columns
  uint4 ov[KS];
  auto load_o = [&]() {
    const int i = 16 * wave + l16;
    const bf16_t* orow = p.o + ((int64_t)(c0 + (i < R ? i : 0)) * HQ + hq) * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      ov[ks] = make_uint4(0, 0, 0, 0);
      if (i < R) ov[ks] = *reinterpret_cast<const uint4*>(orow + 32 * ks + 8 * kb);
    }
  };
  if (EARLY) load_o();
  StageY sy;
  if (fused) sy.load(pq, c0, h, R, vlo, tid);
  if (EARLY) {
    rq.store(Qt, tid);
    ro.store(Ot, tid);
  } else {
    load_o();
  }
  lds_barrier();
  {
    // delta_i = do_i . o_i
    const int i = 16 * wave + l16;
    float acc = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 o8 = __builtin_bit_cast(bf16x8, ov[ks]);
      const bf16x8 dv = lds_frag(Ot, LDT, i, 32 * ks + 8 * kb);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += (float)o8[e] * (float)dv[e];
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (kb == 0 && i < R) p.delta[(int64_t)(c0 + i) * HQ + hq] = acc;
    if (FUSE && kb == 0) dlt[i] = acc;
  }
  bf16_t* ap = p.ap + ((int64_t)chunk * HQ + hq) * BT * BT;
  bf16_t* bp = p.bp + ((int64_t)chunk * HQ + hq) * BT * BT;
  RowOps rops;
  if (fused) rops.load(pq, c0, R, h, hq, 16 * wave + l16, kb);
  f32x4 cUr[FUSE ? 4 : 1], cPr[FUSE ? 4 : 1];
#pragma unroll
  for (int blk = 0; blk < 4; ++blk) {
    f32x4 cA = {0.f, 0.f, 0.f, 0.f}, cB = cA, cU = cA, cP = cA;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 xq = lds_frag(Qt, LDT, 16 * blk + l16, 32 * ks + 8 * kb);
      const bf16x8 xo = lds_frag(Ot, LDT, 16 * blk + l16, 32 * ks + 8 * kb);
      cA = mfma16(xq, yk[ks], cA);
      cU = mfma16(xq, yhk[ks], mfma16(xq, yhkl[ks], cU));
      cB = mfma16(xo, yv[ks], cB);
      cP = mfma16(xo, yhv[ks], mfma16(xo, yhvl[ks], cP));
    }
    if (FUSE) {
      cUr[blk] = cU;
      cPr[blk] = cP;
    }
    // C[i = 16 blk + 4 kb + r][j = 16 wave + l16]
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * blk + 4 * kb + r;
      if (fused) {   // the tables go to LDS; their global copies are written from there in 16-byte pieces below
        const bool in = j <= i && i < R;
        At[i * TLD + j] = f32_to_bf16(in ? cA[r] : 0.f);
        Bt[i * TLD + j] = f32_to_bf16(in ? cB[r] : 0.f);
      } else {
        ap[i * BT + j] = f32_to_bf16(cA[r]);
        bp[i * BT + j] = f32_to_bf16(cB[r]);
      }
      if (!fused && i < R) {
        const int64_t tq = ((int64_t)(c0 + i) * HQ + hq) * BT + j;
        p.ust[tq] = cU[r];
        p.dpst[tq] = cP[r];
      }
    }
  }
  if constexpr (FUSE) {
    if (!fused) return;   // uniform over the workgroup
    sy.store(Yh, Yl, R, vlo, tid);
    lds_barrier();
    // global copies of the two score tables for the intra-chunk kernel (masked like the LDS tables: above the
    // diagonal and past the last row they are zero, and every reader masks those elements itself)
#pragma unroll
    for (int u = 0; u < BT * BT / 8 / 256; ++u) {
      const int e = tid + 256 * u, i = e >> 3, c8 = (e & 7) * 8;
      const nha_u32x4 ta = *reinterpret_cast<const NHA_LDS nha_u32x4*>(At + i * TLD + c8);
      const nha_u32x4 tb = *reinterpret_cast<const NHA_LDS nha_u32x4*>(Bt + i * TLD + c8);
      *reinterpret_cast<nha_u32x4*>(ap + i * BT + c8) = ta;
      *reinterpret_cast<nha_u32x4*>(bp + i * BT + c8) = tb;
    }
    slot_q_rows<true>(pq, At, Bt, Yh, Yl, c0, R, h, hq, wave, lane, cUr, cPr, dlt, rops);
  }
}


__global__ __launch_bounds__(256) void bwd_slot_intra_kernel(const SP3 p) {
  extern __shared__ __align__(16) unsigned char smem[];
  // tables [64 rows][TLD]; X0 = scale du_i[m] e^(gc_i[m]), X1 = scale du_i[m] e^(gc_i[m] - gc_31[m])
  // (rows >= 32 only: 32-row tables whose pointers are set back by 32 rows, so that row i is indexed as in the
  // others), P0 / P1 the same with p; each as a high and a low part.  Y is the same for every q-head and each
  // lane needs the same four fragments of it throughout: they are read into registers once and the transposed
  // A / B tables of the heads then use Y's place.  Eight tables = 72 KB: two workgroups per CU.
  lbf16* const T0 = (lbf16*)smem;
  lbf16* const X0h = T0, * const X0l = T0 + BT * TLD, * const P0h = T0 + 2 * BT * TLD, * const P0l = T0 + 3 * BT * TLD;
  lbf16* const Yh = T0 + 4 * BT * TLD;   // [64 r][TLD]
  lbf16* const Yl = T0 + 5 * BT * TLD;
  lbf16* const AT = Yh;                  // [64 i][TLD]  A[i][r], zero for i < r; read with the transposing LDS read
  lbf16* const BT_ = Yl;                 // [64 i][TLD]  B[i][r]
  lbf16* const X1h = T0 + (6 * BT - 32) * TLD, * const X1l = T0 + 6 * BT * TLD;
  lbf16* const P1h = T0 + (7 * BT - 32) * TLD, * const P1l = T0 + 7 * BT * TLD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  const int h = blockIdx.x, chunk = blockIdx.y;
  if (p.big[(int64_t)chunk * H + h]) return;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  int vlo = p.shift - it * BT;
  vlo = vlo < 0 ? 0 : vlo;
  StageY sy;
  sy.load(p, c0, h, R, vlo, tid);
  const int col = 16 * wave + l16;
  // columns r of ck / cv in the first half take the tables with ref 0, the others ref gc_31
  const lbf16* const Xch = wave < 2 ? X0h : X1h;
  const lbf16* const Xcl = wave < 2 ? X0l : X1l;
  const lbf16* const Pch = wave < 2 ? P0h : P1h;
  const lbf16* const Pcl = wave < 2 ? P0l : P1l;
  f32x4 accS[4];
#pragma unroll
  for (int rb = 0; rb < 4; ++rb) accS[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
  // two 4-element groups per thread at a time: their twelve 16-byte reads are in flight together.  The
  // first pair of a q-head is requested before the products of the head before it, the second pair
  // before the first is converted: a head waits out one partly hidden memory latency instead of two.
  struct Pair {
    float4 du[2], pv[2];
    uint2 av[2], bv[2];   // four bf16 each
  };
  // e^(gc_i) and e^(gc_i - gc_31) (rows of the second half) of this thread's sixteen elements: the same for every
  // q-head of the group, read and formed once
  float4 e0v[4], e1v[2];   // groups 2 and 3 of a thread are the rows >= 32
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int e = 4 * (tid + 256 * u), i = e >> 6, c = e & 63;
    e0v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (u >= 2) e1v[u - 2] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < R) {
      const float4 g = *reinterpret_cast<const float4*>(p.gc + ((int64_t)(c0 + i) * H + h) * BT + c);
      e0v[u] = make_float4(__expf(g.x), __expf(g.y), __expf(g.z), __expf(g.w));
      if (u >= 2) {
        const float4 r = *reinterpret_cast<const float4*>(p.gc + ((int64_t)(c0 + 31) * H + h) * BT + c);
        e1v[u - 2] = make_float4(__expf(g.x - r.x), __expf(g.y - r.y), __expf(g.z - r.z), __expf(g.w - r.w));
      }
    }
  }
  auto load_pair = [&](Pair& t, int hq, int u0) {
    const bf16_t* ap = p.ap + ((int64_t)chunk * HQ + hq) * BT * BT;
    const bf16_t* bp = p.bp + ((int64_t)chunk * HQ + hq) * BT * BT;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int e = 4 * (tid + 256 * (u0 + u)), i = e >> 6, c = e & 63;
      t.du[u] = t.pv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      t.av[u] = t.bv[u] = make_uint2(0, 0);
      if (i < R) {
        t.du[u] = *reinterpret_cast<const float4*>(p.dus + ((int64_t)(c0 + i) * HQ + hq) * BT + c);
        t.pv[u] = *reinterpret_cast<const float4*>(p.pp + ((int64_t)(c0 + i) * HQ + hq) * BT + c);
        if (c <= i) {
          t.av[u] = *reinterpret_cast<const uint2*>(ap + e);
          t.bv[u] = *reinterpret_cast<const uint2*>(bp + e);
        }
      }
    }
  };
  auto store_pair = [&](const Pair& t, int u0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int e = 4 * (tid + 256 * (u0 + u)), i = e >> 6, c = e & 63;
      const bool second = u0 >= 2;   // rows >= 32: the only ones the ref-gc_31 tables hold
      const float4 ev0 = e0v[u0 + u], ev1 = second ? e1v[u0 + u - 2] : make_float4(0.f, 0.f, 0.f, 0.f);
      const float e0q[4] = {ev0.x, ev0.y, ev0.z, ev0.w}, e1q[4] = {ev1.x, ev1.y, ev1.z, ev1.w};
      const float d4[4] = {t.du[u].x, t.du[u].y, t.du[u].z, t.du[u].w}, q4[4] = {t.pv[u].x, t.pv[u].y, t.pv[u].z, t.pv[u].w};
      {
        // elements c + q > i (and rows i >= R, which were not read) are zero
        typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
        const int d = i < R ? i - c : -1;
        const uint32_t m0 = (d >= 0 ? 0xffffu : 0u) | (d >= 1 ? 0xffff0000u : 0u);
        const uint32_t m1 = (d >= 2 ? 0xffffu : 0u) | (d >= 3 ? 0xffff0000u : 0u);
        *reinterpret_cast<NHA_LDS u32x2_t*>(AT + i * TLD + c) = (u32x2_t){t.av[u].x & m0, t.av[u].y & m1};
        *reinterpret_cast<NHA_LDS u32x2_t*>(BT_ + i * TLD + c) = (u32x2_t){t.bv[u].x & m0, t.bv[u].y & m1};
      }
      float x0[4], x1[4], p0[4], p1[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float e0 = e0q[q], e1 = e1q[q];
        x0[q] = d4[q] * e0;
        p0[q] = q4[q] * e0;
        x1[q] = d4[q] * e1;
        p1[q] = q4[q] * e1;
      }
      split4_bf16(make_float4(x0[0], x0[1], x0[2], x0[3]), X0h, X0l, i * TLD + c);
      split4_bf16(make_float4(p0[0], p0[1], p0[2], p0[3]), P0h, P0l, i * TLD + c);
      if (second) {
        split4_bf16(make_float4(x1[0], x1[1], x1[2], x1[3]), X1h, X1l, i * TLD + c);
        split4_bf16(make_float4(p1[0], p1[1], p1[2], p1[3]), P1h, P1l, i * TLD + c);
      }
    }
  };
  static_assert(BT * BT / 4 / 256 == 4, "two pairs of element groups per thread");
  Pair t0, t1;
  load_pair(t0, h * NG, 0);
  sy.store(Yh, Yl, R, vlo, tid);
  lds_barrier();
  bf16x8 yfh[2], yfl[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    yfh[ks] = lds_frag(Yh, TLD, col, 32 * ks + 8 * kb);
    yfl[ks] = lds_frag(Yl, TLD, col, 32 * ks + 8 * kb);
  }
  for (int a = 0; a < NG; ++a) {
    const int hq = h * NG + a;
    load_pair(t1, hq, 2);
    lds_barrier();   // the Y fragments are read (first head) / the head before is done with the tables
    store_pair(t0, 0);
    store_pair(t1, 2);
    lds_barrier();
    if (a + 1 < NG) load_pair(t0, hq + 1, 0);
    // ck[i][r = col] = sum_m X[i][m] Y[r][m], cv with Xp
    float* ckp = p.ck + ((int64_t)chunk * HQ + hq) * BT * BT;
    float* cvp = p.cv + ((int64_t)chunk * HQ + hq) * BT * BT;
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
      if (blk < wave) continue;   // rows above this wave's columns: nothing to store (and no X1 / P1 rows below 32)
      f32x4 c1 = {0.f, 0.f, 0.f, 0.f}, c2 = c1;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 yh = yfh[ks], yl = yfl[ks];
        const bf16x8 xh = lds_frag(Xch, TLD, 16 * blk + l16, 32 * ks + 8 * kb);
        const bf16x8 ph = lds_frag(Pch, TLD, 16 * blk + l16, 32 * ks + 8 * kb);
        c1 = mfma16(xh, yh, mfma16(xh, yl, mfma16(lds_frag(Xcl, TLD, 16 * blk + l16, 32 * ks + 8 * kb), yh, c1)));
        c2 = mfma16(ph, yh, mfma16(ph, yl, mfma16(lds_frag(Pcl, TLD, 16 * blk + l16, 32 * ks + 8 * kb), yh, c2)));
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = 16 * blk + 4 * kb + q;
        if (i >= col && i < R) {
          ckp[i * BT + col] = c1[q];
          cvp[i * BT + col] = c2[q];
        }
      }
    }
    // ds[r][m = col] += sum_i A[i][r] X[i][m] + B[i][r] Xp[i][m]   (rows r < 32: ref 0, else ref gc_31)
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const bf16x8 x0h = lds_frag_tr(X0h, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 x0l = lds_frag_tr(X0l, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 p0h = lds_frag_tr(P0h, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
      const bf16x8 p0l = lds_frag_tr(P0l, TLD, 32 * hf, 32 * hf + 16, 16 * wave, lane);
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const bf16x8 af = lds_frag_tr(AT, TLD, 32 * hf, 32 * hf + 16, 16 * rb, lane);
        const bf16x8 bf = lds_frag_tr(BT_, TLD, 32 * hf, 32 * hf + 16, 16 * rb, lane);
        accS[rb] = mfma16(af, x0h, mfma16(af, x0l, accS[rb]));
        accS[rb] = mfma16(bf, p0h, mfma16(bf, p0l, accS[rb]));
      }
    }
    {
      // rows r >= 32 only meet rows i >= 32: the second half of the contraction
      const bf16x8 x1h = lds_frag_tr(X1h, TLD, 32, 48, 16 * wave, lane), x1l = lds_frag_tr(X1l, TLD, 32, 48, 16 * wave, lane);
      const bf16x8 p1h = lds_frag_tr(P1h, TLD, 32, 48, 16 * wave, lane), p1l = lds_frag_tr(P1l, TLD, 32, 48, 16 * wave, lane);
#pragma unroll
      for (int rb = 2; rb < 4; ++rb) {
        const bf16x8 af = lds_frag_tr(AT, TLD, 32, 48, 16 * rb, lane), bf = lds_frag_tr(BT_, TLD, 32, 48, 16 * rb, lane);
        accS[rb] = mfma16(af, x1h, mfma16(af, x1l, accS[rb]));
        accS[rb] = mfma16(bf, p1h, mfma16(bf, p1l, accS[rb]));
      }
    }
  }
#pragma unroll
  for (int rb = 0; rb < 4; ++rb)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 16 * rb + 4 * kb + q;
      if (r < R) {
        const int64_t idx = ((int64_t)(c0 + r) * H + h) * BT + col;
        p.dsi[idx] = accS[rb][q] * __expf(ref_of(p, c0, h, r, col) - p.gc[idx]);
      }
    }
}

template <int D, int TK>
int launch_dq(const WP& p, int NT, hipStream_t st) {
  const size_t lds = (size_t)4 * TK * (D + 16) * 2;
  static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)bwd_dq_kernel<D, TK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((bwd_dq_kernel<D, TK>), dim3(p.HQ, NT), dim3(256), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(window dq)");
  return NHA_OK;
}

template <int D, int TQ, int MODE>
int launch_dkv(const WP& p, int NT, hipStream_t st) {
  const size_t lds = (size_t)4 * TQ * (D + 16) * 2 + 4 * TQ * 4;
  static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)bwd_dkv_kernel<D, TQ, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((bwd_dkv_kernel<D, TQ, MODE>), dim3(p.H, NT), dim3(256), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(window dk, dv)");
  return NHA_OK;
}

WP make_wp(const NhaPrefillBwdArgs* a, const float* delta, const float* dvs) {
  WP p;
  p.q = (const bf16_t*)a->q_swa; p.k = (const bf16_t*)a->k_swa; p.v = (const bf16_t*)a->v;
  p.dout = (const bf16_t*)a->dout;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa; p.delta = delta; p.dvs = dvs;
  p.dq = (bf16_t*)a->dq_swa; p.dk = (bf16_t*)a->dk_swa; p.dv = (bf16_t*)a->dv;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.wl = a->wl; p.scale = a->scale;
  return p;
}

}  // namespace

bool bwd_window_mfma_supported(const NhaPrefillBwdArgs* a) {
  return a->dtype == NHA_DTYPE_BF16 && a->K == a->V && (a->K == 64 || a->K == 128 || a->K == 256) &&
         a->dlse_swa == nullptr && a->NT <= 65535;
}

int bwd_window_mfma_dq(const NhaPrefillBwdArgs* a, const float* delta, void* ld) {
  if (bwd_ring_supported(a)) return bwd_ring_dq(a, delta, (float2*)ld);
  const WP p = make_wp(a, delta, nullptr);
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return launch_dq<64, 64>(p, a->NT, st);
  if (a->K == 128) return launch_dq<128, 64>(p, a->NT, st);
  return launch_dq<256, 32>(p, a->NT, st);
}

int bwd_window_mfma_dkv(const NhaPrefillBwdArgs* a, const float* delta, const float* dvs, const void* ld) {
  if (bwd_ring_supported(a)) return bwd_ring_dkv(a, (const float2*)ld, dvs);
  const WP p = make_wp(a, delta, dvs);
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return launch_dkv<64, 64, 0>(p, a->NT, st);
  if (a->K == 128) return launch_dkv<128, 64, 0>(p, a->NT, st);
  int rc = launch_dkv<256, 32, 1>(p, a->NT, st);
  if (rc != NHA_OK) return rc;
  return launch_dkv<256, 32, 2>(p, a->NT, st);
}

template <int D, bool FUSE>
static int launch_slot_products(const SP1& p, const SP3& pq, int NT, hipStream_t st) {
  const size_t lds = (size_t)2 * BT * (D + 16) * 2 + (FUSE ? (size_t)4 * BT * TLD * 2 + BT * 4 : 0);
  static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)bwd_slot_products_kernel<D, FUSE>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((bwd_slot_products_kernel<D, FUSE>), dim3(p.HQ, NT), dim3(256), lds, st, p, pq);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(slot products)");
  return NHA_OK;
}

static SP3 make_sp3(const NhaPrefillBwdArgs* a, const int* big, const bf16_t* ap, const bf16_t* bp, const float* ust,
                    const float* dpst, const float* gc, const float* delta, float* dus, float* pp, float* xg, float* ck,
                    float* cv, float* dsi) {
  SP3 p;
  p.s = (const bf16_t*)a->s;
  p.ap = ap; p.bp = bp; p.ust = ust; p.dpst = dpst; p.gc = gc; p.delta = delta;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa; p.dlse_gsa = a->dlse_gsa;
  p.dus = dus; p.pp = pp; p.xg = xg; p.ck = ck; p.cv = cv; p.dsi = dsi; p.big = big;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.shift = a->shift; p.scale = a->scale;
  return p;
}

// With `big` (the decay flags) and head dims up to 128 the per-token stage is fused in and
// bwd_slot_products_fuses_q() tells the caller to skip bwd_slot_products3(which = 0).
bool bwd_slot_products_fuses_q(const NhaPrefillBwdArgs* a) { return a->K <= 128; }

int bwd_slot_products(const NhaPrefillBwdArgs* a, const void* hkb, const void* hvb, const void* hkl, const void* hvl, bf16_t* ap,
                      bf16_t* bp, float* ust, float* dpst, float* delta, const int* big, const float* gc, float* dus, float* pp,
                      float* xg) {
  SP1 p;
  p.q = (const bf16_t*)a->q_gsa; p.dout = (const bf16_t*)a->dout; p.kg = (const bf16_t*)a->k_gsa; p.v = (const bf16_t*)a->v;
  p.hkb = (const bf16_t*)hkb; p.hvb = (const bf16_t*)hvb;
  p.hkl = (const bf16_t*)hkl; p.hvl = (const bf16_t*)hvl;
  p.ap = ap; p.bp = bp; p.ust = ust; p.dpst = dpst;
  p.o = (const bf16_t*)a->o; p.delta = delta;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.shift = a->shift;
  const SP3 pq = make_sp3(a, big, ap, bp, ust, dpst, gc, delta, dus, pp, xg, nullptr, nullptr, nullptr);
  hipStream_t st = (hipStream_t)a->stream;
  const bool fuse = big != nullptr && bwd_slot_products_fuses_q(a);
  if (a->K == 64) return fuse ? launch_slot_products<64, true>(p, pq, a->NT, st) : launch_slot_products<64, false>(p, pq, a->NT, st);
  if (a->K == 128) return fuse ? launch_slot_products<128, true>(p, pq, a->NT, st) : launch_slot_products<128, false>(p, pq, a->NT, st);
  return launch_slot_products<256, false>(p, pq, a->NT, st);
}

template <int D>
static int launch_slot_stage2(const SP2& p, int NT, int which, hipStream_t st) {
  // (the state kernel takes all columns in one workgroup: split in two at head size 256 it stages its tables twice
  // and was measured slower, 110 against 103 us)
  const size_t lds_s = (size_t)BT * (D + 16) * 2 + (size_t)4 * BT * TLD * 2;
  const size_t lds_q = (size_t)BT * (D + 16) * 2 + (size_t)2 * BT * TLD * 2;
  constexpr int DWI = D > 128 ? 128 : D;   // columns per workgroup of the inter kernel
  const size_t lds_i = (size_t)BT * (DWI + 16) * 2 + (size_t)2 * DWI * (BT + 8) * 2 + (size_t)2 * BT * TLD * 2;
  static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
  if (!configured) {
    hipError_t e1 = hipFuncSetAttribute((const void*)bwd_slot_state_kernel<D, D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_s);
    hipError_t e2 = hipFuncSetAttribute((const void*)bwd_slot_dq_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_q);
    hipError_t e3 = hipFuncSetAttribute((const void*)bwd_slot_inter_kernel<D, DWI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_i);
    if (e1 == hipSuccess) e1 = e3;
    if (e1 != hipSuccess || e2 != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve LDS: %s", hipGetErrorString(e1 != hipSuccess ? e1 : e2));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  if (which == 1) hipLaunchKernelGGL((bwd_slot_state_kernel<D, D>), dim3(p.H, NT, 2), dim3(256), lds_s, st, p);
  else if (which == 2) hipLaunchKernelGGL((bwd_slot_inter_kernel<D, DWI>), dim3(p.H, NT, 2 * (D / DWI)), dim3(256), lds_i, st, p);
  else hipLaunchKernelGGL((bwd_slot_dq_kernel<D>), dim3(p.HQ, NT), dim3(256), lds_q, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(slot products, second stage)");
  return NHA_OK;
}

// which = 0: dq_gsa (bwd_slot_dq_kernel); 1: N_c and the intra-chunk parts of dk' / dv'
// (bwd_slot_state_kernel); 2: the parts that involve the scanned E_c (bwd_slot_inter_kernel).
// Same shapes as bwd_slot_products.
// partial-ds slabs per state that bwd_slot_inter_kernel writes: one per column range of a workgroup
int bwd_slot_inter_slabs(const NhaPrefillBwdArgs* a) { return a->K > 128 ? a->K / 128 : 1; }

int bwd_slot_products2(const NhaPrefillBwdArgs* a, int which, const void* hkb, const float* dus, const float* pp,
                       const float* ck, const float* cv, const float* gc, float* ek, float* ev, float* dks, float* dvs,
                       float* dsp) {
  SP2 p;
  p.q = (const bf16_t*)a->q_gsa; p.dout = (const bf16_t*)a->dout; p.kg = (const bf16_t*)a->k_gsa; p.s = (const bf16_t*)a->s;
  p.hkb = (const bf16_t*)hkb;
  p.dus = dus; p.pp = pp; p.ck = ck; p.cv = cv; p.gc = gc;
  p.ek = ek; p.ev = ev; p.dks = dks; p.dvs = dvs; p.dsp = dsp;
  p.v = (const bf16_t*)a->v; p.dkg = (bf16_t*)a->dk_gsa; p.T_tot = a->T_tot;
  p.dq = (bf16_t*)a->dq_gsa;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.shift = a->shift;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return launch_slot_stage2<64>(p, a->NT, which, st);
  if (a->K == 128) return launch_slot_stage2<128>(p, a->NT, which, st);
  return launch_slot_stage2<256>(p, a->NT, which, st);
}

// which = 0: bwd_slot_q_kernel (per-token vectors); 1: bwd_slot_intra_kernel (ck, cv, intra part of
// ds).  Chunks flagged in `big` are left to the fp32 VALU kernels.
int bwd_slot_products3(const NhaPrefillBwdArgs* a, int which, const int* big, const bf16_t* ap, const bf16_t* bp, const float* ust,
                       const float* dpst, const float* gc, const float* delta, float* dus, float* pp, float* xg, float* ck,
                       float* cv, float* dsi) {
  const SP3 p = make_sp3(a, big, ap, bp, ust, dpst, gc, delta, dus, pp, xg, ck, cv, dsi);
  hipStream_t st = (hipStream_t)a->stream;
  if (which == 0) hipLaunchKernelGGL(bwd_slot_q_kernel, dim3(a->HQ, a->NT), dim3(256), 0, st, p);
  else {
    const size_t lds = (size_t)8 * BT * TLD * 2;
    static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
    if (!configured) {
      hipError_t e = hipFuncSetAttribute((const void*)bwd_slot_intra_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) {
        set_error("nha_prefill_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        return NHA_ERR_LAUNCH;
      }
      configured = true;
    }
    hipLaunchKernelGGL(bwd_slot_intra_kernel, dim3(a->H, a->NT), dim3(256), lds, st, p);
  }
  NHA_CHECK_LAUNCH("nha_prefill_bwd(slot products, intra-chunk)");
  return NHA_OK;
}

}  // namespace nha
