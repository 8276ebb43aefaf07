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
  const int hq = blockIdx.x, h = hq / p.NG;
  const int chunk = blockIdx.y;
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
  const int h = blockIdx.x, chunk = blockIdx.y;
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
  float rl = 0.f, rd = 0.f;
  auto issue = [&](int i) {
    const int qt = i / NG, hq = h * NG + i % NG;
    const int64_t grow0 = (int64_t)j0 + TQ * qt;
    int vhi = eos - (int)grow0;
    vhi = vhi < 0 ? 0 : (vhi > TQ ? TQ : vhi);
    rq.load(p.q + (int64_t)hq * D, (int64_t)HQ * D, grow0, vhi, tid);
    ro.load(p.dout + (int64_t)hq * D, (int64_t)HQ * D, grow0, vhi, tid);
    rl = 0.f;
    rd = 0.f;
    if (tid < TQ && tid < vhi) {
      const int64_t tq = (grow0 + tid) * HQ + hq;
      rl = logaddexp_f(p.lse_swa[tq], p.lse_gsa[tq]) * LOG2E;
      rd = p.delta[tq];
    }
  };
  auto stage = [&](int buf) {
    rq.store(tiles + buf * TILE, tid);
    ro.store(tiles + (2 + buf) * TILE, tid);
    if (tid < TQ) {
      lsb[buf * TQ + tid] = rl;
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
    const int ybase = TQ * (i / NG);   // first query of the tile, relative to j0
    const bool edge = (ybase < 63) || (p.wl >= 0 && ybase + TQ - 1 > p.wl) || (j0 + ybase + TQ > eos);
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
          S[kk] = mfma16(lds_frag(Qt, LDT, 32 * hf + 16 * kk + l16, 32 * ks + 8 * kb), kf[ks], S[kk]);
          if (DO_K) dP[kk] = mfma16(lds_frag(Ot, LDT, 32 * hf + 16 * kk + l16, 32 * ks + 8 * kb), vf[ks], dP[kk]);
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
  const bf16_t *hkb, *hvb;           // [NT][H][64][D] chunk-start states, hk transposed
  float *ap, *bp;                    // [NT][HQ][64][64]
  float *ust, *dpst;                 // [T][HQ][64]
  const int32_t *cu, *cidx;
  int HQ, H, NG, shift;
};

template <int D>
__global__ __launch_bounds__(256) void bwd_slot_products_kernel(const SP1 p) {
  constexpr int KS = D / 32, LDT = D + 16, TILE = BT * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const Qt = (lbf16*)smem;
  lbf16* const Ot = Qt + TILE;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ;
  const int hq = blockIdx.x, h = hq / p.NG;
  const int chunk = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  {
    Tile<BT, D> rq, ro;
    rq.load(p.q + (int64_t)hq * D, (int64_t)HQ * D, c0, R, tid);
    ro.load(p.dout + (int64_t)hq * D, (int64_t)HQ * D, c0, R, tid);
    rq.store(Qt, tid);
    ro.store(Ot, tid);
  }
  // this lane's Y rows: row j = 16 wave + l16 of the chunk (source token c0 + j - shift), slot m = j
  const int j = 16 * wave + l16;
  const int tl = it * BT + j - p.shift;
  const bool has = j < R && tl >= 0;
  const int64_t sj = ((int64_t)bos + (has ? tl : 0)) * H + h;
  const int64_t cg = ((int64_t)chunk * H + h) * BT + j;
  bf16x8 yk[KS], yv[KS], yhk[KS], yhv[KS];
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
  }
  lds_barrier();
  float* ap = p.ap + ((int64_t)chunk * HQ + hq) * BT * BT;
  float* bp = p.bp + ((int64_t)chunk * HQ + hq) * BT * BT;
#pragma unroll
  for (int blk = 0; blk < 4; ++blk) {
    f32x4 cA = {0.f, 0.f, 0.f, 0.f}, cB = cA, cU = cA, cP = cA;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 xq = lds_frag(Qt, LDT, 16 * blk + l16, 32 * ks + 8 * kb);
      const bf16x8 xo = lds_frag(Ot, LDT, 16 * blk + l16, 32 * ks + 8 * kb);
      cA = mfma16(xq, yk[ks], cA);
      cU = mfma16(xq, yhk[ks], cU);
      cB = mfma16(xo, yv[ks], cB);
      cP = mfma16(xo, yhv[ks], cP);
    }
    // C[i = 16 blk + 4 kb + r][j = 16 wave + l16]
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = 16 * blk + 4 * kb + r;
      ap[i * BT + j] = cA[r];
      bp[i * BT + j] = cB[r];
      if (i < R) {
        const int64_t tq = ((int64_t)(c0 + i) * HQ + hq) * BT + j;
        p.ust[tq] = cU[r];
        p.dpst[tq] = cP[r];
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Slot branch, products over the rows of a chunk (bf16 operands, fp32 accumulation).
//
// bwd_slot_state_kernel, grid (H, NT, 2): per (chunk, kv-head) and state (z = 0: k-state with
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
  float* dsp;                        // [2][T][H][64] inter-chunk part of ds per state
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

template <int D>
__global__ __launch_bounds__(256) void bwd_slot_state_kernel(const SP2 p) {
  constexpr int DB = D / 16, LDT = D + 16, TILE = BT * LDT;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const Xt = (lbf16*)smem;        // [64 rows i][D]
  lbf16* const Wt = Xt + TILE;           // [64 m][TLD]  (w_i[m] e^(gc_i[m]))^T
  lbf16* const Ct = Wt + BT * TLD;       // [64 r][TLD]  c[i][r]^T, zero for i < r
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  const int h = blockIdx.x, chunk = blockIdx.y;
  const bool isv = blockIdx.z != 0;
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
  for (int a = 0; a < NG; ++a) {
    const int hq = h * NG + a;
    if (a > 0) lds_barrier();   // everyone is done with the previous head's tiles
    {
      Tile<BT, D> rx;
      rx.load(xsrc + (int64_t)hq * D, (int64_t)HQ * D, c0, R, tid);
      rx.store(Xt, tid);
    }
    const float* cp = csrc + ((int64_t)chunk * HQ + hq) * BT * BT;
    for (int e = tid; e < BT * BT; e += 256) {
      const int i = e >> 6, c = e & 63;   // coalesced reads over c, transposed writes
      float w = 0.f, cc = 0.f;
      if (i < R) {
        w = wsrc[((int64_t)(c0 + i) * HQ + hq) * BT + c] * __expf(p.gc[((int64_t)(c0 + i) * H + h) * BT + c]);
        if (c <= i) cc = cp[i * BT + c];
      }
      Wt[c * TLD + i] = f32_to_bf16(w);
      Ct[c * TLD + i] = f32_to_bf16(cc);
    }
    lds_barrier();
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const bf16x8 bw = table_frag(Wt, col, hf, kb);
      const bf16x8 bc = table_frag(Ct, col, hf, kb);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16x8 xa = lds_frag_tr(Xt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane);   // X^T[x][i]
        accN[db] = mfma16(xa, bw, accN[db]);
        accO[db] = mfma16(xa, bc, accO[db]);
      }
    }
  }
  // N[x = 16 db + 4 kb + r][m = col];  out^T[x][row = col]
  float* ep = (isv ? p.ev : p.ek) + ((int64_t)chunk * H + h) * D * BT;
  const int tl = it * BT + col - p.shift;
  const bool has = col < R && tl >= 0;
  float* op = (isv ? p.dvs : p.dks) + (((int64_t)bos + (has ? tl : 0)) * H + h) * D;
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
  lbf16* const Ht = (lbf16*)smem;        // [64 m][D]  hk0^T
  lbf16* const Kt = Ht + TILE;           // [64 j][D]  k' rows
  lbf16* const Wt = Kt + TILE;           // [64 i][TLD]  scale du_i[m] e^(gc_i[m])
  lbf16* const Ct = Wt + BT * TLD;       // [64 i][TLD]  ck[i][j], zero for j > i
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ;
  const int hq = blockIdx.x, h = hq / p.NG, chunk = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  {
    Tile<BT, D> rh, rk;
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
    rh.store(Ht, tid);
    rk.store(Kt, tid);
  }
  const float* cp = p.ck + ((int64_t)chunk * HQ + hq) * BT * BT;
  for (int e = tid; e < BT * BT; e += 256) {
    const int i = e >> 6, c = e & 63;
    float w = 0.f, cc = 0.f;
    if (i < R) {
      w = p.dus[((int64_t)(c0 + i) * HQ + hq) * BT + c] * __expf(p.gc[((int64_t)(c0 + i) * H + h) * BT + c]);
      if (c <= i) cc = cp[i * BT + c];
    }
    Wt[i * TLD + c] = f32_to_bf16(w);
    Ct[i * TLD + c] = f32_to_bf16(cc);
  }
  lds_barrier();
  const int i = 16 * wave + l16;   // this lane's row of the chunk
  f32x4 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) acc[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const bf16x8 bw = table_frag(Wt, i, hf, kb);   // contraction over m
    const bf16x8 bc = table_frag(Ct, i, hf, kb);   // contraction over j
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      acc[db] = mfma16(lds_frag_tr(Ht, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane), bw, acc[db]);   // hk0[d][m]
      acc[db] = mfma16(lds_frag_tr(Kt, LDT, 32 * hf, 32 * hf + 16, 16 * db, lane), bc, acc[db]);   // k'_j[d]
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

// bwd_slot_inter_kernel, grid (H, NT, 2): the parts that involve E_c, the state gradient carried
// into the END of chunk c (z = 0: k-state, rows k', output dk_gsa; z = 1: v-state, rows v', output
// dvs), with dec_r[m] = e^(gl[m] - gc_r[m]):
//   out[r][x] = intra part + sum_m (s_r[m] dec_r[m]) E[x][m]         as out^T = E sE^T
//   dsp[r][m] = dec_r[m] sum_x y_r[x] E[x][m]                         as Y E
template <int D>
__global__ __launch_bounds__(256) void bwd_slot_inter_kernel(const SP2 p) {
  constexpr int DB = D / 16, LDT = D + 16, TILE = BT * LDT, ELD = BT + 8;
  extern __shared__ __align__(16) unsigned char smem[];
  lbf16* const Yt = (lbf16*)smem;        // [64 rows r][D]   k' / v'
  lbf16* const Et = Yt + TILE;           // [D x][ELD]       E[x][m]
  lbf16* const St = Et + D * ELD;        // [64 r][TLD]      s_r[m] dec_r[m]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H;
  const int h = blockIdx.x, chunk = blockIdx.y;
  const bool isv = blockIdx.z != 0;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const bf16_t* ysrc = isv ? p.v : p.kg;
  int vlo = p.shift - it * BT;
  vlo = vlo < 0 ? 0 : vlo;
  {
    Tile<BT, D> ry;
#pragma unroll
    for (int u = 0; u < Tile<BT, D>::NPC; ++u) {
      const int c = tid + 256 * u;
      const int row = c / (D / 8), cc = (c % (D / 8)) * 8;
      uint4 x = make_uint4(0, 0, 0, 0);
      if (row >= vlo && row < R) x = *reinterpret_cast<const uint4*>(ysrc + (((int64_t)c0 + row - p.shift) * H + h) * D + cc);
      ry.r[u] = x;
    }
    ry.store(Yt, tid);
  }
  const float* ep = (isv ? p.ev : p.ek) + ((int64_t)chunk * H + h) * D * BT;
  for (int e = tid; e < D * BT; e += 256) Et[(e >> 6) * ELD + (e & 63)] = f32_to_bf16(ep[e]);
  const float* gcb = p.gc + ((int64_t)c0 * H + h) * BT;
  for (int e = tid; e < BT * BT; e += 256) {
    const int r = e >> 6, m = e & 63;
    float v = 0.f;
    if (r >= vlo && r < R)
      v = bf16_to_f32(p.s[(((int64_t)c0 + r - p.shift) * H + h) * BT + m]) *
          __expf(gcb[(int64_t)(R - 1) * H * BT + m] - gcb[(int64_t)r * H * BT + m]);
    St[r * TLD + m] = f32_to_bf16(v);
  }
  lds_barrier();
  const int col = 16 * wave + l16;
  // out^T[x][r = col] = sum_m E[x][m] sE[r][m]: A = E rows (plain), B = sE rows (plain), contraction m in 2 steps
  f32x4 accO[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) accO[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const bf16x8 bs = lds_frag(St, TLD, col, 32 * ks + 8 * kb);
#pragma unroll
    for (int db = 0; db < DB; ++db) accO[db] = mfma16(lds_frag(Et, ELD, 16 * db + l16, 32 * ks + 8 * kb), bs, accO[db]);
  }
  const bool has = col >= vlo && col < R;
  if (has) {
    const int64_t oi = (((int64_t)c0 + col - p.shift) * H + h) * D;
    float* part = isv ? p.dvs : p.dks;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const float4 pv = *reinterpret_cast<const float4*>(part + oi + 16 * db + 4 * kb);
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
    for (int xs = 0; xs < D / 32; ++xs) {
      struct { bf16x4 a, b; } t;
      t.a = *reinterpret_cast<const NHA_LDS bf16x4*>(Yt + (16 * rb + l16) * LDT + 32 * xs + 4 * kb);
      t.b = *reinterpret_cast<const NHA_LDS bf16x4*>(Yt + (16 * rb + l16) * LDT + 32 * xs + 16 + 4 * kb);
      acc = mfma16(__builtin_bit_cast(bf16x8, t), lds_frag_tr(Et, ELD, 32 * xs, 32 * xs + 16, 16 * wave, lane), acc);
    }
    // C[r = 16 rb + 4 kb + q][m = col]
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 16 * rb + 4 * kb + q;
      if (r < R) {
        const float dec = __expf(gcb[(int64_t)(R - 1) * H * BT + col] - gcb[(int64_t)r * H * BT + col]);
        p.dsp[(((int64_t)(isv ? 1 : 0) * p.T_tot + c0 + r) * H + h) * BT + col] = acc[q] * dec;
      }
    }
  }
}

template <int D, int TK>
int launch_dq(const WP& p, int NT, hipStream_t st) {
  const size_t lds = (size_t)4 * TK * (D + 16) * 2;
  static bool configured = false;
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
  static bool configured = false;
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

int bwd_window_mfma_dq(const NhaPrefillBwdArgs* a, const float* delta) {
  const WP p = make_wp(a, delta, nullptr);
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return launch_dq<64, 64>(p, a->NT, st);
  if (a->K == 128) return launch_dq<128, 64>(p, a->NT, st);
  return launch_dq<256, 32>(p, a->NT, st);
}

int bwd_window_mfma_dkv(const NhaPrefillBwdArgs* a, const float* delta, const float* dvs) {
  const WP p = make_wp(a, delta, dvs);
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return launch_dkv<64, 64, 0>(p, a->NT, st);
  if (a->K == 128) return launch_dkv<128, 64, 0>(p, a->NT, st);
  int rc = launch_dkv<256, 32, 1>(p, a->NT, st);
  if (rc != NHA_OK) return rc;
  return launch_dkv<256, 32, 2>(p, a->NT, st);
}

template <int D>
static int launch_slot_products(const SP1& p, int NT, hipStream_t st) {
  const size_t lds = (size_t)2 * BT * (D + 16) * 2;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)bwd_slot_products_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((bwd_slot_products_kernel<D>), dim3(p.HQ, NT), dim3(256), lds, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(slot products)");
  return NHA_OK;
}

// bf16, K == V in {64,128,256}, M == 64 (the shapes of the matrix-core state pass)
int bwd_slot_products(const NhaPrefillBwdArgs* a, const void* hkb, const void* hvb, float* ap, float* bp, float* ust, float* dpst) {
  SP1 p;
  p.q = (const bf16_t*)a->q_gsa; p.dout = (const bf16_t*)a->dout; p.kg = (const bf16_t*)a->k_gsa; p.v = (const bf16_t*)a->v;
  p.hkb = (const bf16_t*)hkb; p.hvb = (const bf16_t*)hvb;
  p.ap = ap; p.bp = bp; p.ust = ust; p.dpst = dpst;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.shift = a->shift;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->K == 64) return launch_slot_products<64>(p, a->NT, st);
  if (a->K == 128) return launch_slot_products<128>(p, a->NT, st);
  return launch_slot_products<256>(p, a->NT, st);
}

template <int D>
static int launch_slot_stage2(const SP2& p, int NT, int which, hipStream_t st) {
  const size_t lds_s = (size_t)BT * (D + 16) * 2 + (size_t)2 * BT * TLD * 2;
  const size_t lds_q = (size_t)2 * BT * (D + 16) * 2 + (size_t)2 * BT * TLD * 2;
  const size_t lds_i = (size_t)BT * (D + 16) * 2 + (size_t)D * (BT + 8) * 2 + (size_t)BT * TLD * 2;
  static bool configured = false;
  if (!configured) {
    hipError_t e1 = hipFuncSetAttribute((const void*)bwd_slot_state_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_s);
    hipError_t e2 = hipFuncSetAttribute((const void*)bwd_slot_dq_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_q);
    hipError_t e3 = hipFuncSetAttribute((const void*)bwd_slot_inter_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_i);
    if (e1 == hipSuccess) e1 = e3;
    if (e1 != hipSuccess || e2 != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve LDS: %s", hipGetErrorString(e1 != hipSuccess ? e1 : e2));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  if (which == 1) hipLaunchKernelGGL((bwd_slot_state_kernel<D>), dim3(p.H, NT, 2), dim3(256), lds_s, st, p);
  else if (which == 2) hipLaunchKernelGGL((bwd_slot_inter_kernel<D>), dim3(p.H, NT, 2), dim3(256), lds_i, st, p);
  else hipLaunchKernelGGL((bwd_slot_dq_kernel<D>), dim3(p.HQ, NT), dim3(256), lds_q, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(slot products, second stage)");
  return NHA_OK;
}

// which = 0: dq_gsa (bwd_slot_dq_kernel); 1: N_c and the intra-chunk parts of dk' / dv'
// (bwd_slot_state_kernel); 2: the parts that involve the scanned E_c (bwd_slot_inter_kernel).
// Same shapes as bwd_slot_products.
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

}  // namespace nha
