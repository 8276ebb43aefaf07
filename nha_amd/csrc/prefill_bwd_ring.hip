// Window branch of the NHA prefill backward, dq_swa, for groups of four query heads per kv-head at
// K == V == D == 128 (bf16): the data movement of ring_out_kernel (prefill_ring.hip) applied to the
// products of bwd_dq_kernel (prefill_bwd_mfma.hip; the part nha_fla/ops/nha/chunk.py:499-511 hands to
// flash-attn's backward).  With the merged log-sum-exp and delta = do . o of the whole op per (token,
// q-head):
//   S^T = K Q^T (log2 units, started at -lse),  dP^T = V dO^T,  dS^T = 2^S (dP^T - delta),
//   dQ^T += K^T dS^T,   dq_swa = scale dQ.
// One workgroup of 8 waves = one 64-token chunk x 4 query heads of one kv-head (32 queries per wave), so
// the K / V rows of the window are fetched once for the four heads; they go from global memory straight
// into LDS (global_load_lds_dwordx4) in units of 32 keys through a ring of four unit buffers.  A unit is
// three tiles: K and V as row fragments (A operands of the two score products) and K once more in the
// layout of the transposing read (A operand of K^T dS^T).  LDS layouts as in prefill_ring.hip.
#include "common.h"
#include "mfma_common.h"

#include <mutex>

namespace nha {
namespace {
using namespace mf;

typedef NHA_LDS unsigned char lbyte;

__device__ __forceinline__ void g2l16(const void* gbase, uint32_t voff_bytes, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff_bytes), "s"(gbase), "s"(lds_base) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

struct DqP {
  const bf16_t *q, *k, *v, *dout;          // q_swa [T,HQ,D]; k_swa, v [T,H,D]; dout [T,HQ,D]
  const float *lse_swa, *lse_gsa, *delta;  // [T,HQ]
  bf16_t* dq;
  const int32_t *cu, *cidx;
  int HQ, H, NG, NT, wl;
  float scale;
};

constexpr int D = 128;
constexpr int KS = D / 32;            // contraction steps of the score products
constexpr int DB = D / 16;            // 16-row blocks of dQ^T
constexpr int UB = 32 * D * 2;        // bytes of a 32-row tile
constexpr int HB = UB / 2;
constexpr int NR = 4;                 // ring slots
constexpr int UNIT = 3 * UB;          // K rows | V rows | K for the transposing read
constexpr int KR = 0, VR = UB, KT = 2 * UB;
constexpr int LPW = 3;                // LDS-direct loads per wave and unit (24 blocks of 1 KB, 8 waves)
constexpr int BYTES = NR * UNIT;
constexpr int RQB = 2;                // 16-row query blocks per wave

__global__ __launch_bounds__(512, 1) void ring_dq_kernel(const DqP p) {
  extern __shared__ __align__(1024) unsigned char smem_[];
  lbyte* const lds = (lbyte*)smem_;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  // grid = (kv-head x group of four q-heads, chunk), chunks from the last to the first
  const int chunk = p.NT - 1 - blockIdx.y;
  const int ngrp = NG / 4;
  const int h = blockIdx.x / ngrp, grp = blockIdx.x % ngrp;
  const int hq = h * NG + grp * 4 + wave / 2;
  const int qb0 = (wave % 2) * RQB;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int rows = (eos - c0) < BT ? (eos - c0) : BT;
  const float cs = p.scale * LOG2E;

  // unit u covers keys [c0 + 32 - 32 u, c0 + 64 - 32 u); c0 - bos is a multiple of 64, so no unit starts
  // before its sequence; units 0 and 1 are the chunk's own rows and may run past eos
  int lowest = bos;
  if (p.wl >= 0 && c0 - p.wl > bos) lowest = c0 - p.wl;
  const int nunits = (c0 + 64 - lowest + 31) / 32;   // >= 2

  // block b = wave + 8 i of a unit: tile b / 8, 16-row half (b % 8) / KS, 32-column block b % KS
  const int lrow16 = lane & 15, lpk = lane >> 4;                             // row fragments: piece lane / 16 of row lane % 16
  const int lrowv = (lane & 31) >> 1, lpv = 2 * (lane >> 5) + (lane & 1);    // transposing read: two planes of 32-byte rows
  const bf16_t* const kbase = p.k + ((int64_t)bos * H + h) * D;
  const bf16_t* const vbase = p.v + ((int64_t)bos * H + h) * D;
  // rows past eos (units 0 and 1 only) are read from row eos - 1: always masked, always finite
  auto issue_unit = [&](int u) {
    const int key0 = c0 + 32 - 32 * u;
    const int slot = u & (NR - 1);
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int b = wave + 8 * i;
      const int tile = b >> 3, rh = (b & 7) / KS, cq = b % KS;
      const bool tr = tile == 2;
      int row = key0 + 16 * rh + (tr ? lrowv : lrow16);
      row = row < eos ? row : eos - 1;
      const uint32_t off = ((uint32_t)(row - bos) * (uint32_t)(H * D) + (uint32_t)(4 * cq + (tr ? lpv : lpk)) * 8) * 2;
      g2l16(tile == 1 ? vbase : kbase, off, lds0 + slot * UNIT + tile * UB + rh * HB + cq * 1024);
    }
  };
#pragma unroll
  for (int u = 0; u < NR - 1; ++u)
    if (u < nunits) issue_unit(u);

  // query-side fragments: q pre-scaled by scale * log2(e) (the rounding the forward's scores saw), do as it is
  bf16x8 qf[RQB][KS], df[RQB][KS];
  float nlse[RQB], dl[RQB];
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    const bool valid = irow < rows;
    const int64_t tq = (int64_t)(c0 + (valid ? irow : 0)) * HQ + hq;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 x = make_uint4(0, 0, 0, 0), y = x;
      if (valid) {
        x = *reinterpret_cast<const uint4*>(p.q + tq * D + 32 * ks + 8 * kb);
        y = *reinterpret_cast<const uint4*>(p.dout + tq * D + 32 * ks + 8 * kb);
      }
      const uint32_t w[4] = {x.x, x.y, x.z, x.w};
      bf16x8 r;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = __uint_as_float((e & 1) ? (w[e >> 1] & 0xffff0000u) : (w[e >> 1] << 16));
        r[e] = (__bf16)(f * cs);
      }
      qf[qb][ks] = r;
      df[qb][ks] = as_bf16x8(y);
    }
    float ls = 0.f, lg = 0.f;
    if (valid) {
      ls = p.lse_swa[tq];
      lg = p.lse_gsa[tq];
    }
    const float mx = fmaxf(ls, lg);
    nlse[qb] = valid ? -(mx + __logf(__expf(ls - mx) + __expf(lg - mx))) * LOG2E : 0.f;
    dl[qb] = valid ? p.delta[tq] : 0.f;
  }
  f32x4 dQ[DB][RQB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) dQ[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const uint32_t kaddr = (uint32_t)(lane * 16);
  const uint32_t vaddr = (uint32_t)((4 * kb + (l16 >> 2)) * 32 + 8 * (l16 & 3));
  // row fragment (rows 16 kk + l16 of a tile, columns 32 ks + 8 kb ..) of a row-fragment tile at byte address a
  auto rfrag = [&](uint32_t a, int kk, int ks) -> bf16x8 {
    return *reinterpret_cast<const NHA_LDS bf16x8*>(lds + (a + kaddr) + kk * HB + ks * 1024);
  };
  // transposed fragment of the third tile: X[4 kb + e][16 db + l16] (e < 4) and X[16 + 4 kb + e - 4][..]
  auto tfrag = [&](uint32_t a, int db) -> bf16x8 {
    const lbyte* pa = lds + (a + vaddr) + (db >> 1) * 1024 + (db & 1) * 512;
    struct { s16x4 a, b; } t;
    t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
    t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)(pa + HB));
    return __builtin_bit_cast(bf16x8, t);
  };
  auto is_edge = [&](int u) -> bool { return (63 - 32 * u > 0) || (p.wl >= 0 && 32 - 32 * u < 63 - p.wl); };

  for (int u = 0; u < nunits; ++u) {
    // unit u has landed (this wave's part), then everybody's; units u+1, u+2 may stay in flight
    if (u + 2 < nunits) wait_vm<2 * LPW>();
    else if (u + 1 < nunits) wait_vm<LPW>();
    else wait_vm<0>();
    lds_barrier();
    // every wave is past unit u-1: its slot takes unit u+3
    if (u + NR - 1 < nunits) issue_unit(u + NR - 1);
    const uint32_t base = (uint32_t)((u & (NR - 1)) * UNIT);
    f32x4 S[2][RQB], dP[2][RQB];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) {
        S[kk][qb] = (f32x4){nlse[qb], nlse[qb], nlse[qb], nlse[qb]};
        dP[kk][qb] = (f32x4){-dl[qb], -dl[qb], -dl[qb], -dl[qb]};
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const bf16x8 ka = rfrag(base + KR, kk, ks), va = rfrag(base + VR, kk, ks);
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) {
          S[kk][qb] = mfma16(ka, qf[qb][ks], S[kk][qb]);
          dP[kk][qb] = mfma16(va, df[qb][ks], dP[kk][qb]);
        }
      }
    if (is_edge(u)) {
      const int xbase = 32 - 32 * u;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int qb = 0; qb < RQB; ++qb) {
          const int y = 16 * (qb0 + qb) + l16;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int x = xbase + 16 * kk + 4 * kb + r;
            const bool ok = (x <= y) && (p.wl < 0 || x >= y - p.wl);
            if (!ok) S[kk][qb][r] = -INFINITY;
          }
        }
    }
    bf16x8 dSb[RQB];
#pragma unroll
    for (int qb = 0; qb < RQB; ++qb) {
      f32x4 d0, d1;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        d0[r] = fexp2(S[0][qb][r]) * dP[0][qb][r];
        d1[r] = fexp2(S[1][qb][r]) * dP[1][qb][r];
      }
      dSb[qb] = pack8(d0, d1);
    }
    // dQ^T[d][q] += K^T[d][key] dS^T[key][q]
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const bf16x8 kt = tfrag(base + KT, db);
#pragma unroll
      for (int qb = 0; qb < RQB; ++qb) dQ[db][qb] = mfma16(kt, dSb[qb], dQ[db][qb]);
    }
  }
#pragma unroll
  for (int qb = 0; qb < RQB; ++qb) {
    const int irow = 16 * (qb0 + qb) + l16;
    if (irow >= rows) continue;
    bf16_t* op = p.dq + ((int64_t)(c0 + irow) * HQ + hq) * D + 4 * kb;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 pk;
#pragma unroll
      for (int r = 0; r < 4; ++r) pk[r] = (__bf16)(dQ[db][qb][r] * p.scale);
      *reinterpret_cast<bf16x4*>(op + 16 * db) = pk;
    }
  }
}

}  // namespace

// Served: four (or a multiple of four) query heads per kv-head at D = 128, tensors of one call below 4 GiB
// (32-bit lane offsets of the LDS-direct loads).
bool bwd_ring_dq_supported(const NhaPrefillBwdArgs* a) {
  static const bool off = getenv("NHA_BWD_NO_RING") != nullptr;   // A/B switch for measurements
  if (off || a->K != 128 || a->V != 128 || a->HQ % a->H != 0 || (a->HQ / a->H) % 4 != 0) return false;
  return (int64_t)a->T_tot * a->H * 128 * 2 < ((int64_t)1 << 32);
}

int bwd_ring_dq(const NhaPrefillBwdArgs* a, const float* delta) {
  DqP p;
  p.q = (const bf16_t*)a->q_swa; p.k = (const bf16_t*)a->k_swa; p.v = (const bf16_t*)a->v; p.dout = (const bf16_t*)a->dout;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa; p.delta = delta;
  p.dq = (bf16_t*)a->dq_swa;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.NT = a->NT; p.wl = a->wl; p.scale = a->scale;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] { attr_err = hipFuncSetAttribute((const void*)ring_dq_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, BYTES); });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_bwd: cannot reserve %d bytes of LDS: %s", BYTES, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(ring_dq_kernel, dim3(p.H * (p.NG / 4), p.NT), dim3(512), BYTES, (hipStream_t)a->stream, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(window dq, ring)");
  return NHA_OK;
}

}  // namespace nha
