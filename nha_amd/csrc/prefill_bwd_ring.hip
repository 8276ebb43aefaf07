// Window branch of the NHA prefill backward for K == V == D == 128 (bf16) with four (or a multiple of
// four) query heads per kv-head: the data movement of ring_out_kernel (prefill_ring.hip) applied to the
// products of bwd_dq_kernel / bwd_dkv_kernel (prefill_bwd_mfma.hip; the part
// nha_fla/ops/nha/chunk.py:499-511 hands to flash-attn's backward).  With the merged log-sum-exp and
// delta = do . o of the whole op per (token, q-head), window logits w = scale q.k:
//   pi = e^(w - lse),  dw = pi (do.v - delta),
//   dq_swa_q = scale sum_j dw k_j,   dk_swa_j = scale sum_q dw q_q,   dv_j += sum_q pi do_q.
// Every streamed operand goes from global memory straight into LDS (global_load_lds_dwordx4) through a
// ring of four buffers; LDS layouts as in prefill_ring.hip (row-fragment tiles read as consecutive
// bytes, tiles for the transposing read in two planes of 32-byte rows).
//
// ring_dq_kernel: one workgroup of 8 waves = one 64-token chunk x 4 query heads of one kv-head (a query
//   per lane, 32 queries per wave), so the K / V rows of the window are fetched once for the four heads,
//   in units of 32 keys.  A unit is three tiles: K and V as row fragments (A operands of S^T = K Q^T and
//   dP^T = V dO^T) and K once more for the transposing read (A operand of dQ^T += K^T dS^T).  It also
//   leaves (-lse / scale, -delta) per (token, q-head) as pairs for the kernel below, whose score and
//   dP accumulators start from them.
// ring_dkv_kernel: one workgroup of 8 waves = 256 keys of one kv-head (a key per lane and 16-key block, 32 keys per wave,
//   K and V rows in registers); the q / do rows of every query head of the group stream through the ring
//   in items of 32 queries: four tiles (q and do as row fragments for S = Q K^T and dP = dO V^T, and once
//   more for the transposing read: dV^T += dO^T P, dK^T += Q^T dS) plus the 32 (lse, delta) pairs.
//   The first and the last units of a head are triangles over the waves (causal edge, window edge) that
//   complement each other: such units are held in LDS two at a time and every wave works on its own.
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
  float2* ld;                              // [T,HQ] out: (-lse / scale, -delta) of the merged softmax
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
  const int ngrp = NG / 4;
  int vx, vy;
  xcd_tile(ngrp, p.NT, vx, vy);
  const int chunk = p.NT - 1 - vy;
  const int h = vx / ngrp, grp = vx % ngrp;
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
    if (valid && kb == 0) p.ld[tq] = make_float2(nlse[qb] / cs, -dl[qb]);
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

// ------------------------------------------------------------------------------------------------------
struct DkvP {
  const bf16_t *q, *k, *v, *dout;          // q_swa [T,HQ,D]; k_swa, v [T,H,D]; dout [T,HQ,D]
  const float2* ld;                        // [T,HQ] (-lse / scale, -delta): what the two score accumulators start from
  const float* dvs;                        // [T,H,D] slot-branch part of dv
  bf16_t *dk, *dv;
  const int32_t *cu, *cidx;
  int HQ, H, NG, NT, wl;
  float scale;
};

constexpr int KV_ITEM = 4 * UB + 1024;   // q rows | do rows | q transposing | do transposing | 32 (lse, delta) pairs
constexpr int KV_QR = 0, KV_OR = UB, KV_QT = 2 * UB, KV_OT = 3 * UB, KV_LD = 4 * UB;
constexpr int KV_BYTES = NR * KV_ITEM;

__device__ __forceinline__ void g2l4(const void* gbase, uint32_t voff_bytes, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff_bytes), "s"(gbase), "s"(lds_base) : "memory");
}

// KEYS: keys per workgroup, 256 or 128 (a wave holds KEYS / 8 of them).  With 256 every q / do fragment read from LDS
// feeds two matrix products, with 128 one: long windows, which are bound by those reads, take 256 (headline shape:
// 1.17 ms against 1.5 ms); windows up to 160 keys, where a workgroup's walk is a few items long and the half-size
// key groups spread more evenly over the CUs, take 128 (window 64: whole backward 1.63 against 1.70 ms).
template <int KEYS>
__global__ __launch_bounds__(512, 1) void ring_dkv_kernel(const DkvP p) {
  constexpr int NKB = KEYS / 16 / 8;       // 16-key blocks per wave
  constexpr int CPG = KEYS / 64;           // chunks per key group
  constexpr int UPG = KEYS / 32;           // 32-query units that a key group spans
  constexpr int KV_LPW = 4;   // tile loads per wave and item (32 blocks of 1 KB, 8 waves)
  extern __shared__ __align__(1024) unsigned char smem_[];
  lbyte* const lds = (lbyte*)smem_;
  const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kb = lane >> 4;
  const int H = p.H, HQ = p.HQ, NG = p.NG;
  // grid = (kv-head, chunk): the workgroup of every CPG-th chunk of a sequence (every fourth, at 256 keys) takes that
  // chunk and the next CPG - 1; the others leave at once.  Workgroups are handed to the shader engines in turn, in
  // launch order: were the working ones every fourth of that order they would all land on the same engine.  The
  // launch order therefore walks the chunks with stride CPG (chunks 0, 4, 8, ... first, then 1, 5, 9, ...), so that
  // the chunks of a sequence that start a key group are neighbours in it; chunks from the last to the first.
  const int nq = (p.NT + CPG - 1) / CPG;
  const int cperm = CPG * (blockIdx.y % nq) + blockIdx.y / nq;
  if (cperm >= p.NT) return;
  const int chunk = p.NT - 1 - cperm;
  const int h = blockIdx.x;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  if (it & (CPG - 1)) return;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int kspan = (eos - c0) < KEYS ? (eos - c0) : KEYS;
  const float cs = p.scale * LOG2E;
  // queries that see a key of the workgroup: [c0, qend), in items of 32 per query head
  int qend = eos;
  if (p.wl >= 0 && c0 + kspan + p.wl < eos) qend = c0 + kspan + p.wl;
  const int nun = (qend - c0 + 31) / 32;   // >= 1
  const int total = NG * nun;

  // block (16-row half wave / 4, 32-column block wave % 4) of each of the four tiles of an item
  const int rh = wave >> 2, cq = wave & 3;
  // item (g, u): rows [c0 + 32 u, c0 + 32 u + 32) of query head h NG + g; rows past eos are read from row
  // eos - 1 (always masked, always finite)
  auto issue_item = [&](int g, int u, int slot) {
    // what follows from the lane number is derived again at every request: kept across the loop it would
    // cost registers the accumulators need
    int ln = threadIdx.x & 63;
    asm volatile("" : "+v"(ln));
    const int lrow16 = ln & 15, lpk = ln >> 4;
    const int lrowv = (ln & 31) >> 1, lpv = 2 * (ln >> 5) + (ln & 1);
    const int hq = h * NG + g;
    const int q0 = c0 + 32 * u;
    const bf16_t* const qbase = p.q + ((int64_t)bos * HQ + hq) * D;
    const bf16_t* const obase = p.dout + ((int64_t)bos * HQ + hq) * D;
    int rr = q0 + 16 * rh + lrow16;
    rr = rr < eos ? rr : eos - 1;
    int rt = q0 + 16 * rh + lrowv;
    rt = rt < eos ? rt : eos - 1;
    const uint32_t offr = ((uint32_t)(rr - bos) * (uint32_t)(HQ * D) + (uint32_t)(4 * cq + lpk) * 8) * 2;
    const uint32_t offt = ((uint32_t)(rt - bos) * (uint32_t)(HQ * D) + (uint32_t)(4 * cq + lpv) * 8) * 2;
    const uint32_t dst = lds0 + slot * KV_ITEM + rh * HB + cq * 1024;
    g2l16(qbase, offr, dst + KV_QR);
    g2l16(obase, offr, dst + KV_OR);
    g2l16(qbase, offt, dst + KV_QT);
    g2l16(obase, offt, dst + KV_OT);
    if (wave == 0) {
      int r = q0 + (ln >> 1);
      r = r < eos ? r : eos - 1;
      g2l4(p.ld, (uint32_t)(((int64_t)r * HQ + hq) * 2 + (ln & 1)) * 4u, lds0 + slot * KV_ITEM + KV_LD);
    }
  };
  // The workgroups of neighbouring key groups of a sequence run at the same time on one XCD, and their
  // query ranges overlap by all but 8 units.  Each walks the units of a head cyclically, starting where
  // the walk of the sequence's first key group would be at that moment: neighbours then request the same
  // q / do rows at about the same time and the second request finds them in L2.
  const int rot = (nun - (UPG * (it / CPG)) % nun) % nun;
  // Complementary units.  Against the 256 keys of the workgroup the first units of a head are triangles (wave w has
  // work in unit u only if w <= u: the queries of a unit must not all lie before the wave's keys) and so are the last
  // ones (the keys must not all have left the window: unit a + K0 has work only for the waves w >= a + 1), and a
  // workgroup takes as long over a unit as its busiest wave.  Units a < npair are therefore worked on together with
  // unit a + K0: both are in LDS at once and every wave takes the one it has work in, never both.
  const int K0 = p.wl >= 0 ? (p.wl + 63) / 32 : 0;
  int npair = 0;
  if (p.wl >= 0 && K0 >= UPG - 1 && nun > K0) npair = (nun - K0) < UPG - 1 ? (nun - K0) : UPG - 1;
  // the walk of a head: its units in cyclic order from rot, the second units of the pairs left out
  auto walk_skip = [&](int x) {
    if (x >= nun) x -= nun;
    if (x >= K0 && x < K0 + npair) {   // empty range without pairs
      x = K0 + npair;
      if (x >= nun) x -= nun;
    }
    return x;
  };
  const int rot0 = walk_skip(rot);
  struct Walk { int g, u, cnt; };
  auto advance = [&](Walk& w) {
    w.cnt += (w.u < npair) ? 2 : 1;
    w.u = walk_skip(w.u + 1);
    if (w.cnt == nun) {
      w.cnt = 0;
      w.u = rot0;
      ++w.g;
    }
  };
  // requests, in the order the loop below consumes the items: the unit of a step, then the unit paired with it
  Walk pw = {0, rot0, 0};
  int pend_u = -1, pend_g = 0;
  auto issue_next = [&](int slot) {
    if (pend_u >= 0) {
      issue_item(pend_g, pend_u, slot);
      pend_u = -1;
      return;
    }
    issue_item(pw.g, pw.u, slot);
    if (pw.u < npair) {
      pend_u = pw.u + K0;
      pend_g = pw.g;
    }
    advance(pw);
  };
  int issued = 0;
  for (; issued < NR - 1 && issued < total; ++issued) issue_next(issued);

  // this lane's keys (one per 16-key block of the wave) and their K / V rows (B operands: K[key][32 ks + 8 kb ..])
  const int kbase = 16 * NKB * wave;               // first key of the wave, relative to c0
  bf16x8 kfr[NKB][KS], vfr[NKB][KS];
#pragma unroll
  for (int kk = 0; kk < NKB; ++kk) {
    const int tk = c0 + kbase + 16 * kk + l16;
    const int64_t jk = (int64_t)(tk < eos ? tk : eos - 1) * H + h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kfr[kk][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(p.k + jk * D + 32 * ks + 8 * kb));
      vfr[kk][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(p.v + jk * D + 32 * ks + 8 * kb));
    }
  }
  // the K / V rows are in their registers before the loop starts: left to the compiler, the wait for them sits
  // at their first use inside the loop, as a wait for every load in flight, the LDS-direct ones included
#pragma unroll
  for (int kk = 0; kk < NKB; ++kk)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      asm volatile("" : "+v"(kfr[kk][ks]));
      asm volatile("" : "+v"(vfr[kk][ks]));
    }
  f32x4 dK[DB][NKB], dV[DB][NKB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int kk = 0; kk < NKB; ++kk) {
      dK[db][kk] = (f32x4){0.f, 0.f, 0.f, 0.f};
      dV[db][kk] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  uint32_t kaddr, vaddr;   // set per item (see issue_item)
  auto rfrag = [&](uint32_t a, int kk, int ks) -> bf16x8 {
    return *reinterpret_cast<const NHA_LDS bf16x8*>(lds + (a + kaddr) + kk * HB + ks * 1024);
  };
  auto tfrag = [&](uint32_t a, int db) -> bf16x8 {
    const lbyte* pa = lds + (a + vaddr) + (db >> 1) * 1024 + (db & 1) * 512;
    struct { s16x4 a, b; } t;
    t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
    t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)(pa + HB));
    return __builtin_bit_cast(bf16x8, t);
  };

  // queries [32 u, 32 u + 32) against keys [kbase, kbase + 16 NKB), both relative to c0: nothing to do if
  // every query is before every key or past the window of every key
  auto no_work = [&](int u) { return (32 * u + 31 < kbase) || (p.wl >= 0 && 32 * u > kbase + 16 * NKB - 1 + p.wl); };
  Walk cw = {0, rot0, 0};
  for (int k = 0; k < total;) {
    const int prim = cw.u;
    const int need = prim < npair ? 2 : 1;   // items of this step: k .. k + need - 1
    advance(cw);
    // they have landed (this wave's part; wave 0 carries one more load per item), then everybody's; the
    // requests after them stay in flight
    const int younger = issued - (k + need);
    if (younger >= 2) {
      if (wave == 0) wait_vm<2 * (KV_LPW + 1)>();
      else wait_vm<2 * KV_LPW>();
    } else if (younger == 1) {
      if (wave == 0) wait_vm<KV_LPW + 1>();
      else wait_vm<KV_LPW>();
    } else {
      wait_vm<0>();
    }
    lds_barrier();
    // every wave is past the items before k: their slots take the next requests
    for (; issued < total && issued < k + NR; ++issued) issue_next(issued & (NR - 1));
    int u = prim;
    uint32_t base = (uint32_t)((k & (NR - 1)) * KV_ITEM);
    if (need == 2 && no_work(prim)) {
      u = prim + K0;
      base = (uint32_t)(((k + 1) & (NR - 1)) * KV_ITEM);
    }
    k += need;
    int lc = threadIdx.x & 63;
    asm volatile("" : "+v"(lc));
    const int l16 = lc & 15, kb = lc >> 4;
    kaddr = (uint32_t)(lc * 16);
    vaddr = (uint32_t)((4 * kb + (l16 >> 2)) * 32 + 8 * (l16 & 3));
    if (!no_work(u)) {
      const bool edge = (32 * u < kbase + 16 * NKB - 1) || (p.wl >= 0 && 32 * u + 31 > kbase + p.wl) || (c0 + 32 * u + 32 > eos);
      // ---- phase 1: S = Q K^T and dP = dO V^T, one 16-key block at a time (two blocks of scores beside both
      //      gradient accumulators do not fit the register file, so the q / do row fragments are read once per
      //      block); step i = (contraction step i / 2, 16-query block i % 2).  PD1 / PD2: how many steps ahead
      //      of its product a fragment is requested from LDS; what the register file allows here (as two
      //      launches, one gradient each, there is room for 2-3 steps and both blocks of scores: 873 + 709 us
      //      against 1178 us for this kernel) ----
      constexpr int N1 = 2 * KS;
      constexpr int GS = 1;
      constexpr int PD1 = NKB == 2 ? 0 : 1;
      constexpr int PD2 = 1;
      bf16x8 Pb[NKB], dSb[NKB];
      bf16x8 ot[DB], qt[DB];
#pragma unroll
      for (int g0 = 0; g0 < NKB; g0 += GS) {
        f32x4 S[2][GS], dP[2][GS];
        bf16x8 qa[N1], oa[N1];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < PD1; ++i) {
          qa[i] = rfrag(base + KV_QR, i & 1, i >> 1);
          oa[i] = rfrag(base + KV_OR, i & 1, i >> 1);
        }
        // rows of the accumulators are the queries 16 qb + 4 kb + r, the column is this lane's key of block
        // g0 + j; they start from (-lse / scale, -delta) of their rows
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          const NHA_LDS f32x4* lp = reinterpret_cast<const NHA_LDS f32x4*>(lds + base + KV_LD + (16 * qb + 4 * kb) * 8);
          const f32x4 a0 = lp[0], a1 = lp[1];   // the pairs of rows r = 0, 1 and r = 2, 3
#pragma unroll
          for (int j = 0; j < GS; ++j) {
            S[qb][j] = (f32x4){a0[0], a0[2], a1[0], a1[2]};
            dP[qb][j] = (f32x4){a0[1], a0[3], a1[1], a1[3]};
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < N1; ++i) {
          const int qb = i & 1, ks = i >> 1;
          if (i + PD1 < N1) {
            qa[i + PD1] = rfrag(base + KV_QR, (i + PD1) & 1, (i + PD1) >> 1);
            oa[i + PD1] = rfrag(base + KV_OR, (i + PD1) & 1, (i + PD1) >> 1);
          }
#pragma unroll
          for (int j = 0; j < GS; ++j) {
            S[qb][j] = mfma16(qa[i], kfr[g0 + j][ks], S[qb][j]);
            dP[qb][j] = mfma16(oa[i], vfr[g0 + j][ks], dP[qb][j]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        // the first transposed fragments of phase 2 are requested before the last exponentials
        if (g0 + GS == NKB) {
#pragma unroll
          for (int i = 0; i < PD2; ++i) {
            ot[i] = tfrag(base + KV_OT, i);
            qt[i] = tfrag(base + KV_QT, i);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < GS; ++j) {
          const int kk = g0 + j;
          f32x4 P[2], dS[2];
#pragma unroll
          for (int qb = 0; qb < 2; ++qb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float x = S[qb][j][r] * cs;
              if (edge) {
                const int y = 32 * u + 16 * qb + 4 * kb + r, xk = kbase + 16 * kk + l16;
                const bool ok = (xk <= y) && (p.wl < 0 || y - xk <= p.wl) && (c0 + y < eos);
                if (!ok) x = -INFINITY;
              }
              const float pr = fexp2(x);
              P[qb][r] = pr;
              dS[qb][r] = pr * dP[qb][j][r];
            }
          Pb[kk] = pack8(P[0], P[1]);
          dSb[kk] = pack8(dS[0], dS[1]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- phase 2: dV^T[d][key] += dO^T[d][q] P[q][key];  dK^T[d][key] += Q^T[d][q] dS[q][key] ----
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        if (db + PD2 < DB) {
          ot[db + PD2] = tfrag(base + KV_OT, db + PD2);
          qt[db + PD2] = tfrag(base + KV_QT, db + PD2);
        }
#pragma unroll
        for (int kk = 0; kk < NKB; ++kk) {
          dV[db][kk] = mfma16(ot[db], Pb[kk], dV[db][kk]);
          dK[db][kk] = mfma16(qt[db], dSb[kk], dK[db][kk]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
#pragma unroll
  for (int kk = 0; kk < NKB; ++kk) {
    const int tk = c0 + kbase + 16 * kk + l16;
    if (tk >= eos) continue;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int64_t off = ((int64_t)tk * H + h) * D + 16 * db + 4 * kb;
      bf16x4 pk;
      {
#pragma unroll
        for (int r = 0; r < 4; ++r) pk[r] = (__bf16)(dK[db][kk][r] * p.scale);
        *reinterpret_cast<bf16x4*>(p.dk + off) = pk;
      }
      {
        const float4 sv = *reinterpret_cast<const float4*>(p.dvs + off);
        pk[0] = (__bf16)(dV[db][kk][0] + sv.x);
        pk[1] = (__bf16)(dV[db][kk][1] + sv.y);
        pk[2] = (__bf16)(dV[db][kk][2] + sv.z);
        pk[3] = (__bf16)(dV[db][kk][3] + sv.w);
        *reinterpret_cast<bf16x4*>(p.dv + off) = pk;
      }
    }
  }
}

}  // namespace

// Served: four (or a multiple of four) query heads per kv-head at D = 128, tensors of one call below 4 GiB
// (32-bit lane offsets of the LDS-direct loads).
bool bwd_ring_supported(const NhaPrefillBwdArgs* a) {
#ifdef NHA_AB_SWITCHES   // measurement builds only (-DNHA_AB_SWITCHES)
  static const bool off = getenv("NHA_BWD_NO_RING") != nullptr;
#else
  constexpr bool off = false;
#endif
  if (off || a->K != 128 || a->V != 128 || a->HQ % a->H != 0 || (a->HQ / a->H) % 4 != 0) return false;
  return (int64_t)a->T_tot * a->HQ * 128 * 2 < ((int64_t)1 << 32);
}

int bwd_ring_dq(const NhaPrefillBwdArgs* a, const float* delta, float2* ld) {
  DqP p;
  p.q = (const bf16_t*)a->q_swa; p.k = (const bf16_t*)a->k_swa; p.v = (const bf16_t*)a->v; p.dout = (const bf16_t*)a->dout;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa; p.delta = delta;
  p.dq = (bf16_t*)a->dq_swa; p.ld = ld;
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

int bwd_ring_dkv(const NhaPrefillBwdArgs* a, const float2* ld, const float* dvs) {
  DkvP p;
  p.q = (const bf16_t*)a->q_swa; p.k = (const bf16_t*)a->k_swa; p.v = (const bf16_t*)a->v; p.dout = (const bf16_t*)a->dout;
  p.ld = ld; p.dvs = dvs;
  p.dk = (bf16_t*)a->dk_swa; p.dv = (bf16_t*)a->dv;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices;
  p.HQ = a->HQ; p.H = a->H; p.NG = a->HQ / a->H; p.NT = a->NT; p.wl = a->wl; p.scale = a->scale;
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute((const void*)ring_dkv_kernel<256>, hipFuncAttributeMaxDynamicSharedMemorySize, KV_BYTES);
    if (attr_err == hipSuccess)
      attr_err = hipFuncSetAttribute((const void*)ring_dkv_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize, KV_BYTES);
  });
  if (attr_err != hipSuccess) {
    set_error("nha_prefill_bwd: cannot reserve %d bytes of LDS: %s", KV_BYTES, hipGetErrorString(attr_err));
    return NHA_ERR_LAUNCH;
  }
  // one launch row per chunk, rounded up to whole key groups (4 chunks of 256 keys, 2 of 128)
  if (p.wl >= 0 && p.wl < 160)
    hipLaunchKernelGGL(ring_dkv_kernel<128>, dim3(p.H, 2 * ((p.NT + 1) / 2)), dim3(512), KV_BYTES, (hipStream_t)a->stream, p);
  else
    hipLaunchKernelGGL(ring_dkv_kernel<256>, dim3(p.H, 4 * ((p.NT + 3) / 4)), dim3(512), KV_BYTES, (hipStream_t)a->stream, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(window dk, dv, ring)");
  return NHA_OK;
}

}  // namespace nha
