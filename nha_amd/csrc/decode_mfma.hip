// Matrix-core decode step for gfx950: bf16, K == V == D in {64,128,256}, M == 64 slots, up to 8 query
// heads per kv-head; window or ring mode with a pre-rotated window query, or window mode with
// in-kernel rotate-half RoPE of the raw query and window keys (cos / sin tables,
// nha_fla/ops/nha/fused_recurrent.py:309-329).
//
// Same work split as decode.hip (one workgroup per (sequence, kv-head), state and window read
// once), but the window is streamed ONCE, in 32-key blocks dealt round-robin to the waves:
//   S^T[key][head] = K Q^T       A = 16 key rows loaded from HBM straight into the A-operand layout
//                                (lane l: row l%16, 16-byte piece l/16 of each 64-byte k-step)
//   O^T[v][head]  += V^T P^T     V rows go HBM -> registers -> a wave-private LDS tile and come back
//                                transposed (ds_read_b64_tr_b16); P leaves the accumulator layout of
//                                S^T as the B operand with no lane movement
// so a lane owns one query head and the online softmax needs two cross-lane steps per block.  The
// per-key VALU work of the two-sweep kernel (convert, 8 FMA per head, row reductions) disappears
// and each wave keeps two 32-key blocks (32 KB) of loads in flight.  Slot state update, slot
// logits and slot read stay fp32 VALU (nha_fla/ops/nha/fused_recurrent.py:305, :342-349, :416);
// slots and the per-wave window partials are merged at the end under one softmax.
#include "common.h"
#include <stdlib.h>

namespace nha {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define NHA_LDS __attribute__((address_space(3)))
typedef NHA_LDS bf16_t lbf16;
typedef NHA_LDS float lfloat;

constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 u) { return __builtin_bit_cast(bf16x8, u); }
__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
// workgroup barrier that orders LDS traffic only; global loads stay in flight across it
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// max over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48)
__device__ __forceinline__ float max_over_rows(float x) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned v = __float_as_uint(x);
  const auto b = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float sum_over_rows(float x) {
  const unsigned u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const unsigned v = __float_as_uint(x);
  const auto b = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// the lane (c = l%16, kb = l/16) receives X[4*kb + e][col0 + c] for e = 0..3 and
// X[16 + 4*kb + e][col0 + c] for e = 4..7 of a row-major [32][ld] bf16 LDS tile
__device__ __forceinline__ bf16x8 lds_frag_tr(const lbf16* tile, int ld, int col0, int lane) {
  const int l16 = lane & 15, kb = lane >> 4;
  const lbf16* pa = tile + (4 * kb + (l16 >> 2)) * ld + col0 + 4 * (l16 & 3);
  const lbf16* pb = pa + 16 * ld;
  struct { s16x4 a, b; } t;
  t.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pa);
  t.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NHA_LDS s16x4*)pb);
  return __builtin_bit_cast(bf16x8, t);
}

// 16 bytes of a window row: read once per step and never again, so the load is marked
// non-temporal (it does not displace the state lines in L2; measured 145 -> 134 us per step)
__device__ __forceinline__ uint4 ld16_stream(const bf16_t* p) {
  const u32x4 x = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(x[0], x[1], x[2], x[3]);
}

constexpr int MS = 64;   // slots

static size_t lds_bytes_for(int D, int G, int NW, bool rot) {
  const size_t fl = (size_t)2 * MS + 2 * D + (size_t)G * D + (size_t)G * MS + (size_t)NW * G * (D > MS ? D : MS) + 16 * NW * 2 + 32;
  // rotary: per wave the cos and sin pieces of one 32-key block, 16 bytes per lane and piece
  return fl * 4 + (size_t)NW * 32 * (D + 16) * 2 + (rot ? (size_t)NW * 4 * (D / 32) * 1024 : 0);
}

// 16 bytes per lane from global memory into LDS at lds_base + 16 * lane (lds_base wave-uniform): the
// cos / sin pieces of the next block wait there instead of in registers.  Outside the compiler's
// memory model: no wait the compiler places knows of it, so its reader waits by count (s_waitcnt vmcnt)
// for everything issued up to it.
__device__ __forceinline__ void g2l16(const void* gbase, uint32_t voff_bytes, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff_bytes), "s"(gbase), "s"(lds_base) : "memory");
}

// rotate-half of the column pair (c, c + D/2), 8 columns at a time: xa holds columns c.., xb columns
// c + D/2..; out_a = xa cos_a - xb sin_a, out_b = xb cos_b + xa sin_b (fp32, rounded to bf16 once)
__device__ __forceinline__ void rope8(uint4& xa, uint4& xb, uint4 ca, uint4 sa, uint4 cb, uint4 sb) {
  const uint32_t a[4] = {xa.x, xa.y, xa.z, xa.w}, b[4] = {xb.x, xb.y, xb.z, xb.w};
  const uint32_t c0[4] = {ca.x, ca.y, ca.z, ca.w}, s0[4] = {sa.x, sa.y, sa.z, sa.w};
  const uint32_t c1[4] = {cb.x, cb.y, cb.z, cb.w}, s1[4] = {sb.x, sb.y, sb.z, sb.w};
  uint32_t oa[4], ob[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float ra[2], rb[2];
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      auto f = [&](uint32_t w) { return __uint_as_float(hlf ? (w & 0xffff0000u) : (w << 16)); };
      ra[hlf] = f(a[i]) * f(c0[i]) - f(b[i]) * f(s0[i]);
      rb[hlf] = f(b[i]) * f(c1[i]) + f(a[i]) * f(s1[i]);
    }
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 pa, pb;
    pa[0] = (__bf16)ra[0]; pa[1] = (__bf16)ra[1];
    pb[0] = (__bf16)rb[0]; pb[1] = (__bf16)rb[1];
    oa[i] = __builtin_bit_cast(uint32_t, pa);
    ob[i] = __builtin_bit_cast(uint32_t, pb);
  }
  xa = make_uint4(oa[0], oa[1], oa[2], oa[3]);
  xb = make_uint4(ob[0], ob[1], ob[2], ob[3]);
}

// One workgroup of NW waves per (sequence, kv-head): slot branch, then window branch, then the
// merge.  NW = 2 with up to 256 registers per lane puts a grid of 1024 workgroups on the chip at
// once (4 workgroups per CU), so nothing waits for a second round.  The slot branch issues every
// load it needs up front (popped entry first, then all state rows): its dependent chain is
// count -> popped row, and no workgroup's state rows queue behind another's window stream.
// ROT: window mode with cos / sin tables.  Row w of the window is rotated by row w of the tables (the
// tables' last W rows, ascending in time like the window), the query by row W-1.  A column and its
// partner at +-D/2 sit in the same lane (k-steps j and j +- KS/2), so the rotation moves nothing
// between lanes; the cos / sin pieces of a block are as many bytes again as twice its keys, so they
// wait in a per-wave LDS area (requested one block ahead) instead of doubling the register buffers.
template <int D, int G, int NW, bool ROT>
__global__ __launch_bounds__(64 * NW, 2) void decode_mfma_kernel(const NhaDecodeArgs a) {
  constexpr int NT = 64 * NW;
  constexpr int LDT = D + 16;   // bf16 row stride of a V tile
  constexpr int KS = D / 32;    // MFMA k-steps over the head dim
  constexpr int NVT = D / 16;   // 16-row blocks of O^T == 16-byte V loads per lane and block
  constexpr int LV = D / 8;     // lanes per V / hv row
  constexpr int RV = 64 / LV;   // rows per wave-wide load
  constexpr int M = MS;
  constexpr int LM = M / 8, RM = 64 / LM;
  constexpr int NIK = D / (RM * NW);   // hk rows per lane
  constexpr int NIV = M / (RV * NW);   // hv rows per lane
  constexpr int MV = D > M ? D : M;
  extern __shared__ __align__(16) float lds_raw[];
  const int W = a.W, H = a.H, HQ = a.HQ;
  const int NG = HQ / H;
  float* eg = lds_raw;
  float* sg = eg + M;
  float* kp = sg + M;
  float* vp = kp + D;
  float* qs = vp + D;               // [G][D] slot-branch query, scale * log2(e) folded in
  float* ok = qs + G * D;           // [G][M] slot probabilities (unnormalised)
  float* part = ok + G * M;         // [NW][G][MV] per-wave partial sums
  float* wm = part + NW * G * MV;   // [NW][16] per-wave window max (log2 units)
  float* wl = wm + 16 * NW;         // [NW][16] per-wave window sum
  float* ms = wl + 16 * NW;         // [16] slot max, [16] slot sum
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, qd = lane >> 4;
  lbf16* X = (lbf16*)(NHA_LDS void*)(ms + 32) + wave * 32 * LDT;   // wave-private V tile [32][LDT]
  // rotary: [table cos|sin][row half t][k-step j] x 1 KB (16 bytes per lane), per wave
  NHA_LDS unsigned char* const CS = (NHA_LDS unsigned char*)((lbf16*)(NHA_LDS void*)(ms + 32) + NW * 32 * LDT) + wave * (4 * KS * 1024);
  const uint32_t cs_lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)CS);   // wave-uniform: it goes to m0
  int b = blockIdx.x / H, h = blockIdx.x % H;
  if constexpr (ROT) {
    // Workgroups are dealt to the 8 XCDs in launch order: with consecutive workgroups the kv-heads of one sequence,
    // the cos / sin rows of a sequence -- the same for all its heads -- would be fetched into eight L2s, once each
    // (as many bytes again as the keys and values of the whole step).  With tables of their own per sequence, XCD x
    // takes the sequences b % 8 == x with all their heads, which run at the same time and find each other's table
    // rows in their L2 (B = 128, 8 kv-heads, W = 1024: 186 -> 168 us per step; tables shared by the batch are in
    // every L2 anyway and keep the plain order).
    const int B = gridDim.x / H;
    if (a.cos_sb != 0 && (B & 7) == 0) {
      const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
      b = (j / H) * 8 + x;
      h = j % H;
    }
  }
  const int64_t bh = (int64_t)b * H + h;
  const float qscale = a.scale * LOG2E;

  // ---- window geometry -------------------------------------------------------------------------
  const bool ring = a.mode == NHA_DECODE_RING;
  int slot = -1, nvalid = W, cnt = 0;
  if (ring) {
    cnt = a.count[b];
    slot = cnt % W;
    nvalid = cnt + 1 < W ? cnt + 1 : W;
    if (a.count_next && h == 0 && tid == 0) a.count_next[b] = cnt + 1;
  }
  const bf16_t* kwin = (const bf16_t*)(ring ? a.ring_k : a.win_k) + ((int64_t)b * W * H + h) * D;
  const bf16_t* vwin = (const bf16_t*)(ring ? a.ring_v : a.win_v) + ((int64_t)b * W * H + h) * D;
  const bf16_t* knew = ring ? (const bf16_t*)a.k_new + bh * D : nullptr;
  const bf16_t* vnew = ring ? (const bf16_t*)a.v_new + bh * D : nullptr;
  const int nblk = (nvalid + 31) >> 5;

  // rows past the valid range are clamped to the last valid row (finite data); their logits are
  // masked below.  Ring row `slot` is the new token, read from k_new / v_new.
  // Unconditional (uniform control flow keeps the load counters exact, so a block's data is
  // awaited while the next block stays in flight): rows past the valid range are clamped to the
  // last valid row (finite data, one cache line) and their logits are masked below.  Ring row
  // `slot` is the new token, read from k_new / v_new.
  const uint32_t rstride = (uint32_t)H * D;
  auto load_block = [&](uint4(&kr)[2 * KS], uint4(&vr)[NVT], int blk) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int w = 32 * blk + 16 * t + l16;
      w = w < nvalid ? w : nvalid - 1;
      const bf16_t* pw = kwin + (uint32_t)w * rstride;
      const bf16_t* row = (w == slot ? knew : pw) + 8 * qd;
#pragma unroll
      for (int j = 0; j < KS; ++j) kr[t * KS + j] = ld16_stream(row + 32 * j);
    }
#pragma unroll
    for (int u = 0; u < NVT; ++u) {
      int w = 32 * blk + u * RV + lane / LV;
      w = w < nvalid ? w : nvalid - 1;
      const bf16_t* pw = vwin + (uint32_t)w * rstride;
      const bf16_t* row = (w == slot ? vnew : pw) + 8 * (lane % LV);
      vr[u] = ld16_stream(row);
    }
  };

  // ================= slot branch (all waves; three LDS-only barriers) ============================
  auto slot_branch = [&]() {
    const int cm = lane % LM, rm = lane / LM;
    const int m0 = cm * 8;
    // Load order = queue order: the popped entry and the queries first (small, and the only loads
    // on the dependent chain count -> slot -> popped row), then all state rows of this lane.
    // Nothing below waits on more than its own data, so the state rows of every workgroup are
    // queued before any workgroup starts streaming its window.
    bool has_pop = true;
    const bf16_t *kpop, *vpop, *gpop, *spop = nullptr;
    if (ring) {
      has_pop = cnt >= W;
      const int64_t row = ((int64_t)b * W + slot) * H + h;
      kpop = (const bf16_t*)a.ring_kg + row * D;
      vpop = (const bf16_t*)a.ring_v + row * D;
      gpop = (const bf16_t*)a.ring_g + row * M;
    } else {
      kpop = (const bf16_t*)a.k_pop + bh * D;
      vpop = (const bf16_t*)a.v_pop + bh * D;
      gpop = (const bf16_t*)a.g_pop + bh * M;
      if (a.s_pop) spop = (const bf16_t*)a.s_pop + bh * M;
    }
    constexpr int NPM = (M + NT - 1) / NT, NPD = (D + NT - 1) / NT, NPQ = (G * D + NT - 1) / NT;
    bf16_t rg[NPM], rs[NPM], rk[NPD], rv[NPD], rq[NPQ];
#pragma unroll
    for (int i = 0; i < NPM; ++i) {
      const int x = tid + i * NT;
      rg[i] = (has_pop && x < M) ? gpop[x] : (bf16_t)0;
      rs[i] = (has_pop && spop && x < M) ? spop[x] : (bf16_t)0;
    }
#pragma unroll
    for (int i = 0; i < NPD; ++i) {
      const int x = tid + i * NT;
      rk[i] = (has_pop && x < D) ? kpop[x] : (bf16_t)0;
      rv[i] = (has_pop && x < D) ? vpop[x] : (bf16_t)0;
    }
#pragma unroll
    for (int i = 0; i < NPQ; ++i) {
      const int x = tid + i * NT;
      const int gq = x / D, kk = x - gq * D;
      rq[i] = (x < G * D && gq < NG) ? ((const bf16_t*)a.q)[((int64_t)b * HQ + h * NG + gq) * D + kk] : (bf16_t)0;
    }
    __builtin_amdgcn_sched_barrier(0);
    float hkr[NIK][8], hvr[NIV][8];
    const float* hkin = a.hk_in ? a.hk_in + bh * D * M + m0 : nullptr;
    float* hkout = a.hk_out ? a.hk_out + bh * D * M + m0 : nullptr;
    const float* hvin = a.hv_in ? a.hv_in + bh * M * D + (lane % LV) * 8 : nullptr;
    float* hvout = a.hv_out ? a.hv_out + bh * M * D + (lane % LV) * 8 : nullptr;
#pragma unroll
    for (int i = 0; i < NIK; ++i) {
      const int kk = (i * NW + wave) * RM + rm;
      if (hkin) {
        Elem<float>::ld8(hkin + (int64_t)kk * M, hkr[i]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) hkr[i][e] = 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < NIV; ++i) {
      const int m = (i * NW + wave) * RV + lane / LV;
      if (hvin) {
        Elem<float>::ld8(hvin + (int64_t)m * D, hvr[i]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) hvr[i][e] = 0.f;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NPM; ++i) {
      const int x = tid + i * NT;
      if (x < M) {
        float e = 1.f, sv = 0.f;
        if (has_pop) {
          e = expf(bf16_to_f32(rg[i]));
          sv = spop ? bf16_to_f32(rs[i]) : 1.f - e;
        }
        eg[x] = e;
        sg[x] = sv;
      }
    }
#pragma unroll
    for (int i = 0; i < NPD; ++i) {
      const int x = tid + i * NT;
      if (x < D) {
        kp[x] = bf16_to_f32(rk[i]);
        vp[x] = bf16_to_f32(rv[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < NPQ; ++i) {
      const int x = tid + i * NT;
      if (x < G * D) qs[x] = bf16_to_f32(rq[i]) * qscale;
    }
    lds_barrier();
    // the popped entry is in LDS (its loads have returned): the new token may take its ring slot
    if (ring) {
      const int64_t row = ((int64_t)b * W + slot) * H + h;
      if (tid < D / 8) {
        reinterpret_cast<uint4*>((bf16_t*)a.ring_k + row * D)[tid] = reinterpret_cast<const uint4*>((const bf16_t*)a.k_new + bh * D)[tid];
        reinterpret_cast<uint4*>((bf16_t*)a.ring_kg + row * D)[tid] = reinterpret_cast<const uint4*>((const bf16_t*)a.kg_new + bh * D)[tid];
      } else if (tid >= 64 && tid < 64 + D / 8) {
        reinterpret_cast<uint4*>((bf16_t*)a.ring_v + row * D)[tid - 64] = reinterpret_cast<const uint4*>((const bf16_t*)a.v_new + bh * D)[tid - 64];
      } else if (tid >= 96 && tid < 96 + M / 8) {
        reinterpret_cast<uint4*>((bf16_t*)a.ring_g + row * M)[tid - 96] = reinterpret_cast<const uint4*>((const bf16_t*)a.g_new + bh * M)[tid - 96];
      }
    }
    // ---- hk <- hk*exp(g) + k s^T ; slot logits ok[g][m] = scale q . hk[:,m] --------------------
    {
      float eg8[8], s8[8], acc[G][8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        eg8[e] = eg[m0 + e];
        s8[e] = sg[m0 + e];
      }
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
#pragma unroll
      for (int i = 0; i < NIK; ++i) {
        const int kk = (i * NW + wave) * RM + rm;
        const float kv = kp[kk];
#pragma unroll
        for (int e = 0; e < 8; ++e) hkr[i][e] = hkr[i][e] * eg8[e] + kv * s8[e];
        if (hkout) Elem<float>::st8(hkout + (int64_t)kk * M, hkr[i]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float qg = qs[g * D + kk];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] += qg * hkr[i][e];
        }
      }
#pragma unroll
      for (int mask = LM; mask < 64; mask <<= 1)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], mask, 64);
      if (rm == 0)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int e = 0; e < 8; ++e) part[(wave * G + g) * MV + m0 + e] = acc[g][e];
    }
    lds_barrier();
    // slot softmax statistics, one head per wave at a time (M == 64: one slot per lane)
    for (int g = wave; g < G; g += NW) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) v += part[(w * G + g) * MV + lane];
      const float mx = wave_max(v);
      const float e = fexp2(v - mx);
      const float sum = wave_sum(e);
      ok[g * M + lane] = e;
      if (lane == 0) {
        ms[g] = mx;
        ms[16 + g] = sum;
      }
    }
    lds_barrier();
    // ---- hv <- hv*exp(g) + s v^T ; slot read ---------------------------------------------------
    {
      const int v0 = (lane % LV) * 8;
      float acc[G][8], vp8[8];
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) vp8[e] = vp[v0 + e];
#pragma unroll
      for (int i = 0; i < NIV; ++i) {
        const int m = (i * NW + wave) * RV + lane / LV;
        const float egm = eg[m], sm = sg[m];
#pragma unroll
        for (int e = 0; e < 8; ++e) hvr[i][e] = hvr[i][e] * egm + sm * vp8[e];
        if (hvout) Elem<float>::st8(hvout + (int64_t)m * D, hvr[i]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float p = ok[g * M + m];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] += p * hvr[i][e];
        }
      }
#pragma unroll
      for (int mask = LV; mask < 64; mask <<= 1)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], mask, 64);
      if (lane / LV == 0)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int e = 0; e < 8; ++e) part[(wave * G + g) * MV + v0 + e] = acc[g][e];
    }
  };

  // ================= window branch: one pass, 32 keys per block, blocks wave, wave+NW, ... =======
  auto window_branch = [&]() {
    // cos / sin pieces of block `blk` for this lane's two rows -> the wave's LDS area
    const bf16_t* ctab = ROT ? (const bf16_t*)a.cos + (int64_t)b * a.cos_sb : nullptr;
    const bf16_t* stab = ROT ? (const bf16_t*)a.sin + (int64_t)b * a.cos_sb : nullptr;
    auto request_cs = [&](int blk) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        int w = 32 * blk + 16 * t + l16;
        w = w < nvalid ? w : nvalid - 1;
        const uint32_t off = ((uint32_t)w * (uint32_t)a.cos_sw + 8 * qd) * 2;
#pragma unroll
        for (int j = 0; j < KS; ++j) {
          g2l16(ctab, off + 64 * j, cs_lds + ((0 * 2 + t) * KS + j) * 1024);
          g2l16(stab, off + 64 * j, cs_lds + ((1 * 2 + t) * KS + j) * 1024);
        }
      }
    };
    auto cs_piece = [&](int tab, int t, int j) -> uint4 {
      const u32x4 x = *reinterpret_cast<const NHA_LDS u32x4*>(CS + ((tab * 2 + t) * KS + j) * 1024 + lane * 16);
      return make_uint4(x[0], x[1], x[2], x[3]);
    };
    // window-query B fragments: lane (head l%16, piece l/16) of each 32-wide k-step
    bf16x8 qf[KS];
    {
      uint4 qx[KS];
      const bf16_t* qsrc = ROT ? (const bf16_t*)a.q : (const bf16_t*)a.sq;
#pragma unroll
      for (int j = 0; j < KS; ++j) {
        qx[j] = make_uint4(0, 0, 0, 0);
        if (l16 < NG) qx[j] = *reinterpret_cast<const uint4*>(qsrc + ((int64_t)b * HQ + h * NG + l16) * D + 32 * j + 8 * qd);
      }
      if (ROT) {   // the query's own position is the last row of the tables
        const bf16_t* cq = ctab + (int64_t)(W - 1) * a.cos_sw + 8 * qd;
        const bf16_t* sq_ = stab + (int64_t)(W - 1) * a.cos_sw + 8 * qd;
#pragma unroll
        for (int j = 0; j < KS / 2; ++j) {
          const uint4 ca = *reinterpret_cast<const uint4*>(cq + 32 * j), sa = *reinterpret_cast<const uint4*>(sq_ + 32 * j);
          const uint4 cb = *reinterpret_cast<const uint4*>(cq + 32 * (j + KS / 2)), sb = *reinterpret_cast<const uint4*>(sq_ + 32 * (j + KS / 2));
          rope8(qx[j], qx[j + KS / 2], ca, sa, cb, sb);
        }
      }
#pragma unroll
      for (int j = 0; j < KS; ++j) qf[j] = as_bf16x8(qx[j]);
    }
    // register buffers of 32-key blocks per wave: two at head sizes up to 128 (32 KB in flight), one at 256
    // (a block is 32 KB there, and twice the waves per workgroup keep as many bytes in flight per CU)
    constexpr int NBUF = D > 128 ? 1 : 2;
    uint4 kr0[2 * KS], vr0[NVT], kr1[NBUF == 2 ? 2 * KS : 1], vr1[NBUF == 2 ? NVT : 1];
    // issue order is the consumption order (the waits count loads still in flight)
    __builtin_amdgcn_sched_barrier(0);
    if (ROT) request_cs(wave);
    __builtin_amdgcn_sched_barrier(0);
    load_block(kr0, vr0, wave);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NBUF == 2) {
      load_block(reinterpret_cast<uint4(&)[2 * KS]>(kr1), reinterpret_cast<uint4(&)[NVT]>(vr1), wave + NW);
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x4 O[NVT];
#pragma unroll
    for (int vt = 0; vt < NVT; ++vt) O[vt] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float mrun = -INFINITY, lsum = 0.f;

    // consumes the block held in (kr, vr) and refills the registers as soon as they are free
    auto process = [&](uint4(&kr)[2 * KS], uint4(&vr)[NVT], int blk) {
      if (ROT) {
        // The pieces of this block were requested after the keys of this block and before the refill of the other
        // register buffer: waiting for the keys (the compiler's wait on kr) does not cover them.  Everything up to
        // that refill has landed once at most one block of loads is in flight (the first block's pieces were requested
        // ahead of both buffers: covered as well).  Then rotate in place and ask for the next block's pieces.
        if constexpr (NBUF == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * KS + NVT) : "memory");
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < KS / 2; ++j)
            rope8(kr[t * KS + j], kr[t * KS + j + KS / 2], cs_piece(0, t, j), cs_piece(1, t, j), cs_piece(0, t, j + KS / 2),
                  cs_piece(1, t, j + KS / 2));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the pieces have left LDS before new ones may land
        __builtin_amdgcn_sched_barrier(0);
        request_cs(blk + NW);
        __builtin_amdgcn_sched_barrier(0);
      }
      f32x4 S0 = {0.f, 0.f, 0.f, 0.f}, S1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < KS; ++j) S0 = mfma16(as_bf16x8(kr[j]), qf[j], S0);
#pragma unroll
      for (int j = 0; j < KS; ++j) S1 = mfma16(as_bf16x8(kr[KS + j]), qf[j], S1);
#pragma unroll
      for (int u = 0; u < NVT; ++u) {
        const u32x4 x = {vr[u].x, vr[u].y, vr[u].z, vr[u].w};
        *reinterpret_cast<NHA_LDS u32x4*>(X + (u * RV + lane / LV) * LDT + 8 * (lane % LV)) = x;
      }
      // pin the refill here: right after its registers are free, NBUF blocks ahead of its use
      __builtin_amdgcn_sched_barrier(0);
      load_block(kr, vr, blk + NBUF * NW);
      __builtin_amdgcn_sched_barrier(0);
      // S^T rows of this lane: keys 32*blk + 4*qd + r (S0) and + 16 (S1), head l16
      const int wb = 32 * blk + 4 * qd;
      float s[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[r] = wb + r < nvalid ? S0[r] * qscale : -INFINITY;
        s[4 + r] = wb + 16 + r < nvalid ? S1[r] * qscale : -INFINITY;
      }
      float mx = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
      mx = max_over_rows(mx);
      const float mnew = fmaxf(mrun, mx);
      const float alpha = fexp2(mrun - mnew);
      mrun = mnew;
      float ps = 0.f;
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        s[r] = fexp2(s[r] - mnew);
        ps += s[r];
      }
      lsum = lsum * alpha + ps;
      bf16x8 P;
#pragma unroll
      for (int r = 0; r < 8; ++r) P[r] = (__bf16)s[r];
#pragma unroll
      for (int vt = 0; vt < NVT; ++vt) {
        O[vt] *= alpha;
        O[vt] = mfma16(lds_frag_tr(X, LDT, 16 * vt, lane), P, O[vt]);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if constexpr (NBUF == 2) {
      for (int blk = wave; blk < nblk; blk += 2 * NW) {
        process(kr0, vr0, blk);
        process(reinterpret_cast<uint4(&)[2 * KS]>(kr1), reinterpret_cast<uint4(&)[NVT]>(vr1), blk + NW);   // past the end: a fully masked block, contributes nothing
      }
    } else {
      for (int blk = wave; blk < nblk; blk += NW) process(kr0, vr0, blk);
    }
    lsum = sum_over_rows(lsum);
    if (qd == 0) {
      wm[wave * 16 + l16] = mrun;
      wl[wave * 16 + l16] = lsum;
    }
    // O^T[v = 16*vt + 4*qd + r][head l16] -> wave-private fp32 [G][D] over this wave's V tile
    lfloat* Ow = (lfloat*)(NHA_LDS void*)X;
    if (l16 < G) {
#pragma unroll
      for (int vt = 0; vt < NVT; ++vt) *reinterpret_cast<NHA_LDS f32x4*>(Ow + l16 * D + 16 * vt + 4 * qd) = O[vt];
    }
  };

  slot_branch();
  window_branch();

  // ---- merge: slots + window partials under one softmax ----------------------------------------
  lds_barrier();
  const lfloat* Oall = (const lfloat*)(NHA_LDS void*)(ms + 32);
  constexpr int OWS = 32 * LDT / 2;   // floats between the tiles of consecutive waves
  for (int i = tid; i < G * D; i += NT) {
    const int g = i / D, v = i - g * D;
    if (g < NG) {
      const float m_s = ms[g];
      float mt = m_s;
#pragma unroll
      for (int w = 0; w < NW; ++w) mt = fmaxf(mt, wm[w * 16 + g]);
      const float cs = fexp2(m_s - mt);
      float num = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) num += part[(w * G + g) * MV + v];
      num *= cs;
      float den = ms[16 + g] * cs;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const float cw = fexp2(wm[w * 16 + g] - mt);
        num += Oall[w * OWS + g * D + v] * cw;
        den += wl[w * 16 + g] * cw;
      }
      ((bf16_t*)a.o)[((int64_t)b * HQ + h * NG + g) * D + v] = f32_to_bf16(num / den);
    }
  }
}

#ifndef NHA_DEC_NW
#define NHA_DEC_NW 2
#endif

template <int D, int G, bool ROT>
int launch(const NhaDecodeArgs* a) {
  constexpr int NW = D > 128 ? 4 : NHA_DEC_NW;
  const size_t lds = lds_bytes_for(D, G, NW, ROT);
  static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
  if (!configured && lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)decode_mfma_kernel<D, G, NW, ROT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("decode: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  hipLaunchKernelGGL((decode_mfma_kernel<D, G, NW, ROT>), dim3(a->B * a->H), dim3(64 * NW), lds, (hipStream_t)a->stream, *a);
  NHA_CHECK_LAUNCH("nha_decode_step");
  return NHA_OK;
}

template <int D, bool ROT>
int dispatch(const NhaDecodeArgs* a, int G) {
  switch (G) {
    case 1: return launch<D, 1, ROT>(a);
    case 2: return launch<D, 2, ROT>(a);
    case 4: return launch<D, 4, ROT>(a);
    default: return launch<D, 8, ROT>(a);
  }
}

}  // namespace

bool decode_mfma_supported(const NhaDecodeArgs* a) {
  if (a->dtype != NHA_DTYPE_BF16 || a->K != a->V || (a->K != 64 && a->K != 128 && a->K != 256)) return false;
  if (a->K == 256 && a->cos) return false;   // the rotary tables of a block do not fit beside the V tiles at this head size
  if (a->mode != NHA_DECODE_WINDOW && a->mode != NHA_DECODE_RING) return false;
  // either a pre-rotated query, or (window mode) cos / sin tables whose rows are 16-byte aligned pieces
  const bool rot = a->cos != nullptr;
  if (rot) {
    if (a->mode != NHA_DECODE_WINDOW || !a->sin || a->sq) return false;
    if (a->cos_sw % 8 != 0 || a->cos_sb % 8 != 0 || ((uintptr_t)a->cos & 15) || ((uintptr_t)a->sin & 15)) return false;
    if (a->cos_sw * (int64_t)a->W >= ((int64_t)1 << 30)) return false;
  } else if (!a->sq) {
    return false;
  }
  const int NG = a->HQ / a->H;
  // window rows are addressed with 32-bit element offsets
  return NG <= 8 && a->M == MS && (int64_t)a->W * a->H * a->K < ((int64_t)1 << 31);
}

int decode_mfma_impl(const NhaDecodeArgs* a) {
  const int NG = a->HQ / a->H;
  int G = 1;
  while (G < NG) G <<= 1;
  if (a->cos) return a->K == 64 ? dispatch<64, true>(a, G) : dispatch<128, true>(a, G);
  if (a->K == 256) return dispatch<256, false>(a, G);
  return a->K == 64 ? dispatch<64, false>(a, G) : dispatch<128, false>(a, G);
}

}  // namespace nha
