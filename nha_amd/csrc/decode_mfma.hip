// Matrix-core decode step for gfx950: bf16, K == V == D in {64,128}, window or ring mode with a
// pre-rotated window query, up to 8 query heads per kv-head.
//
// Same work split as decode.hip (one workgroup per (sequence, kv-head), state and window read
// once), but the window is streamed ONCE in 32-key blocks by each of the four waves:
//   S^T[key][head] = K Q^T       A = 16 key rows loaded from HBM straight into the A-operand layout
//                                (lane l: row l%16, 16-byte piece l/16 of each 64-byte k-step)
//   O^T[v][head]  += V^T P^T     V rows go HBM -> registers -> a wave-private LDS tile and come back
//                                transposed (ds_read_b64_tr_b16); P leaves the accumulator layout of
//                                S^T as the B operand with no lane movement
// so a lane owns one query head and the online softmax needs two cross-lane steps per block.  The
// per-key VALU work of the two-sweep kernel (convert, 8 FMA per head, row reductions) disappears
// and each wave keeps two 32-key blocks (32 KB) of loads in flight.  Slot state update, slot
// logits and slot read stay fp32 VALU (nha_fla/ops/nha/fused_recurrent.py:305, :342-349, :416);
// slots and the four window partials are merged at the end under one softmax.
#include "common.h"

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

__host__ __device__ constexpr int imax(int a, int b) { return a > b ? a : b; }

static size_t lds_bytes_for(int D, int G, int M) {
  const size_t fl = (size_t)2 * M + 2 * D + (size_t)G * D + (size_t)G * M + (size_t)4 * G * imax(M, D) + 64 + 64 + 32;
  return fl * 4 + (size_t)4 * 32 * (D + 16) * 2;
}

template <int D, int G>
__global__ __launch_bounds__(256, 2) void decode_mfma_kernel(const NhaDecodeArgs a, const int LM) {
  constexpr int LDT = D + 16;   // bf16 row stride of a V tile
  constexpr int KS = D / 32;    // MFMA k-steps over the head dim
  constexpr int NVT = D / 16;   // 16-row blocks of O^T == 16-byte V loads per lane and block
  constexpr int LV = D / 8;     // lanes per V / hv row
  constexpr int RV = 64 / LV;   // rows per wave-wide load
  extern __shared__ __align__(16) float lds_raw[];
  const int M = a.M, W = a.W, H = a.H, HQ = a.HQ;
  const int NG = HQ / H;
  const int MV = M > D ? M : D;
  float* eg = lds_raw;
  float* sg = eg + M;
  float* kp = sg + M;
  float* vp = kp + D;
  float* qs = vp + D;              // [G][D] slot-branch query, scale * log2(e) folded in
  float* ok = qs + G * D;          // [G][M] slot logits, then slot probabilities
  float* part = ok + G * M;        // [4][G][MV] per-wave partial sums
  float* wm = part + 4 * G * MV;   // [4][16] per-wave window max (log2 units)
  float* wl = wm + 64;             // [4][16] per-wave window sum
  float* ms = wl + 64;             // [16] slot max, [16] slot sum
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, qd = lane >> 4;
  lbf16* X = (lbf16*)(NHA_LDS void*)(ms + 32) + wave * 32 * LDT;   // wave-private V tile [32][LDT]
  const int b = blockIdx.x / H, h = blockIdx.x % H;
  const int64_t bh = (int64_t)b * H + h;
  const float qscale = a.scale * LOG2E;

  // ---- popped entry and window geometry ------------------------------------------------------
  const bool ring = a.mode == NHA_DECODE_RING;
  int slot = -1, nvalid = W;
  bool has_pop = true;
  const bf16_t *kpop, *vpop, *gpop, *spop = nullptr;
  if (ring) {
    const int c = a.count[b];
    slot = c % W;
    has_pop = c >= W;
    nvalid = c + 1 < W ? c + 1 : W;
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
  const bf16_t* kwin = (const bf16_t*)(ring ? a.ring_k : a.win_k) + ((int64_t)b * W * H + h) * D;
  const bf16_t* vwin = (const bf16_t*)(ring ? a.ring_v : a.win_v) + ((int64_t)b * W * H + h) * D;
  const bf16_t* knew = ring ? (const bf16_t*)a.k_new + bh * D : nullptr;
  const bf16_t* vnew = ring ? (const bf16_t*)a.v_new + bh * D : nullptr;
  const int64_t rstride = (int64_t)H * D;
#ifdef NHA_DEC_NOWIN
  const int nblk = 0;
#else
  const int nblk = (nvalid + 31) >> 5;
#endif

  // rows past the valid range are clamped to the last valid row (finite data); their logits are
  // masked below.  Ring row `slot` is the new token, read from k_new / v_new.
  auto load_block = [&](uint4(&kr)[2 * KS], uint4(&vr)[NVT], int blk) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int w = 32 * blk + 16 * t + l16;
      w = w < nvalid ? w : nvalid - 1;
      const bf16_t* row = (w == slot ? knew : kwin + (int64_t)w * rstride) + 8 * qd;
#pragma unroll
      for (int j = 0; j < KS; ++j) kr[t * KS + j] = *reinterpret_cast<const uint4*>(row + 32 * j);
    }
#pragma unroll
    for (int u = 0; u < NVT; ++u) {
      int w = 32 * blk + u * RV + lane / LV;
      w = w < nvalid ? w : nvalid - 1;
      const bf16_t* row = (w == slot ? vnew : vwin + (int64_t)w * rstride) + 8 * (lane % LV);
      vr[u] = *reinterpret_cast<const uint4*>(row);
    }
  };

  // ---- phase 0: small operands -> LDS; first two window blocks of this wave go in flight ------
  for (int i = tid; i < M; i += 256) {
    float e = 1.f, s = 0.f;
    if (has_pop) {
      e = expf(bf16_to_f32(gpop[i]));
      s = spop ? bf16_to_f32(spop[i]) : 1.f - e;
    }
    eg[i] = e;
    sg[i] = s;
  }
  for (int i = tid; i < D; i += 256) {
    kp[i] = has_pop ? bf16_to_f32(kpop[i]) : 0.f;
    vp[i] = has_pop ? bf16_to_f32(vpop[i]) : 0.f;
  }
  for (int i = tid; i < G * D; i += 256) {
    const int gq = i / D, kk = i - gq * D;
    qs[i] = gq < NG ? bf16_to_f32(((const bf16_t*)a.q)[((int64_t)b * HQ + h * NG + gq) * D + kk]) * qscale : 0.f;
  }
  // window-query B fragments: lane (head l%16, piece l/16) of each 32-wide k-step
  bf16x8 qf[KS];
#pragma unroll
  for (int j = 0; j < KS; ++j) {
    uint4 x = make_uint4(0, 0, 0, 0);
    if (l16 < NG) x = *reinterpret_cast<const uint4*>((const bf16_t*)a.sq + ((int64_t)b * HQ + h * NG + l16) * D + 32 * j + 8 * qd);
    qf[j] = as_bf16x8(x);
  }
  uint4 kr0[2 * KS], vr0[NVT], kr1[2 * KS], vr1[NVT];
  if (wave < nblk) load_block(kr0, vr0, wave);
  if (wave + 4 < nblk) load_block(kr1, vr1, wave + 4);
  lds_barrier();

  // ring mode: the popped entry now lives in LDS; store the new token in its slot
  if (ring) {
    const int64_t row = ((int64_t)b * W + slot) * H + h;
    if (tid < D / 8) {
      reinterpret_cast<uint4*>((bf16_t*)a.ring_k + row * D)[tid] = reinterpret_cast<const uint4*>((const bf16_t*)a.k_new + bh * D)[tid];
    } else if (tid >= 64 && tid < 64 + D / 8) {
      reinterpret_cast<uint4*>((bf16_t*)a.ring_kg + row * D)[tid - 64] = reinterpret_cast<const uint4*>((const bf16_t*)a.kg_new + bh * D)[tid - 64];
    } else if (tid >= 128 && tid < 128 + D / 8) {
      reinterpret_cast<uint4*>((bf16_t*)a.ring_v + row * D)[tid - 128] = reinterpret_cast<const uint4*>((const bf16_t*)a.v_new + bh * D)[tid - 128];
    } else if (tid >= 192 && tid < 192 + M / 8) {
      reinterpret_cast<uint4*>((bf16_t*)a.ring_g + row * M)[tid - 192] = reinterpret_cast<const uint4*>((const bf16_t*)a.g_new + bh * M)[tid - 192];
    }
  }

  // ---- phase 1: hk <- hk*exp(g) + k s^T ; slot logits ok[g][m] = scale q . hk[:,m] ------------
  {
    const int cm = lane % LM, rm = lane / LM, RM = 64 / LM;
    const int m0 = cm * 8;
    const bool act = m0 < M;
    float eg8[8], s8[8], acc[G][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      eg8[e] = act ? eg[m0 + e] : 0.f;
      s8[e] = act ? sg[m0 + e] : 0.f;
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    if (act) {
#ifdef NHA_DEC_NOSTATE
      const float* hin = nullptr;
      float* hout = nullptr;
#else
      const float* hin = a.hk_in ? a.hk_in + bh * D * M + m0 : nullptr;
      float* hout = a.hk_out ? a.hk_out + bh * D * M + m0 : nullptr;
#endif
#pragma unroll 4
      for (int kk = wave * RM + rm; kk < D; kk += 4 * RM) {
        float hr[8];
        if (hin) {
          Elem<float>::ld8(hin + (int64_t)kk * M, hr);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) hr[e] = 0.f;
        }
        const float kv = kp[kk];
#pragma unroll
        for (int e = 0; e < 8; ++e) hr[e] = hr[e] * eg8[e] + kv * s8[e];
        if (hout) Elem<float>::st8(hout + (int64_t)kk * M, hr);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float qg = qs[g * D + kk];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] += qg * hr[e];
        }
      }
    }
    for (int mask = LM; mask < 64; mask <<= 1)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], mask, 64);
    if (rm == 0 && act)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) part[(wave * G + g) * MV + m0 + e] = acc[g][e];
  }
  lds_barrier();
  for (int i = tid; i < G * M; i += 256) {
    const int g = i / M, m = i - g * M;
    ok[i] = part[g * MV + m] + part[(G + g) * MV + m] + part[(2 * G + g) * MV + m] + part[(3 * G + g) * MV + m];
  }
  lds_barrier();
  // slot softmax statistics: ok <- 2^(ok - max), ms[g] = max, ms[16+g] = sum
  for (int g = wave; g < G; g += 4) {
    float mx = -INFINITY;
    for (int i = lane; i < M; i += 64) mx = fmaxf(mx, ok[g * M + i]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int i = lane; i < M; i += 64) {
      const float e = fexp2(ok[g * M + i] - mx);
      ok[g * M + i] = e;
      sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) {
      ms[g] = mx;
      ms[16 + g] = sum;
    }
  }
  lds_barrier();

  // ---- phase 2: hv <- hv*exp(g) + s v^T ; slot read partials ---------------------------------
  {
    const int cv = lane % LV, rv = lane / LV;
    const int v0 = cv * 8;
    float acc[G][8], vp8[8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) vp8[e] = vp[v0 + e];
#ifdef NHA_DEC_NOSTATE
    const float* hin = nullptr;
    float* hout = nullptr;
#else
    const float* hin = a.hv_in ? a.hv_in + bh * M * D + v0 : nullptr;
    float* hout = a.hv_out ? a.hv_out + bh * M * D + v0 : nullptr;
#endif
#pragma unroll 4
    for (int m = wave * RV + rv; m < M; m += 4 * RV) {
      float hr[8];
      if (hin) {
        Elem<float>::ld8(hin + (int64_t)m * D, hr);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) hr[e] = 0.f;
      }
      const float egm = eg[m], sm = sg[m];
#pragma unroll
      for (int e = 0; e < 8; ++e) hr[e] = hr[e] * egm + sm * vp8[e];
      if (hout) Elem<float>::st8(hout + (int64_t)m * D, hr);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float p = ok[g * M + m];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] += p * hr[e];
      }
    }
    for (int mask = LV; mask < 64; mask <<= 1)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], mask, 64);
    if (rv == 0)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) part[(wave * G + g) * MV + v0 + e] = acc[g][e];
  }

  // ---- phase 3: window, one pass, 32 keys per block, this wave's blocks wave, wave+4, ... ------
  f32x4 O[NVT];
#pragma unroll
  for (int vt = 0; vt < NVT; ++vt) O[vt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float mrun = -INFINITY, lsum = 0.f;

  auto process = [&](uint4(&kr)[2 * KS], uint4(&vr)[NVT], int blk) {
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
    if (blk + 8 < nblk) load_block(kr, vr, blk + 8);
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
  };

  for (int blk = wave; blk < nblk; blk += 8) {
    process(kr0, vr0, blk);
    if (blk + 4 < nblk) process(kr1, vr1, blk + 4);
  }

  // ---- merge: slots + four window partials under one softmax ----------------------------------
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
  lds_barrier();
  const lfloat* Oall = (const lfloat*)(NHA_LDS void*)(ms + 32);
  constexpr int OWS = 32 * LDT / 2;   // floats between the tiles of consecutive waves
  for (int i = tid; i < G * D; i += 256) {
    const int g = i / D, v = i - g * D;
    if (g < NG) {
      const float m_s = ms[g];
      float mt = m_s;
#pragma unroll
      for (int w = 0; w < 4; ++w) mt = fmaxf(mt, wm[w * 16 + g]);
      const float cs = fexp2(m_s - mt);
      float num = (part[g * MV + v] + part[(G + g) * MV + v] + part[(2 * G + g) * MV + v] + part[(3 * G + g) * MV + v]) * cs;
      float den = ms[16 + g] * cs;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float cw = fexp2(wm[w * 16 + g] - mt);
        num += Oall[w * OWS + g * D + v] * cw;
        den += wl[w * 16 + g] * cw;
      }
      ((bf16_t*)a.o)[((int64_t)b * HQ + h * NG + g) * D + v] = f32_to_bf16(num / den);
    }
  }
}

template <int D, int G>
int launch(const NhaDecodeArgs* a) {
  const size_t lds = lds_bytes_for(D, G, a->M);
  static size_t configured = 0;
  if (lds > configured) {
    hipError_t e = hipFuncSetAttribute((const void*)decode_mfma_kernel<D, G>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      set_error("decode: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = lds;
  }
  hipLaunchKernelGGL((decode_mfma_kernel<D, G>), dim3(a->B * a->H), dim3(256), lds, (hipStream_t)a->stream, *a,
                     next_pow2_i(a->M / 8));
  NHA_CHECK_LAUNCH("nha_decode_step");
  return NHA_OK;
}

template <int D>
int dispatch(const NhaDecodeArgs* a, int G) {
  switch (G) {
    case 1: return launch<D, 1>(a);
    case 2: return launch<D, 2>(a);
    case 4: return launch<D, 4>(a);
    default: return launch<D, 8>(a);
  }
}

}  // namespace

bool decode_mfma_supported(const NhaDecodeArgs* a) {
  if (a->dtype != NHA_DTYPE_BF16 || a->K != a->V || (a->K != 64 && a->K != 128)) return false;
  if (a->mode != NHA_DECODE_WINDOW && a->mode != NHA_DECODE_RING) return false;
  if (!a->sq || a->cos) return false;
  const int NG = a->HQ / a->H;
  if (NG > 8 || a->M % 8 || a->M > 512) return false;
  int G = 1;
  while (G < NG) G <<= 1;
  return lds_bytes_for(a->K, G, a->M) <= 64 * 1024;
}

int decode_mfma_impl(const NhaDecodeArgs* a) {
  const int NG = a->HQ / a->H;
  int G = 1;
  while (G < NG) G <<= 1;
  return a->K == 64 ? dispatch<64>(a, G) : dispatch<128>(a, G);
}

}  // namespace nha
