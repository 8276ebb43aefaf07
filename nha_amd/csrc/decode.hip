// Single-token NHA decode step for gfx950: one launch, one workgroup per (sequence, kv-head)
// serving all HQ/H query heads, so the fp32 slot state and the W-row K/V window are each read
// from HBM exactly once per step.  HBM-bound: every global access below is a 16- or 32-byte
// per-lane vector access over contiguous rows.
//
// Semantics follow nha_fla/ops/nha/fused_recurrent.py:228-428 (decode k/v kernels: state write
// :305/:416, fused softmax over [M | W] :342-349, rotate-half pairing :309-329) and :47-149
// (caller-supplied window logits).  fp32 math on bf16/fp32 loads, state fp32.
#include "common.h"
#include <stdlib.h>

namespace nha {

namespace {

struct Lds {
  float *eg, *s, *kp, *vp, *q, *sq, *ok, *inv, *part, *logit;
};

template <int G>
__device__ __forceinline__ Lds carve(float* base, int K, int V, int M, int W) {
  Lds l;
  float* p = base;
  l.eg = p; p += M;
  l.s = p; p += M;
  l.kp = p; p += K;
  l.vp = p; p += V;
  l.q = p; p += G * K;
  l.sq = p; p += G * K;
  l.ok = p; p += G * M;
  l.inv = p; p += 16;
  const int mv = M > V ? M : V;
  l.part = p; p += 4 * G * mv;
  l.logit = p;
  return l;
}

// sum over the LK lanes (a power of two) that share one row: DPP row operations inside a 16-lane
// row (full-rate VALU), cross-row butterflies beyond it
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row_group_sum(float v, int LK) {
  if (LK > 1) v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
  if (LK > 2) v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
  if (LK > 4) v = dpp_add<0x141>(v);   // row_half_mirror
  if (LK > 8) v = dpp_add<0x140>(v);   // row_mirror
  if (LK > 16) v += __shfl_xor(v, 16, 64);
  if (LK > 32) v += __shfl_xor(v, 32, 64);
  return v;
}

static size_t lds_floats(int G, int K, int V, int M, int W) {
  const int mv = M > V ? M : V;
  return (size_t)2 * M + K + V + (size_t)2 * G * K + (size_t)G * M + 16 + (size_t)4 * G * mv + (size_t)G * W;
}

struct Ctx {
  int slot, nvalid;
};

// phases 0 and 1 shared by both decode kernels: popped entry / gates / queries -> LDS, ring
// store of the new token, hk <- hk*exp(g) + k s^T and the slot logits L.ok[g][m] (query scale
// `qscale` folded in).  Ends with every thread past the barrier that publishes L.ok.
template <typename T, int G, bool ROT>
__device__ __forceinline__ Ctx decode_prologue(const NhaDecodeArgs& a, const Lds& L, const int LM, const float qscale) {
  const int K = a.K, V = a.V, M = a.M, W = a.W, H = a.H, HQ = a.HQ;
  const int NG = HQ / H;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x / H, h = blockIdx.x % H;
  const int64_t bh = (int64_t)b * H + h;
  // ---- phase 0: popped entry, gates, queries -> LDS ---------------------------------------
  int slot = -1, nvalid = W;
  bool has_pop = true;
  const T *kp, *vp, *gp, *sp = nullptr;
  if (a.mode == NHA_DECODE_RING) {
    const int c = a.count[b];
    slot = c % W;
    has_pop = c >= W;
    nvalid = c + 1 < W ? c + 1 : W;
    if (a.count_next && h == 0 && tid == 0) a.count_next[b] = c + 1;
    const int64_t row = ((int64_t)b * W + slot) * H + h;
    kp = (const T*)a.ring_kg + row * K;
    vp = (const T*)a.ring_v + row * V;
    gp = (const T*)a.ring_g + row * M;
  } else {
    kp = (const T*)a.k_pop + bh * K;
    vp = (const T*)a.v_pop + bh * V;
    gp = (const T*)a.g_pop + bh * M;
    if (a.s_pop) sp = (const T*)a.s_pop + bh * M;
  }
  for (int i = tid; i < M; i += 256) {
    float e = 1.f, s = 0.f;
    if (has_pop) {
      e = expf(Elem<T>::ld(gp + i));
      s = sp ? Elem<T>::ld(sp + i) : 1.f - e;
    }
    L.eg[i] = e;
    L.s[i] = s;
  }
  for (int i = tid; i < K; i += 256) L.kp[i] = has_pop ? Elem<T>::ld(kp + i) : 0.f;
  for (int i = tid; i < V; i += 256) L.vp[i] = has_pop ? Elem<T>::ld(vp + i) : 0.f;
  for (int i = tid; i < G * K; i += 256) {
    const int gq = i / K, kk = i - gq * K;
    float qv = 0.f, sv = 0.f;
    if (gq < NG) {
      const T* qrow = (const T*)a.q + ((int64_t)b * HQ + h * NG + gq) * K;
      qv = Elem<T>::ld(qrow + kk);
      if (ROT) {
        const int half = K >> 1;
        const int pr = kk < half ? kk + half : kk - half;
        const float sgn = kk < half ? -1.f : 1.f;
        const int64_t co = (int64_t)b * a.cos_sb + (int64_t)(W - 1) * a.cos_sw + kk;
        sv = qv * Elem<T>::ld((const T*)a.cos + co) + sgn * Elem<T>::ld(qrow + pr) * Elem<T>::ld((const T*)a.sin + co);
      } else if (a.sq) {
        sv = Elem<T>::ld((const T*)a.sq + ((int64_t)b * HQ + h * NG + gq) * K + kk);
      }
    }
    L.q[i] = qv * qscale;
    L.sq[i] = sv * qscale;
  }
  __syncthreads();

  // ring mode: the popped entry now lives in LDS; store the new token in its slot.  The window
  // loops below read the new token from k_new / v_new, never back from the ring.
  if (a.mode == NHA_DECODE_RING) {
    const int64_t row = ((int64_t)b * W + slot) * H + h;
    for (int i = tid; i < K; i += 256) {
      ((T*)a.ring_k)[row * K + i] = ((const T*)a.k_new)[bh * K + i];
      ((T*)a.ring_kg)[row * K + i] = ((const T*)a.kg_new)[bh * K + i];
    }
    for (int i = tid; i < V; i += 256) ((T*)a.ring_v)[row * V + i] = ((const T*)a.v_new)[bh * V + i];
    for (int i = tid; i < M; i += 256) ((T*)a.ring_g)[row * M + i] = ((const T*)a.g_new)[bh * M + i];
  }

  // ---- phase 1: hk <- hk*exp(g) + k s^T ; slot logits ok[g][m] = scale q . hk[:,m] ----------
  {
    const int cm = lane % LM, rm = lane / LM, RM = 64 / LM;
    const int m0 = cm * 8;
    const bool act = m0 < M;
    float eg8[8], s8[8], acc[G][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      eg8[e] = act ? L.eg[m0 + e] : 0.f;
      s8[e] = act ? L.s[m0 + e] : 0.f;
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    if (act) {
      const float* hin = a.hk_in ? a.hk_in + bh * K * M + m0 : nullptr;
      float* hout = a.hk_out ? a.hk_out + bh * K * M + m0 : nullptr;
#pragma unroll 4
      for (int kk = wave * RM + rm; kk < K; kk += 4 * RM) {
        float hr[8];
        if (hin) {
          Elem<float>::ld8(hin + (int64_t)kk * M, hr);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) hr[e] = 0.f;
        }
        const float kv = L.kp[kk];
#pragma unroll
        for (int e = 0; e < 8; ++e) hr[e] = hr[e] * eg8[e] + kv * s8[e];
        if (hout) Elem<float>::st8(hout + (int64_t)kk * M, hr);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float qg = L.q[g * K + kk];
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
        for (int e = 0; e < 8; ++e) L.part[(wave * G + g) * M + m0 + e] = acc[g][e];
  }
  __syncthreads();
  for (int i = tid; i < G * M; i += 256)
    L.ok[i] = L.part[i] + L.part[G * M + i] + L.part[2 * G * M + i] + L.part[3 * G * M + i];

  __syncthreads();
  Ctx c;
  c.slot = slot;
  c.nvalid = nvalid;
  return c;
}

template <typename T, int G, bool ROT>
__global__ __launch_bounds__(256, G <= 4 ? 4 : 2) void decode_kernel(const NhaDecodeArgs a, const int LK, const int LV,
                                                     const int LM) {
  extern __shared__ __align__(16) float lds_raw[];
  const int K = a.K, V = a.V, M = a.M, W = a.W, H = a.H, HQ = a.HQ;
  const int NG = HQ / H;
  const Lds L = carve<G>(lds_raw, K, V, M, W);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x / H, h = blockIdx.x % H;
  const int64_t bh = (int64_t)b * H + h;
  const Ctx cx = decode_prologue<T, G, ROT>(a, L, LM, a.scale);
  const int slot = cx.slot, nvalid = cx.nvalid;

  // ---- phase 2: window logits --------------------------------------------------------------
  if (a.mode == NHA_DECODE_LOGITS) {
    for (int i = tid; i < G * W; i += 256) {
      const int g = i / W, w = i - g * W;
      if (g < NG) L.logit[i] = Elem<T>::ld((const T*)a.win_logits + ((int64_t)b * HQ + h * NG + g) * W + w);
    }
  } else {
    const int ck = lane % LK, rk = lane / LK, RK = 64 / LK;
    const int k0 = ck * 8;
    const bool act = k0 < K;
    float qr[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) qr[g][e] = act ? L.sq[g * K + k0 + e] : 0.f;
    const T* kbase = (const T*)(a.mode == NHA_DECODE_RING ? a.ring_k : a.win_k) + ((int64_t)b * W * H + h) * K + k0;
    const T* knew = a.mode == NHA_DECODE_RING ? (const T*)a.k_new + bh * K + k0 : nullptr;
    const float sgn = ck < (LK >> 1) ? -1.f : 1.f;
    constexpr int UNR = 4;   // independent 16-byte row pieces in flight per lane
    for (int wb = wave * RK * UNR; wb < nvalid; wb += 4 * RK * UNR) {
      float kv[UNR][8];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int w = wb + u * RK + rk;
        if (act && w < nvalid) {
          const T* row = (w == slot) ? knew : kbase + (int64_t)w * H * K;
          Elem<T>::ld8_stream(row, kv[u]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) kv[u][e] = 0.f;
        }
      }
      if (ROT) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const int w = wb + u * RK + rk;
          const bool ok = act && w < nvalid;
          float cs[8], sn[8];
          if (ok) {
            const int64_t co = (int64_t)b * a.cos_sb + (int64_t)w * a.cos_sw + k0;
            Elem<T>::ld8((const T*)a.cos + co, cs);
            Elem<T>::ld8((const T*)a.sin + co, sn);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float pr = __shfl_xor(kv[u][e], LK >> 1, 64);
            if (ok) kv[u][e] = kv[u][e] * cs[e] + sgn * pr * sn[e];
          }
        }
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int w = wb + u * RK + rk;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          float d = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) d += qr[g][e] * kv[u][e];
          d = row_group_sum(d, LK);
          if (ck == 0 && w < nvalid) L.logit[g * W + w] = d;
        }
      }
    }
  }
  __syncthreads();

  // ---- phase 3: ONE softmax over [M slot logits | window logits] per query head ------------
  for (int g = wave; g < NG; g += 4) {
    float mx = -INFINITY;
    for (int i = lane; i < M; i += 64) mx = fmaxf(mx, L.ok[g * M + i]);
    for (int i = lane; i < nvalid; i += 64) mx = fmaxf(mx, L.logit[g * W + i]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int i = lane; i < M; i += 64) {
      const float e = expf(L.ok[g * M + i] - mx);
      L.ok[g * M + i] = e;
      sum += e;
    }
    for (int i = lane; i < nvalid; i += 64) {
      const float e = expf(L.logit[g * W + i] - mx);
      L.logit[g * W + i] = e;
      sum += e;
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    if (lane == 0) L.inv[g] = inv;
    if (a.mode == NHA_DECODE_LOGITS && a.win_probs) {
      float* pr = a.win_probs + ((int64_t)b * HQ + h * NG + g) * W;
      for (int i = lane; i < W; i += 64) pr[i] = L.logit[g * W + i] * inv;
    }
  }
  __syncthreads();

  // ---- phase 4: hv <- hv*exp(g) + s v^T ; o = p_slots . hv + p_win . V_win -------------------
  {
    const int cv = lane % LV, rv = lane / LV, RV = 64 / LV;
    const int v0 = cv * 8;
    const bool act = v0 < V;
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    if (act) {
      float vp8[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) vp8[e] = L.vp[v0 + e];
      const float* hin = a.hv_in ? a.hv_in + bh * M * V + v0 : nullptr;
      float* hout = a.hv_out ? a.hv_out + bh * M * V + v0 : nullptr;
#pragma unroll 4
      for (int m = wave * RV + rv; m < M; m += 4 * RV) {
        float hr[8];
        if (hin) {
          Elem<float>::ld8(hin + (int64_t)m * V, hr);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) hr[e] = 0.f;
        }
        const float eg = L.eg[m], sm = L.s[m];
#pragma unroll
        for (int e = 0; e < 8; ++e) hr[e] = hr[e] * eg + sm * vp8[e];
        if (hout) Elem<float>::st8(hout + (int64_t)m * V, hr);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float p = L.ok[g * M + m];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] += p * hr[e];
        }
      }
      if (a.mode != NHA_DECODE_LOGITS) {
        const T* vbase = (const T*)(a.mode == NHA_DECODE_RING ? a.ring_v : a.win_v) + ((int64_t)b * W * H + h) * V + v0;
        const T* vnew = a.mode == NHA_DECODE_RING ? (const T*)a.v_new + bh * V + v0 : nullptr;
        constexpr int UNR = 4;
        for (int wb = wave * RV * UNR; wb < nvalid; wb += 4 * RV * UNR) {
          float vv[UNR][8];
#pragma unroll
          for (int u = 0; u < UNR; ++u) {
            const int w = wb + u * RV + rv;
            if (w < nvalid) {
              const T* row = (w == slot) ? vnew : vbase + (int64_t)w * H * V;
              Elem<T>::ld8_stream(row, vv[u]);
            } else {
#pragma unroll
              for (int e = 0; e < 8; ++e) vv[u][e] = 0.f;
            }
          }
#pragma unroll
          for (int u = 0; u < UNR; ++u) {
            const int w = wb + u * RV + rv;
            if (w < nvalid) {
#pragma unroll
              for (int g = 0; g < G; ++g) {
                const float p = L.logit[g * W + w];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] += p * vv[u][e];
              }
            }
          }
        }
      }
    }
    for (int mask = LV; mask < 64; mask <<= 1)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], mask, 64);
    if (rv == 0 && act)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) L.part[(wave * G + g) * V + v0 + e] = acc[g][e];
  }
  __syncthreads();
  for (int i = tid; i < G * V; i += 256) {
    const int g = i / V, vv = i - g * V;
    if (g < NG) {
      const float r = (L.part[i] + L.part[G * V + i] + L.part[2 * G * V + i] + L.part[3 * G * V + i]) * L.inv[g];
      Elem<T>::st((T*)a.o + ((int64_t)b * HQ + h * NG + g) * V + vv, r);
    }
  }
}


// ------------------------------------------------------------------------------------------
// Streaming variant (K == V, window or ring mode): ONE pass over the window rows.  A lane owns a
// 16-byte piece of a key row and the same piece of the value row; each group of LK lanes keeps a
// running (max, sum, weighted value) per query head (logits in log2 units), so K and V loads
// are in flight together, no logit ever goes through LDS and W is unbounded.  Groups are merged
// inside the wave with shuffles and across the four waves through LDS.
// ------------------------------------------------------------------------------------------
struct LdsS {
  Lds base;
  float *pm, *pl;
};

static size_t lds_stream_floats(int G, int K, int V, int M) { return lds_floats(G, K, V, M, 0) + 2 * 4 * 16; }

template <typename T, int G, bool ROT>
__global__ __launch_bounds__(256, G <= 4 ? 4 : 2) void decode_stream_kernel(const NhaDecodeArgs a, const int LK,
                                                                            const int LM) {
  extern __shared__ __align__(16) float lds_raw[];
  const int K = a.K, V = a.V, M = a.M, W = a.W, H = a.H, HQ = a.HQ;
  const int NG = HQ / H;
  const Lds L = carve<G>(lds_raw, K, V, M, 0);
  float* pm = L.logit;       // [4][16] per-wave running max
  float* pl = pm + 4 * 16;   // [4][16] per-wave sum
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x / H, h = blockIdx.x % H;
  const int64_t bh = (int64_t)b * H + h;
  constexpr float LOG2E = 1.4426950408889634f;
  const Ctx cx = decode_prologue<T, G, ROT>(a, L, LM, a.scale * LOG2E);
  const int slot = cx.slot, nvalid = cx.nvalid;

  const int c = lane % LK, r = lane / LK, R = 64 / LK;
  const int d0 = c * 8;
  const bool act = d0 < K;
  float mrun[G], lsum[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mx = -INFINITY;
    for (int i = lane; i < M; i += 64) mx = fmaxf(mx, L.ok[g * M + i]);
    mrun[g] = wave_max(mx);
    lsum[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
  }
  // ---- slots: hv <- hv*exp(g) + s v^T and the slot read -------------------------------------
  {
    float vp8[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) vp8[e] = act ? L.vp[d0 + e] : 0.f;
    const float* hin = a.hv_in ? a.hv_in + bh * M * V + d0 : nullptr;
    float* hout = a.hv_out ? a.hv_out + bh * M * V + d0 : nullptr;
#pragma unroll 2
    for (int m = wave * R + r; m < M; m += 4 * R) {
      float hr[8];
      if (hin && act) {
        Elem<float>::ld8(hin + (int64_t)m * V, hr);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) hr[e] = 0.f;
      }
      const float eg = L.eg[m], sm = L.s[m];
#pragma unroll
      for (int e = 0; e < 8; ++e) hr[e] = hr[e] * eg + sm * vp8[e];
      if (hout && act) Elem<float>::st8(hout + (int64_t)m * V, hr);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float p = __builtin_amdgcn_exp2f(L.ok[g * M + m] - mrun[g]);
        lsum[g] += p;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] += p * hr[e];
      }
    }
  }
  // ---- window: single pass, two rows per lane group in flight --------------------------------
  {
    float qr[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) qr[g][e] = act ? L.sq[g * K + d0 + e] : 0.f;
    const bool ring = a.mode == NHA_DECODE_RING;
    const T* kbase = (const T*)(ring ? a.ring_k : a.win_k) + ((int64_t)b * W * H + h) * K + d0;
    const T* vbase = (const T*)(ring ? a.ring_v : a.win_v) + ((int64_t)b * W * H + h) * V + d0;
    const T* knew = ring ? (const T*)a.k_new + bh * K + d0 : nullptr;
    const T* vnew = ring ? (const T*)a.v_new + bh * V + d0 : nullptr;
    const float sgn = c < (LK >> 1) ? -1.f : 1.f;
    constexpr int UNR = 2;
    for (int wb = wave * R * UNR; wb < nvalid; wb += 4 * R * UNR) {
      float kv[UNR][8], vv[UNR][8];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int w = wb + u * R + r;
        if (act && w < nvalid) {
          Elem<T>::ld8_stream((w == slot) ? knew : kbase + (int64_t)w * H * K, kv[u]);
          Elem<T>::ld8_stream((w == slot) ? vnew : vbase + (int64_t)w * H * V, vv[u]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            kv[u][e] = 0.f;
            vv[u][e] = 0.f;
          }
        }
      }
      if (ROT) {
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const int w = wb + u * R + r;
          const bool ok = act && w < nvalid;
          float cs[8], sn[8];
          if (ok) {
            const int64_t co = (int64_t)b * a.cos_sb + (int64_t)w * a.cos_sw + d0;
            Elem<T>::ld8((const T*)a.cos + co, cs);
            Elem<T>::ld8((const T*)a.sin + co, sn);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float pr = __shfl_xor(kv[u][e], LK >> 1, 64);
            if (ok) kv[u][e] = kv[u][e] * cs[e] + sgn * pr * sn[e];
          }
        }
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float d[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          float x = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) x += qr[g][e] * kv[u][e];
          x = row_group_sum(x, LK);
          d[u] = (wb + u * R + r < nvalid) ? x : -INFINITY;
        }
        float mnew = mrun[g];
#pragma unroll
        for (int u = 0; u < UNR; ++u) mnew = fmaxf(mnew, d[u]);
        const float alpha = __builtin_amdgcn_exp2f(mrun[g] - mnew);
        mrun[g] = mnew;
        float p[UNR], ps = 0.f;
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          p[u] = __builtin_amdgcn_exp2f(d[u] - mnew);
          ps += p[u];
        }
        lsum[g] = lsum[g] * alpha + ps;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float x = acc[g][e] * alpha;
#pragma unroll
          for (int u = 0; u < UNR; ++u) x += p[u] * vv[u][e];
          acc[g][e] = x;
        }
      }
    }
  }
  // ---- merge the lane groups of this wave, then the four waves -------------------------------
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mw = mrun[g];
    for (int mask = LK; mask < 64; mask <<= 1) mw = fmaxf(mw, __shfl_xor(mw, mask, 64));
    const float sc = __builtin_amdgcn_exp2f(mrun[g] - mw);
    lsum[g] *= sc;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] *= sc;
    for (int mask = LK; mask < 64; mask <<= 1) {
      lsum[g] += __shfl_xor(lsum[g], mask, 64);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], mask, 64);
    }
    if (r == 0 && act) {
#pragma unroll
      for (int e = 0; e < 8; ++e) L.part[(wave * G + g) * V + d0 + e] = acc[g][e];
    }
    if (lane == 0) {
      pm[wave * 16 + g] = mw;
      pl[wave * 16 + g] = lsum[g];
    }
  }
  __syncthreads();
  for (int i = tid; i < G * V; i += 256) {
    const int g = i / V, vv = i - g * V;
    if (g < NG) {
      const float mt = fmaxf(fmaxf(pm[g], pm[16 + g]), fmaxf(pm[32 + g], pm[48 + g]));
      float num = 0.f, den = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float sc = __builtin_amdgcn_exp2f(pm[w * 16 + g] - mt);
        num += L.part[(w * G + g) * V + vv] * sc;
        den += pl[w * 16 + g] * sc;
      }
      Elem<T>::st((T*)a.o + ((int64_t)b * HQ + h * NG + g) * V + vv, num / den);
    }
  }
}

__global__ void advance_kernel(int32_t* count, int B) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < B) count[i] += 1;
}

template <typename T, int G, bool ROT>
int launch(const NhaDecodeArgs* a, int LK, int LV, int LM, size_t lds_bytes) {
  static size_t configured = 0;
  if (lds_bytes > configured) {
    hipError_t e = hipFuncSetAttribute((const void*)decode_kernel<T, G, ROT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) {
      set_error("decode: cannot reserve %zu bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    configured = lds_bytes;
  }
  hipLaunchKernelGGL((decode_kernel<T, G, ROT>), dim3(a->B * a->H), dim3(256), lds_bytes, (hipStream_t)a->stream, *a, LK,
                     LV, LM);
  NHA_CHECK_LAUNCH("nha_decode_step");
  return NHA_OK;
}

template <typename T, bool ROT>
int dispatch_g2(const NhaDecodeArgs* a, int G, int LK, int LV, int LM, size_t lds_bytes) {
  switch (G) {
    case 1: return launch<T, 1, ROT>(a, LK, LV, LM, lds_bytes);
    case 2: return launch<T, 2, ROT>(a, LK, LV, LM, lds_bytes);
    case 4: return launch<T, 4, ROT>(a, LK, LV, LM, lds_bytes);
    case 8: return launch<T, 8, ROT>(a, LK, LV, LM, lds_bytes);
    default: return launch<T, 16, ROT>(a, LK, LV, LM, lds_bytes);
  }
}

template <typename T, int G, bool ROT>
int launch_stream(const NhaDecodeArgs* a, int LK, int LM) {
  const size_t lds_bytes = lds_stream_floats(G, a->K, a->V, a->M) * sizeof(float);
  hipLaunchKernelGGL((decode_stream_kernel<T, G, ROT>), dim3(a->B * a->H), dim3(256), lds_bytes, (hipStream_t)a->stream,
                     *a, LK, LM);
  NHA_CHECK_LAUNCH("nha_decode_step");
  return NHA_OK;
}
template <typename T, bool ROT>
int dispatch_stream(const NhaDecodeArgs* a, int G, int LK, int LM) {
  switch (G) {
    case 1: return launch_stream<T, 1, ROT>(a, LK, LM);
    case 2: return launch_stream<T, 2, ROT>(a, LK, LM);
    case 4: return launch_stream<T, 4, ROT>(a, LK, LM);
    case 8: return launch_stream<T, 8, ROT>(a, LK, LM);
    default: return launch_stream<T, 16, ROT>(a, LK, LM);
  }
}

template <typename T>
int dispatch_g(const NhaDecodeArgs* a, int G, int LK, int LV, int LM, size_t lds_bytes) {
  return a->cos ? dispatch_g2<T, true>(a, G, LK, LV, LM, lds_bytes) : dispatch_g2<T, false>(a, G, LK, LV, LM, lds_bytes);
}

}  // namespace

int decode_step_impl(const NhaDecodeArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_decode_step: null args");
  NHA_CHECK_ARG(a->B > 0 && a->H > 0 && a->HQ > 0 && a->K > 0 && a->V > 0 && a->M > 0 && a->W > 0,
                "nha_decode_step: non-positive dimension");
  NHA_CHECK_ARG(a->HQ % a->H == 0, "nha_decode_step: HQ (%d) must be a multiple of H (%d)", a->HQ, a->H);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_decode_step: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->q && a->o, "nha_decode_step: q and o are required");
  if (a->mode == NHA_DECODE_RING) {
    NHA_CHECK_ARG(a->ring_k && a->ring_kg && a->ring_v && a->ring_g && a->k_new && a->kg_new && a->v_new && a->g_new &&
                      a->count && a->sq,
                  "nha_decode_step: ring mode needs ring_k/kg/v/g, k/kg/v/g_new, count and sq");
    NHA_CHECK_ARG(!a->cos, "nha_decode_step: ring mode stores rotated keys; cos/sin are not accepted");
    NHA_CHECK_ARG((const int32_t*)a->count_next != a->count, "nha_decode_step: count_next must not alias count");
  } else if (a->mode == NHA_DECODE_WINDOW || a->mode == NHA_DECODE_LOGITS) {
    NHA_CHECK_ARG(a->k_pop && a->v_pop && a->g_pop, "nha_decode_step: k_pop, v_pop, g_pop are required");
    if (a->mode == NHA_DECODE_WINDOW) {
      NHA_CHECK_ARG(a->win_k && a->win_v, "nha_decode_step: win_k and win_v are required");
      NHA_CHECK_ARG((a->sq != nullptr) != (a->cos != nullptr),
                    "nha_decode_step: pass either sq (pre-rotated) or cos/sin (in-kernel rotary), not both");
      NHA_CHECK_ARG(!a->cos || a->sin, "nha_decode_step: cos without sin");
      NHA_CHECK_ARG(!a->cos || a->K % 2 == 0, "nha_decode_step: in-kernel rotate-half requires an even head dim");
    } else {
      NHA_CHECK_ARG(a->win_logits, "nha_decode_step: win_logits is required");
    }
  } else {
    NHA_CHECK_ARG(false, "nha_decode_step: unknown mode %d", a->mode);
  }
  const int NG = a->HQ / a->H;
  if (NG > 16 || a->K % 8 || a->V % 8 || a->M % 8 || a->K > 512 || a->V > 512 || a->M > 512) {
    set_error("nha_decode_step: unsupported shape (need HQ/H <= 16 and K, V, M multiples of 8 up to 512; got NG=%d K=%d V=%d M=%d)",
              NG, a->K, a->V, a->M);
    return NHA_ERR_UNSUPPORTED;
  }
  const int LK = next_pow2_i(a->K / 8), LV = next_pow2_i(a->V / 8), LM = next_pow2_i(a->M / 8);
  if (a->cos && LK * 8 != a->K) {
    set_error("nha_decode_step: in-kernel rotary needs a power-of-two head dim, got K=%d", a->K);
    return NHA_ERR_UNSUPPORTED;
  }
  if (a->cos && (a->cos_sw % 8 || a->cos_sb % 8)) {
    set_error("nha_decode_step: cos/sin strides must be multiples of 8 elements");
    return NHA_ERR_UNSUPPORTED;
  }
  // matrix-core kernel for the common bf16 shapes
#ifdef NHA_AB_SWITCHES   // measurement builds only (-DNHA_AB_SWITCHES): NHA_DECODE_VALU=1 keeps the VALU kernels
  static const bool valu_only = getenv("NHA_DECODE_VALU") != nullptr;
#else
  constexpr bool valu_only = false;
#endif
  if (!valu_only && decode_mfma_supported(a)) return decode_mfma_impl(a);
  int G = 1;
  while (G < NG) G <<= 1;
  // two VALU kernels: the two-sweep kernel keeps all window logits in LDS (fewest VALU operations per
  // row); the streaming kernel needs no per-row LDS and serves windows too long for that
  const bool fits_lds = lds_floats(G, a->K, a->V, a->M, a->W) * sizeof(float) <= 40 * 1024;
  if (a->mode != NHA_DECODE_LOGITS && a->K == a->V && !fits_lds) {
    if (lds_stream_floats(G, a->K, a->V, a->M) * sizeof(float) > 64 * 1024) {
      set_error("nha_decode_step: head dims too large (K=%d M=%d HQ/H=%d)", a->K, a->M, NG);
      return NHA_ERR_UNSUPPORTED;
    }
    if (a->dtype == NHA_DTYPE_BF16)
      return a->cos ? dispatch_stream<bf16_t, true>(a, G, LK, LM) : dispatch_stream<bf16_t, false>(a, G, LK, LM);
    return a->cos ? dispatch_stream<float, true>(a, G, LK, LM) : dispatch_stream<float, false>(a, G, LK, LM);
  }
  const size_t lds_bytes = lds_floats(G, a->K, a->V, a->M, a->W) * sizeof(float);
  if (lds_bytes > 160 * 1024) {
    set_error("nha_decode_step: window of %d rows x %d query heads per kv-head needs %zu bytes of LDS (limit 163840)",
              a->W, NG, lds_bytes);
    return NHA_ERR_UNSUPPORTED;
  }
  if (a->dtype == NHA_DTYPE_BF16) return dispatch_g<bf16_t>(a, G, LK, LV, LM, lds_bytes);
  return dispatch_g<float>(a, G, LK, LV, LM, lds_bytes);
}

int decode_advance_impl(int32_t* count, int32_t B, void* stream) {
  NHA_CHECK_ARG(count && B > 0, "nha_decode_advance: bad arguments");
  hipLaunchKernelGGL(advance_kernel, dim3((B + 255) / 256), dim3(256), 0, (hipStream_t)stream, count, B);
  NHA_CHECK_LAUNCH("nha_decode_advance");
  return NHA_OK;
}

}  // namespace nha
