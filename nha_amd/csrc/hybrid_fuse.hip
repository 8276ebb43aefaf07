// Glue of the hybrid decoder models' attention blocks in one launch (nha_hybrid_prologue): what the
// reference runs as a chain of tensor ops between the projections and the attention op --
// per-head RMSNorm of q and k (nha_fla/models/qwen3_moe_nha/qwennha.py:103-106; absent in the dense flavour,
// nha_fla/models/llama3_nha/llamanha.py:79-81), the gates g = logsigmoid(f) / 8 and s = 1 - exp(g)
// (qwennha.py:117-128), the left-padding mask on v and s (:133-144), rotate-half rotary embedding of q and k
// (:240-247) and the copies that make every operand contiguous.  Intermediate values are rounded to the tensor
// dtype where the chain of tensor ops rounds them (norm output, weighted norm output, logsigmoid, g, exp(g)), so a
// bf16 block sees the same operands; the rotation is evaluated in fp32 and rounded once.
//
// The inputs may be column slices of one fused projection output (a row stride per input); every output is
// contiguous.  One workgroup per token; a head row of D elements is spread over D / 8 lanes with 8 consecutive
// elements each (16-byte accesses in bf16), so that a wave instruction covers 512 / D rows and the rotary partner of
// a lane (columns +- D / 2) is the lane D / 16 away in the same row.  Bound by HBM:
// 2 (HQ + H) D reads and 4 (HQ + H) D writes of the head rows per token, plus v and the gates.
#include "common.h"

namespace nha {
namespace {

struct HP {
  const void *q, *k, *v, *f;
  int64_t q_stride, k_stride, v_stride, f_stride;   // elements between the rows of two tokens
  const void *q_weight, *k_weight;                  // [D], or null: no norm
  const void *cos, *sin;                            // [B or 1][T][D]
  int64_t cs_batch_stride;                          // elements; 0 = one table for every sequence
  const int64_t* positions;                         // [B*T] and inv_freq [D/2]: the tables' rows formed here instead
  const float* inv_freq;
  const void* mask;                                 // [B*T] in the tensor dtype, or null
  void *q_out, *sq_out, *k_out, *sk_out, *v_out, *g_out, *s_out;
  int B, T, HQ, H, M;
  float eps, norm;   // gate normalizer: g = logsigmoid(f) / norm
};

template <typename T> __device__ __forceinline__ float rnd(float x);
template <> __device__ __forceinline__ float rnd<float>(float x) { return x; }
template <> __device__ __forceinline__ float rnd<bf16_t>(float x) { return bf16_to_f32(f32_to_bf16(x)); }

template <typename T, int D>
__global__ __launch_bounds__(256) void hybrid_prologue_kernel(const HP p) {
  constexpr int LPR = D / 8;           // lanes per head row
  constexpr int RPW = 64 / LPR;        // rows per wave instruction
  const int tok = blockIdx.x;          // b * T + t
  const int b = tok / p.T, t = tok % p.T;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane % LPR, rsub = lane / LPR;
  const bool first_half = c < LPR / 2;
  float cs[8], sn[8];
  if (p.positions) {
    // cos / sin of position * inv_freq[column % (D / 2)], each rounded to the tensor dtype as a table entry would be
    const float pos = (float)p.positions[tok];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float ang = pos * p.inv_freq[(8 * c + e) % (D / 2)];
      cs[e] = rnd<T>(cosf(ang));
      sn[e] = rnd<T>(sinf(ang));
    }
  } else {
    const int64_t off = (int64_t)b * p.cs_batch_stride + (int64_t)t * D + 8 * c;
    Elem<T>::ld8((const T*)p.cos + off, cs);
    Elem<T>::ld8((const T*)p.sin + off, sn);
  }
  const float mk = p.mask ? Elem<T>::ld((const T*)p.mask + tok) : 1.f;

  // head rows: the HQ query rows, then the H key rows
  const int nrows = p.HQ + p.H;
  for (int r0 = wave * RPW; r0 < nrows; r0 += 4 * RPW) {
    const int r = r0 + rsub;
    if (r >= nrows) continue;          // whole 16-byte rows only: the shuffles below stay inside a row's lanes
    const bool isq = r < p.HQ;
    const int hh = isq ? r : r - p.HQ;
    const T* src = isq ? (const T*)p.q + (int64_t)tok * p.q_stride + (int64_t)hh * D
                       : (const T*)p.k + (int64_t)tok * p.k_stride + (int64_t)hh * D;
    const T* w = (const T*)(isq ? p.q_weight : p.k_weight);
    const int64_t orow = ((int64_t)tok * (isq ? p.HQ : p.H) + hh) * D + 8 * c;
    T* plain = (T*)(isq ? p.q_out : p.k_out) + orow;
    T* rot = (T*)(isq ? p.sq_out : p.sk_out) + orow;
    float x[8];
    Elem<T>::ld8(src + 8 * c, x);
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
#pragma unroll
      for (int msk = LPR / 2; msk >= 1; msk >>= 1) ss += __shfl_xor(ss, msk, 64);
      const float inv = rsqrtf(ss * (1.f / D) + p.eps);
      float wv[8];
      Elem<T>::ld8(w + 8 * c, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = rnd<T>(wv[e] * rnd<T>(x[e] * inv));
    }
    Elem<T>::st8(plain, x);
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xp = __shfl_xor(x[e], LPR / 2, 64);     // column +- D / 2 of the same row
      y[e] = x[e] * cs[e] + (first_half ? -xp : xp) * sn[e];
    }
    Elem<T>::st8(rot, y);
  }

  // values (masked) and gates
  {
    const int n = p.H * D;
    const T* src = (const T*)p.v + (int64_t)tok * p.v_stride;
    T* dst = (T*)p.v_out + (int64_t)tok * n;
    for (int u = tid * 8; u < n; u += 256 * 8) {
      float x[8];
      Elem<T>::ld8(src + u, x);
      if (p.mask) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = rnd<T>(x[e] * mk);
      }
      Elem<T>::st8(dst + u, x);
    }
  }
  {
    const int n = p.H * p.M;
    const T* src = (const T*)p.f + (int64_t)tok * p.f_stride;
    T* dg = (T*)p.g_out + (int64_t)tok * n;
    T* ds = p.s_out ? (T*)p.s_out + (int64_t)tok * n : nullptr;
    for (int u = tid * 8; u < n; u += 256 * 8) {
      float x[8], g[8], s[8];
      if (p.f) {
        Elem<T>::ld8(src + u, x);
      } else {           // a layer without slot writes: g = 0, s = 0
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (!p.f) {
          g[e] = 0.f;
          s[e] = 0.f;
          continue;
        }
        const float ls = rnd<T>(fminf(x[e], 0.f) - log1pf(expf(-fabsf(x[e]))));
        g[e] = rnd<T>(ls / p.norm);
        s[e] = rnd<T>(1.f - rnd<T>(expf(g[e])));
        if (p.mask) s[e] = rnd<T>(s[e] * mk);
      }
      Elem<T>::st8(dg + u, g);
      if (ds) Elem<T>::st8(ds + u, s);
    }
  }
}

// Zero-sink layers (window 2048: sliding-window softmax preceded by `sinks` all-zero key / value rows,
// nha_fla/models/qwen3_moe_nha/qwennha.py:323-336, :400-413) run through the NHA kernels with slot states that stay
// zero: M zero-logit keys with zero values sit in every query's softmax, while the reference's window covers
// n0(t) = clamp(W - 1 - t, 0, M) of them.  Row (token, head) of o is multiplied in place by
// (e^lse + M) / (e^lse + n0(t)), lse = the window's log-sum-exp the kernel returned, formed in log space
// (logaddexp) and capped at the largest float.  One wave per 512 / D... rows of D elements, 8 per lane.
template <typename T, int D>
__global__ __launch_bounds__(256) void zero_sink_rescale_kernel(T* o, const float* lse, int rows, int HQ, int Tlen, int W, int M) {
  constexpr int LPR = D / 8;
  const int r = (blockIdx.x * 256 + threadIdx.x) / LPR, c = threadIdx.x % LPR;
  if (r >= rows) return;
  const int t = (r / HQ) % Tlen;
  int n0 = W - 1 - t;
  n0 = n0 < 0 ? 0 : (n0 > M ? M : n0);
  if (n0 == M) return;                       // every sink is in view: nothing to take out
  const float l = lse[r];
  auto lae = [](float a, float b) {          // log(e^a + e^b), b may be -inf
    const float hi = fmaxf(a, b), lo = fminf(a, b);
    return lo == -INFINITY ? hi : hi + log1pf(expf(lo - hi));
  };
  const float lnum = lae(l, logf((float)M));
  const float lden = lae(l, n0 > 0 ? logf((float)n0) : -INFINITY);
  const float fac = fminf(expf(lnum - lden), 3.4028234664e38f);
  T* p = o + (int64_t)r * D + 8 * c;
  float x[8];
  Elem<T>::ld8(p, x);
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] *= fac;
  Elem<T>::st8(p, x);
}

template <typename T>
void launch(const HP& p, int D, hipStream_t st) {
  const dim3 grid(p.B * p.T), block(256);
  if (D == 64) hipLaunchKernelGGL((hybrid_prologue_kernel<T, 64>), grid, block, 0, st, p);
  else if (D == 128) hipLaunchKernelGGL((hybrid_prologue_kernel<T, 128>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((hybrid_prologue_kernel<T, 256>), grid, block, 0, st, p);
}

template <typename T>
void launch_rescale(void* o, const float* lse, int rows, int HQ, int Tlen, int W, int M, int D, hipStream_t st) {
  const int per = 256 / (D / 8);
  const dim3 grid((rows + per - 1) / per), block(256);
  if (D == 64) hipLaunchKernelGGL((zero_sink_rescale_kernel<T, 64>), grid, block, 0, st, (T*)o, lse, rows, HQ, Tlen, W, M);
  else if (D == 128) hipLaunchKernelGGL((zero_sink_rescale_kernel<T, 128>), grid, block, 0, st, (T*)o, lse, rows, HQ, Tlen, W, M);
  else hipLaunchKernelGGL((zero_sink_rescale_kernel<T, 256>), grid, block, 0, st, (T*)o, lse, rows, HQ, Tlen, W, M);
}

}  // namespace

int zero_sink_rescale_impl(void* o, const float* lse_swa, int B, int T, int HQ, int D, int W, int M, int dtype, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (dtype == NHA_DTYPE_BF16) launch_rescale<bf16_t>(o, lse_swa, B * T * HQ, HQ, T, W, M, D, st);
  else launch_rescale<float>(o, lse_swa, B * T * HQ, HQ, T, W, M, D, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_zero_sink_rescale: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}

int hybrid_prologue_impl(const NhaHybridPrologueArgs* a) {
  HP p = {};
  p.q = a->q; p.k = a->k; p.v = a->v; p.f = a->f;
  p.q_stride = a->q_stride; p.k_stride = a->k_stride; p.v_stride = a->v_stride; p.f_stride = a->f_stride;
  p.q_weight = a->q_weight; p.k_weight = a->k_weight;
  p.cos = a->cos; p.sin = a->sin; p.cs_batch_stride = a->cs_batch_stride;
  p.positions = a->positions; p.inv_freq = a->inv_freq;
  p.mask = a->mask;
  p.q_out = a->q_out; p.sq_out = a->sq_out; p.k_out = a->k_out; p.sk_out = a->sk_out;
  p.v_out = a->v_out; p.g_out = a->g_out; p.s_out = a->s_out;
  p.B = a->B; p.T = a->T; p.HQ = a->HQ; p.H = a->H; p.M = a->M;
  p.eps = a->eps; p.norm = a->gate_logit_normalizer;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch<bf16_t>(p, a->D, st);
  else launch<float>(p, a->D, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_hybrid_prologue: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}

}  // namespace nha
