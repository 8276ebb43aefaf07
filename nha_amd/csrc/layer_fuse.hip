// Elementwise glue of the hybrid layer on either side of the fused op, one launch each:
//   prologue: raw projections q,k,v,f -> rotated window operands, feature-mapped slot operands,
//             silu(v), gate g = logsigmoid(f)/normalizer and write strength s = 1 - exp(g)
//             (nha_fla/layers/nha.py:214-237);
//   epilogue: rms_norm(silu(o)) * weight (+ bias), the input of the output projection
//             (nha_fla/layers/nha.py:278).
// Both are HBM-bound streaming kernels: one wave per token (four tokens per workgroup), 16-byte
// accesses, every input element read once and every output element written once.  Intermediate results are rounded to
// the tensor dtype at the points where the reference's chain of tensor ops rounds them.
#include "common.h"

namespace nha {
namespace {

struct LP {
  const void *q, *k, *v, *f;
  void *q_swa, *k_swa, *q_gsa, *k_gsa, *v_out, *s, *g;
  const float* inv_freq;
  const int32_t* cu;
  int T_tot, N, T, HQ, H, K, V, M, fm, off;
  float inv_norm;
};

template <typename T> __device__ __forceinline__ float rnd(float x);
template <> __device__ __forceinline__ float rnd<float>(float x) { return x; }
template <> __device__ __forceinline__ float rnd<bf16_t>(float x) { return bf16_to_f32(f32_to_bf16(x)); }

// hardware exp2 and reciprocal: ~2 ulp of float32, far below the bf16 rounding and inside the fp32 bar
__device__ __forceinline__ float silu_f(float x) { return x * __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
__device__ __forceinline__ float feature_f(float x, int fm) { return fm == 1 ? silu_f(x) : (fm == 2 ? fmaxf(x, 0.f) : x); }

template <typename T, int VEC> __device__ __forceinline__ void ldv(const T* p, float* o) {
  if constexpr (VEC == 8) Elem<T>::ld8(p, o);
  else o[0] = Elem<T>::ld(p);
}
template <typename T, int VEC> __device__ __forceinline__ void stv(T* p, const float* v) {
  if constexpr (VEC == 8) Elem<T>::st8(p, v);
  else Elem<T>::st(p, v[0]);
}

// rotate-half RoPE of `heads` rows of K elements + the feature map of the same rows
template <typename T, int VEC>
__device__ __forceinline__ void rope_rows(const T* src, T* swa, T* gsa, int heads, int K, const float* cs, int fm,
                                          int lane) {
  const int half = K >> 1, per = half / VEC;
  for (int u = lane; u < heads * per; u += 64) {
    const int h = u / per, i = (u - h * per) * VEC;
    float x1[VEC], x2[VEC], o1[VEC], o2[VEC];
    ldv<T, VEC>(src + (size_t)h * K + i, x1);
    ldv<T, VEC>(src + (size_t)h * K + half + i, x2);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float c = cs[i + e], s = cs[half + i + e];
      o1[e] = x1[e] * c - x2[e] * s;
      o2[e] = x2[e] * c + x1[e] * s;
    }
    stv<T, VEC>(swa + (size_t)h * K + i, o1);
    stv<T, VEC>(swa + (size_t)h * K + half + i, o2);
    if (gsa) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        o1[e] = feature_f(x1[e], fm);
        o2[e] = feature_f(x2[e], fm);
      }
      stv<T, VEC>(gsa + (size_t)h * K + i, o1);
      stv<T, VEC>(gsa + (size_t)h * K + half + i, o2);
    }
  }
}

constexpr int TOK_PER_WG = 4;     // one wave per token
constexpr int ROWS_PER_WAVE = 4;  // epilogue rows a wave walks with its weight slice in registers

template <typename T, int VEC>
__global__ __launch_bounds__(256) void layer_prologue_kernel(LP p) {
  extern __shared__ float cs_all[];  // per wave: cos[K/2], sin[K/2]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* cs = cs_all + wave * p.K;
  const int t_raw = blockIdx.x * TOK_PER_WG + wave;
  const bool live = t_raw < p.T_tot;
  const int t = live ? t_raw : p.T_tot - 1;
  int pos;
  if (p.cu) {
    int lo = 0, hi = p.N;  // largest n with cu[n] <= t
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (p.cu[mid] <= t) lo = mid;
      else hi = mid;
    }
    pos = t - p.cu[lo];
  } else {
    pos = t % p.T;
  }
  pos += p.off;
  const int half = p.K >> 1;
  for (int i = lane; i < half; i += 64) {
    // the angle is the float32 product, as the rotary module's table holds it; reduce it to
    // [-pi, pi] in double so that sincosf stays on its short path at long positions
    const double ang = (double)((float)pos * p.inv_freq[i]);
    const double turns = rint(ang * 0.15915494309189535);
    const float red = (float)fma(-turns, 6.283185307179586, ang);
    float s, c;
    sincosf(red, &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  __syncthreads();
  if (!live) return;
  const size_t tq = (size_t)t * p.HQ * p.K, tk = (size_t)t * p.H * p.K;
  rope_rows<T, VEC>((const T*)p.q + tq, (T*)p.q_swa + tq, p.q_gsa ? (T*)p.q_gsa + tq : nullptr, p.HQ, p.K, cs, p.fm, lane);
  rope_rows<T, VEC>((const T*)p.k + tk, (T*)p.k_swa + tk, p.k_gsa ? (T*)p.k_gsa + tk : nullptr, p.H, p.K, cs, p.fm, lane);
  {
    const int n = p.H * p.V;
    const T* src = (const T*)p.v + (size_t)t * n;
    T* dst = (T*)p.v_out + (size_t)t * n;
    for (int u = lane * VEC; u < n; u += 64 * VEC) {
      float x[VEC];
      ldv<T, VEC>(src + u, x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[e] = silu_f(x[e]);
      stv<T, VEC>(dst + u, x);
    }
  }
  {
    const int n = p.H * p.M;
    const T* src = (const T*)p.f + (size_t)t * n;
    T* dg = (T*)p.g + (size_t)t * n;
    T* ds = (T*)p.s + (size_t)t * n;
    for (int u = lane * VEC; u < n; u += 64 * VEC) {
      float x[VEC], g[VEC], s[VEC];
      ldv<T, VEC>(src + u, x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float ls = rnd<T>(fminf(x[e], 0.f) - log1pf(expf(-fabsf(x[e]))));
        g[e] = rnd<T>(ls * p.inv_norm);
        s[e] = 1.f - rnd<T>(expf(g[e]));
      }
      stv<T, VEC>(dg + u, g);
      stv<T, VEC>(ds + u, s);
    }
  }
}

struct EP {
  const void* o;
  void* y;
  const float *w, *b;
  int rows, dim;
  float eps;
};

// NV > 0: the row (dim <= NV * 64 * VEC) stays in registers between the two passes; NV == 0: any
// dim, the second pass reads the row again (from the cache).
template <typename T, int VEC, int NV>
__global__ __launch_bounds__(256) void layer_epilogue_kernel(EP p) {
  const int row = blockIdx.x * TOK_PER_WG + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row * (NV > 0 ? ROWS_PER_WAVE : 1) >= p.rows) return;
  const T* src = (const T*)p.o + (size_t)row * p.dim;
  T* dst = (T*)p.y + (size_t)row * p.dim;
  float ss = 0.f;
  if constexpr (NV > 0) {
    // the wave keeps its slice of the weight in registers and walks ROWS_PER_WAVE rows with it
    float w[NV][VEC];
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int u = (n * 64 + lane) * VEC;
#pragma unroll
      for (int e = 0; e < VEC; ++e) w[n][e] = 1.f;
      if (p.w && u < p.dim) ldv<float, VEC>(p.w + u, w[n]);
    }
    for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
      const int r = row * ROWS_PER_WAVE + rr;
      if (r >= p.rows) break;
      src = (const T*)p.o + (size_t)r * p.dim;
      dst = (T*)p.y + (size_t)r * p.dim;
      float a[NV][VEC];
      ss = 0.f;
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        const int u = (n * 64 + lane) * VEC;
        if (u < p.dim) {
          ldv<T, VEC>(src + u, a[n]);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            a[n][e] = rnd<T>(silu_f(a[n][e]));
            ss += a[n][e] * a[n][e];
          }
        }
      }
      ss = wave_sum(ss);
      const float rstd = rsqrtf(ss / (float)p.dim + p.eps);
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        const int u = (n * 64 + lane) * VEC;
        if (u < p.dim) {
          float b[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) b[e] = 0.f;
          if (p.b) ldv<float, VEC>(p.b + u, b);
#pragma unroll
          for (int e = 0; e < VEC; ++e) a[n][e] = a[n][e] * rstd * w[n][e] + b[e];
          stv<T, VEC>(dst + u, a[n]);
        }
      }
    }
  } else {
    for (int u = lane * VEC; u < p.dim; u += 64 * VEC) {
      float x[VEC];
      ldv<T, VEC>(src + u, x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float a = rnd<T>(silu_f(x[e]));
        ss += a * a;
      }
    }
    ss = wave_sum(ss);
    const float rstd = rsqrtf(ss / (float)p.dim + p.eps);
    for (int u = lane * VEC; u < p.dim; u += 64 * VEC) {
      float x[VEC];
      ldv<T, VEC>(src + u, x);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float a = rnd<T>(silu_f(x[e])) * rstd;
        if (p.w) a *= p.w[u + e];
        if (p.b) a += p.b[u + e];
        x[e] = a;
      }
      stv<T, VEC>(dst + u, x);
    }
  }
}

template <typename T>
int launch_prologue(const LP& p, hipStream_t st) {
  const bool vec = (p.K % 16 == 0) && (p.V % 8 == 0) && (p.M % 8 == 0);
  const size_t lds = (size_t)TOK_PER_WG * p.K * sizeof(float);
  const dim3 grid((p.T_tot + TOK_PER_WG - 1) / TOK_PER_WG);
  if (vec) hipLaunchKernelGGL((layer_prologue_kernel<T, 8>), grid, dim3(256), lds, st, p);
  else hipLaunchKernelGGL((layer_prologue_kernel<T, 1>), grid, dim3(256), lds, st, p);
  return 0;
}

template <typename T>
int launch_epilogue(const EP& p, hipStream_t st) {
  const dim3 grid((p.rows + TOK_PER_WG - 1) / TOK_PER_WG);
  const dim3 grid_r((p.rows + TOK_PER_WG * ROWS_PER_WAVE - 1) / (TOK_PER_WG * ROWS_PER_WAVE));
  if (p.dim % 8 == 0 && p.dim <= 2 * 512) hipLaunchKernelGGL((layer_epilogue_kernel<T, 8, 2>), grid_r, dim3(256), 0, st, p);
  else if (p.dim % 8 == 0 && p.dim <= 8 * 512) hipLaunchKernelGGL((layer_epilogue_kernel<T, 8, 8>), grid_r, dim3(256), 0, st, p);
  else if (p.dim % 8 == 0) hipLaunchKernelGGL((layer_epilogue_kernel<T, 8, 0>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((layer_epilogue_kernel<T, 1, 0>), grid, dim3(256), 0, st, p);
  return 0;
}

}  // namespace

int layer_prologue_impl(const NhaLayerPrologueArgs* a) {
  LP p;
  p.q = a->q; p.k = a->k; p.v = a->v; p.f = a->f;
  p.q_swa = a->q_swa; p.k_swa = a->k_swa;
  p.q_gsa = a->feature_map ? a->q_gsa : nullptr;
  p.k_gsa = a->feature_map ? a->k_gsa : nullptr;
  p.v_out = a->v_out; p.s = a->s; p.g = a->g;
  p.inv_freq = a->inv_freq;
  p.cu = a->cu_seqlens;
  p.T_tot = a->T_tot; p.N = a->N; p.T = a->T_tot / a->N;
  p.HQ = a->HQ; p.H = a->H; p.K = a->K; p.V = a->V; p.M = a->M;
  p.fm = a->feature_map; p.off = a->seqlen_offset;
  p.inv_norm = 1.f / a->gate_logit_normalizer;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch_prologue<bf16_t>(p, st);
  else launch_prologue<float>(p, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_layer_prologue: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}

int layer_epilogue_impl(const NhaLayerEpilogueArgs* a) {
  EP p;
  p.o = a->o; p.y = a->y; p.w = a->weight; p.b = a->bias; p.rows = a->rows; p.dim = a->dim; p.eps = a->eps;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch_epilogue<bf16_t>(p, st);
  else launch_epilogue<float>(p, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_layer_epilogue: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}

}  // namespace nha
