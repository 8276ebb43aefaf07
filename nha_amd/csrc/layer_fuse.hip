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
  // backward only: cotangents of the seven outputs, gradients of the four inputs
  const void *dq_swa, *dk_swa, *dq_gsa, *dk_gsa, *dv_out, *ds, *dg;
  void *dq, *dk, *dv, *df;
};

constexpr int TOK_PER_WG = 4;     // one wave per token
constexpr int ROWS_PER_WAVE = 4;  // epilogue rows a wave walks with its weight slice in registers
constexpr int BWD_ROWS = 32;      // epilogue backward: rows per workgroup (one partial weight gradient each)

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

// VEC elements as loaded (conversion deferred, so a prefetched row costs half the registers in bf16)
template <typename T, int VEC> struct Raw;
template <> struct Raw<bf16_t, 8> {
  uint4 r;
  __device__ __forceinline__ void load(const bf16_t* p) { r = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void unpack(float* o) const {
    o[0] = __uint_as_float(r.x << 16); o[1] = __uint_as_float(r.x & 0xffff0000u);
    o[2] = __uint_as_float(r.y << 16); o[3] = __uint_as_float(r.y & 0xffff0000u);
    o[4] = __uint_as_float(r.z << 16); o[5] = __uint_as_float(r.z & 0xffff0000u);
    o[6] = __uint_as_float(r.w << 16); o[7] = __uint_as_float(r.w & 0xffff0000u);
  }
};
template <> struct Raw<float, 8> {
  float4 a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  __device__ __forceinline__ void unpack(float* o) const {
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
};
template <typename T> struct Raw<T, 1> {
  T r;
  __device__ __forceinline__ void load(const T* p) { r = *p; }
  __device__ __forceinline__ void unpack(float* o) const { o[0] = Elem<T>::ld(&r); }
};

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

// cos/sin of the token's rotary angles into the wave's LDS slice cs[0..K/2) | cs[K/2..K); returns
// the token index of this wave (clamped) and whether it exists.  All four waves reach the barrier.
__device__ __forceinline__ int token_angles(const LP& p, float* cs, int wave, int lane, bool* live) {
  const int t_raw = blockIdx.x * TOK_PER_WG + wave;
  *live = t_raw < p.T_tot;
  const int t = *live ? t_raw : p.T_tot - 1;
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
    float sn, c;
    sincosf(red, &sn, &c);
    cs[i] = c;
    cs[half + i] = sn;
  }
  __syncthreads();
  return t;
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void layer_prologue_kernel(LP p) {
  extern __shared__ float cs_all[];  // per wave: cos[K/2], sin[K/2]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* cs = cs_all + wave * p.K;
  bool live;
  const int t = token_angles(p, cs, wave, lane, &live);
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

// d silu(x) / dx and the derivative of the feature map
__device__ __forceinline__ float silu_grad_f(float x) {
  const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-x));
  return sg * (1.f + x * (1.f - sg));
}
__device__ __forceinline__ float feature_grad_f(float x, int fm) {
  return fm == 1 ? silu_grad_f(x) : (fm == 2 ? (x > 0.f ? 1.f : 0.f) : 1.f);
}

// gradient of rope_rows: the rotation by the opposite angle of the window cotangent plus the
// feature map's derivative times the slot cotangent
template <typename T, int VEC>
__device__ __forceinline__ void rope_rows_bwd(const T* src, const T* dswa, const T* dgsa, T* dx, int heads, int K,
                                              const float* cs, int fm, int lane) {
  const int half = K >> 1, per = half / VEC;
  for (int u = lane; u < heads * per; u += 64) {
    const int h = u / per, i = (u - h * per) * VEC;
    const size_t o1 = (size_t)h * K + i, o2 = o1 + half;
    float d1[VEC], d2[VEC], r1[VEC], r2[VEC];
    ldv<T, VEC>(dswa + o1, d1);
    ldv<T, VEC>(dswa + o2, d2);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float c = cs[i + e], sn = cs[half + i + e];
      r1[e] = d1[e] * c + d2[e] * sn;
      r2[e] = d2[e] * c - d1[e] * sn;
    }
    if (dgsa) {
      float x1[VEC], x2[VEC];
      ldv<T, VEC>(src + o1, x1);
      ldv<T, VEC>(src + o2, x2);
      ldv<T, VEC>(dgsa + o1, d1);
      ldv<T, VEC>(dgsa + o2, d2);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        r1[e] += feature_grad_f(x1[e], fm) * d1[e];
        r2[e] += feature_grad_f(x2[e], fm) * d2[e];
      }
    }
    stv<T, VEC>(dx + o1, r1);
    stv<T, VEC>(dx + o2, r2);
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void layer_prologue_bwd_kernel(LP p) {
  extern __shared__ float cs_all[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* cs = cs_all + wave * p.K;
  bool live;
  const int t = token_angles(p, cs, wave, lane, &live);
  if (!live) return;
  const size_t tq = (size_t)t * p.HQ * p.K, tk = (size_t)t * p.H * p.K;
  rope_rows_bwd<T, VEC>((const T*)p.q + tq, (const T*)p.dq_swa + tq, p.dq_gsa ? (const T*)p.dq_gsa + tq : nullptr,
                        (T*)p.dq + tq, p.HQ, p.K, cs, p.fm, lane);
  rope_rows_bwd<T, VEC>((const T*)p.k + tk, (const T*)p.dk_swa + tk, p.dk_gsa ? (const T*)p.dk_gsa + tk : nullptr,
                        (T*)p.dk + tk, p.H, p.K, cs, p.fm, lane);
  {
    const int n = p.H * p.V;
    const T* src = (const T*)p.v + (size_t)t * n;
    const T* dsrc = (const T*)p.dv_out + (size_t)t * n;
    T* dst = (T*)p.dv + (size_t)t * n;
    for (int u = lane * VEC; u < n; u += 64 * VEC) {
      float x[VEC], d[VEC];
      ldv<T, VEC>(src + u, x);
      ldv<T, VEC>(dsrc + u, d);
#pragma unroll
      for (int e = 0; e < VEC; ++e) d[e] *= silu_grad_f(x[e]);
      stv<T, VEC>(dst + u, d);
    }
  }
  {
    // g = logsigmoid(f)/n, s = 1 - exp(g):  df = (dg - ds * exp(g)) / n * sigmoid(-f)
    const int n = p.H * p.M;
    const T* src = (const T*)p.f + (size_t)t * n;
    const T* pdg = (const T*)p.dg + (size_t)t * n;
    const T* pds = (const T*)p.ds + (size_t)t * n;
    T* dst = (T*)p.df + (size_t)t * n;
    for (int u = lane * VEC; u < n; u += 64 * VEC) {
      float x[VEC], dg[VEC], ds[VEC];
      ldv<T, VEC>(src + u, x);
      ldv<T, VEC>(pdg + u, dg);
      ldv<T, VEC>(pds + u, ds);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float ls = rnd<T>(fminf(x[e], 0.f) - log1pf(expf(-fabsf(x[e]))));
        const float eg = rnd<T>(expf(rnd<T>(ls * p.inv_norm)));
        dg[e] = (dg[e] - ds[e] * eg) * p.inv_norm / (1.f + expf(x[e]));
      }
      stv<T, VEC>(dst + u, dg);
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
    // the next row's raw elements are in flight while the current row is reduced and written
    Raw<T, VEC> nxt[NV];
    const int r0 = row * ROWS_PER_WAVE;
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int u = (n * 64 + lane) * VEC;
      if (u < p.dim) nxt[n].load((const T*)p.o + (size_t)r0 * p.dim + u);
    }
    for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
      const int r = r0 + rr;
      if (r >= p.rows) break;
      dst = (T*)p.y + (size_t)r * p.dim;
      float a[NV][VEC];
#pragma unroll
      for (int n = 0; n < NV; ++n) nxt[n].unpack(a[n]);
      if (rr + 1 < ROWS_PER_WAVE && r + 1 < p.rows) {
#pragma unroll
        for (int n = 0; n < NV; ++n) {
          const int u = (n * 64 + lane) * VEC;
          if (u < p.dim) nxt[n].load((const T*)p.o + (size_t)(r + 1) * p.dim + u);
        }
      }
      ss = 0.f;
#pragma unroll
      for (int n = 0; n < NV; ++n) {
        const int u = (n * 64 + lane) * VEC;
        if (u < p.dim) {
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

struct EPB {
  const void *o, *dy;
  void* dout;
  const float* w;
  float *dw_part, *db_part;
  int rows, dim;
  float eps;
};

// Backward of y = silu(o) * rstd * w + b for BWD_ROWS rows per workgroup.  Thread `tid` owns the
// columns (n * 256 + tid) * 8 .. + 8, n < NV, of every row, so its share of the weight and bias
// gradients accumulates in registers and leaves as one row of the partial-sum arrays
// dw_part / db_part [gridDim.x, dim] (summed over the first axis by the caller: a fixed order).
template <typename T, int NV>
__global__ __launch_bounds__(256) void layer_epilogue_bwd_kernel(EPB p) {
  __shared__ float red[8];
  const int tid = threadIdx.x;
  float w[NV][8], dw[NV][8], db[NV][8];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    const int u = (n * 256 + tid) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) w[n][e] = 1.f, dw[n][e] = 0.f, db[n][e] = 0.f;
    if (p.w && u < p.dim) ldv<float, 8>(p.w + u, w[n]);
  }
  const int r0 = blockIdx.x * BWD_ROWS;
  for (int rr = 0; rr < BWD_ROWS; ++rr) {
    const int r = r0 + rr;
    if (r >= p.rows) break;  // uniform over the workgroup
    const T* src = (const T*)p.o + (size_t)r * p.dim;
    const T* dsrc = (const T*)p.dy + (size_t)r * p.dim;
    T* dst = (T*)p.dout + (size_t)r * p.dim;
    float x[NV][8], a[NV][8], d[NV][8];
    float ss = 0.f, dot = 0.f;
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int u = (n * 256 + tid) * 8;
      if (u < p.dim) {
        ldv<T, 8>(src + u, x[n]);
        ldv<T, 8>(dsrc + u, d[n]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          a[n][e] = rnd<T>(silu_f(x[n][e]));
          ss += a[n][e] * a[n][e];
          dot += d[n][e] * w[n][e] * a[n][e];
        }
      }
    }
    // both row sums in one pass over the workgroup
    ss = wave_sum(ss);
    dot = wave_sum(dot);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = ss, red[4 + (tid >> 6)] = dot;
    __syncthreads();
    ss = (red[0] + red[1]) + (red[2] + red[3]);
    dot = (red[4] + red[5]) + (red[6] + red[7]);
    const float rstd = rsqrtf(ss / (float)p.dim + p.eps);
    const float coef = dot * rstd * rstd * rstd / (float)p.dim;  // rstd * mean(dn * n), n = a * rstd
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int u = (n * 256 + tid) * 8;
      if (u < p.dim) {
        float g[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          dw[n][e] += d[n][e] * a[n][e] * rstd;
          db[n][e] += d[n][e];
          const float da = rstd * d[n][e] * w[n][e] - coef * a[n][e];
          g[e] = da * silu_grad_f(x[n][e]);
        }
        stv<T, 8>(dst + u, g);
      }
    }
  }
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    const int u = (n * 256 + tid) * 8;
    if (u < p.dim) {
      if (p.dw_part) stv<float, 8>(p.dw_part + (size_t)blockIdx.x * p.dim + u, dw[n]);
      if (p.db_part) stv<float, 8>(p.db_part + (size_t)blockIdx.x * p.dim + u, db[n]);
    }
  }
}

template <typename T>
int launch_epilogue_bwd(const EPB& p, hipStream_t st) {
  const dim3 grid((p.rows + BWD_ROWS - 1) / BWD_ROWS);
  if (p.dim <= 2048) hipLaunchKernelGGL((layer_epilogue_bwd_kernel<T, 1>), grid, dim3(256), 0, st, p);
  else if (p.dim <= 4096) hipLaunchKernelGGL((layer_epilogue_bwd_kernel<T, 2>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((layer_epilogue_bwd_kernel<T, 4>), grid, dim3(256), 0, st, p);
  return 0;
}

template <typename T>
int launch_prologue_bwd(const LP& p, hipStream_t st) {
  const bool vec = (p.K % 16 == 0) && (p.V % 8 == 0) && (p.M % 8 == 0);
  const size_t lds = (size_t)TOK_PER_WG * p.K * sizeof(float);
  const dim3 grid((p.T_tot + TOK_PER_WG - 1) / TOK_PER_WG);
  if (vec) hipLaunchKernelGGL((layer_prologue_bwd_kernel<T, 8>), grid, dim3(256), lds, st, p);
  else hipLaunchKernelGGL((layer_prologue_bwd_kernel<T, 1>), grid, dim3(256), lds, st, p);
  return 0;
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


// ------------------------------------------------------------------------------------------
// Depthwise causal short convolution (+ SiLU) over packed tokens, the layer's use_short_conv option
// (nha_fla/layers/nha.py:186-206):  y[t][c] = act(b[c] + sum_j w[c][j] x[t - (KS-1) + j][c]), taps that
// would reach before the start of t's sequence are zero.  fp32 arithmetic, rounded once.
// ------------------------------------------------------------------------------------------
struct SC {
  const void *x, *w, *b, *dy;
  void *y, *dx;
  float *dw_part, *db_part;
  const int32_t* cu;
  int T_tot, N, T, C, act;
};

constexpr int SC_RUN = 32;    // tokens a thread of the backward walks (one partial weight gradient per run)

// the 8 x KS weights of 8 consecutive channels: contiguous in [C][KS], read as KS 8-element pieces
template <typename T, int KS>
__device__ __forceinline__ void load_taps(const T* w, int c, float (&wt)[KS][8]) {
  float wv[8 * KS];
#pragma unroll
  for (int i = 0; i < KS; ++i) Elem<T>::ld8(w + (int64_t)c * KS + 8 * i, wv + 8 * i);
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int j = 0; j < KS; ++j) wt[j][e] = wv[e * KS + j];
}

// [bos, eos) of the sequence that holds token t0, and the index of the boundary after eos (varlen)
__device__ __forceinline__ void seq_of(const SC& p, int t0, int& bos, int& eos, int& seq_next) {
  seq_next = 0;
  if (!p.cu) {
    bos = (t0 / p.T) * p.T;
    eos = bos + p.T;
    return;
  }
  int lo = 0, hi = p.N - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (p.cu[mid] <= t0) lo = mid; else hi = mid - 1;
  }
  bos = p.cu[lo];
  eos = p.cu[lo + 1];
  seq_next = lo + 1;
}

constexpr int SCF_RUN = 16;   // tokens a thread of the forward walks
constexpr int SC_GRP = 4;     // tokens whose rows are requested together

// one thread: 8 channels of a run of SCF_RUN tokens, the last KS inputs in registers (every input row is
// read once); the rows of SC_GRP tokens are requested together
template <typename T, int KS>
__global__ __launch_bounds__(256) void short_conv_kernel(const SC p) {
  const int c8n = p.C / 8;
  const int cg = blockIdx.y * 256 + threadIdx.x;
  if (cg >= c8n) return;
  const int c = cg * 8;
  const int t0 = blockIdx.x * SCF_RUN;
  const int t1 = (t0 + SCF_RUN) < p.T_tot ? (t0 + SCF_RUN) : p.T_tot;
  const T* __restrict__ xp = (const T*)p.x;
  T* __restrict__ yp = (T*)p.y;
  float w[KS][8], bias[8];
  load_taps<T, KS>((const T*)p.w, c, w);
#pragma unroll
  for (int e = 0; e < 8; ++e) bias[e] = p.b ? Elem<T>::ld((const T*)p.b + c + e) : 0.f;
  float xh[KS][8];   // xh[d] = x[t - d]
#pragma unroll
  for (int d = 0; d < KS; ++d)
#pragma unroll
    for (int e = 0; e < 8; ++e) xh[d][e] = 0.f;
#pragma unroll
  for (int d = 1; d < KS; ++d)
    if (t0 - d >= 0) Elem<T>::ld8(xp + (int64_t)(t0 - d) * p.C + c, xh[d - 1]);
  int bos, eos, seq_next;
  seq_of(p, t0, bos, eos, seq_next);
  for (int tb = t0; tb < t1; tb += SC_GRP) {
    float xin[SC_GRP][8];
#pragma unroll
    for (int i = 0; i < SC_GRP; ++i)
      if (tb + i < t1) Elem<T>::ld8(xp + (int64_t)(tb + i) * p.C + c, xin[i]);
#pragma unroll
    for (int i = 0; i < SC_GRP; ++i) {
      const int t = tb + i;
      if (t >= t1) break;
      while (t >= eos) {   // the walk enters the next sequence
        bos = eos;
        if (!p.cu) eos = bos + p.T;
        else if (seq_next < p.N) { ++seq_next; eos = p.cu[seq_next]; }
        else eos = p.T_tot;   // boundaries that end before the last token: the rest is one more sequence
      }
#pragma unroll
      for (int d = KS - 1; d >= 1; --d)
#pragma unroll
        for (int e = 0; e < 8; ++e) xh[d][e] = xh[d - 1][e];
#pragma unroll
      for (int e = 0; e < 8; ++e) xh[0][e] = xin[i][e];
      const int reach = t - bos;   // taps d <= reach lie inside the sequence
      float acc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float pre = bias[e];
#pragma unroll
        for (int d = 0; d < KS; ++d)
          if (d <= reach) pre += w[KS - 1 - d][e] * xh[d][e];
        acc[e] = p.act ? silu_f(pre) : pre;
      }
      Elem<T>::st8(yp + (int64_t)t * p.C + c, acc);
    }
  }
}

// one thread: 8 channels of a run of SC_RUN tokens, walked in order with the last KS inputs and the KS
// unfinished input gradients in registers; the KS - 1 tokens after the run are walked too (their
// pre-activation gradients reach back into the run).  Weight / bias gradients of the run leave as one
// partial sum per run: [runs][C][KS] and [runs][C], added up by the caller in a fixed order.
template <typename T, int KS>
__global__ __launch_bounds__(256) void short_conv_bwd_kernel(const SC p) {
  const int c8n = p.C / 8;
  const int run = blockIdx.x;
  const int cg = blockIdx.y * 256 + threadIdx.x;
  if (cg >= c8n) return;
  const int c = cg * 8;
  const int t0 = run * SC_RUN;
  const int t1 = (t0 + SC_RUN) < p.T_tot ? (t0 + SC_RUN) : p.T_tot;            // end of the run
  const int t2 = (t1 + KS - 1) < p.T_tot ? (t1 + KS - 1) : p.T_tot;            // end of the walk
  const T* __restrict__ xp = (const T*)p.x;
  const T* __restrict__ dyp = (const T*)p.dy;
  T* __restrict__ dxp = (T*)p.dx;
  float w[KS][8], bias[8];
  load_taps<T, KS>((const T*)p.w, c, w);
#pragma unroll
  for (int e = 0; e < 8; ++e) bias[e] = p.b ? Elem<T>::ld((const T*)p.b + c + e) : 0.f;
  float xh[KS][8], dxr[KS][8], dw[KS][8], db[8];   // xh[d] = x[t - d], dxr[d] = unfinished dx[t - d]
#pragma unroll
  for (int d = 0; d < KS; ++d)
#pragma unroll
    for (int e = 0; e < 8; ++e) xh[d][e] = dxr[d][e] = dw[d][e] = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) db[e] = 0.f;
  // inputs before the run (the walk shifts them into place)
#pragma unroll
  for (int d = 1; d < KS; ++d)
    if (t0 - d >= 0) Elem<T>::ld8(xp + (int64_t)(t0 - d) * p.C + c, xh[d - 1]);
  int bos, eos, seq_next;
  seq_of(p, t0, bos, eos, seq_next);
  for (int tb = t0; tb < t2; tb += SC_GRP) {
    float xin[SC_GRP][8], dyin[SC_GRP][8];
#pragma unroll
    for (int i = 0; i < SC_GRP; ++i)
      if (tb + i < t2) {
        Elem<T>::ld8(xp + (int64_t)(tb + i) * p.C + c, xin[i]);
        Elem<T>::ld8(dyp + (int64_t)(tb + i) * p.C + c, dyin[i]);
      }
#pragma unroll
    for (int i = 0; i < SC_GRP; ++i) {
      const int t = tb + i;
      if (t >= t2) break;
      while (t >= eos) {   // the walk enters the next sequence
        bos = eos;
        if (!p.cu) eos = bos + p.T;
        else if (seq_next < p.N) { ++seq_next; eos = p.cu[seq_next]; }
        else eos = p.T_tot;   // boundaries that end before the last token: the rest is one more sequence
      }
      // shift the histories: slot d now belongs to token t - d
#pragma unroll
      for (int d = KS - 1; d >= 1; --d)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xh[d][e] = xh[d - 1][e];
          dxr[d][e] = dxr[d - 1][e];
        }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xh[0][e] = xin[i][e];
        dxr[0][e] = 0.f;
      }
      const int reach = t - bos;   // taps d <= reach lie inside the sequence
      float dpre[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float pre = bias[e];
#pragma unroll
        for (int d = 0; d < KS; ++d)
          if (d <= reach) pre += w[KS - 1 - d][e] * xh[d][e];
        float g = dyin[i][e];
        if (p.act) {
          const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-pre));
          g *= sg * (1.f + pre * (1.f - sg));
        }
        dpre[e] = g;
      }
      const bool own = t < t1;
#pragma unroll
      for (int d = 0; d < KS; ++d) {
        if (d > reach) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          dxr[d][e] += w[KS - 1 - d][e] * dpre[e];
          if (own) dw[KS - 1 - d][e] += dpre[e] * xh[d][e];
        }
      }
      if (own) {
#pragma unroll
        for (int e = 0; e < 8; ++e) db[e] += dpre[e];
      }
      // token t - (KS-1) has received its last contribution
      const int u = t - (KS - 1);
      if (u >= t0 && u < t1) Elem<T>::st8(dxp + (int64_t)u * p.C + c, dxr[KS - 1]);
    }
  }
  // tokens of the run that the walk could not finish (the tensor ends before their last tap)
#pragma unroll
  for (int d = 0; d < KS - 1; ++d) {
    const int u = t2 - 1 - d;
    if (u >= t0 && u < t1) Elem<T>::st8(dxp + (int64_t)u * p.C + c, dxr[d]);
  }
  if (p.dw_part) {
    float wv[8 * KS];
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int j = 0; j < KS; ++j) wv[e * KS + j] = dw[j][e];
#pragma unroll
    for (int i = 0; i < KS; ++i) Elem<float>::st8(p.dw_part + ((int64_t)run * p.C + c) * KS + 8 * i, wv + 8 * i);
  }
  if (p.db_part) Elem<float>::st8(p.db_part + (int64_t)run * p.C + c, db);
}

template <typename T>
int launch_short_conv(const SC& p, int KS, bool bwd, hipStream_t st) {
  const int c8n = p.C / 8;
  if (!bwd) {
    const dim3 grid((p.T_tot + SCF_RUN - 1) / SCF_RUN, (c8n + 255) / 256);
    if (KS == 2) hipLaunchKernelGGL((short_conv_kernel<T, 2>), grid, dim3(256), 0, st, p);
    else if (KS == 3) hipLaunchKernelGGL((short_conv_kernel<T, 3>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((short_conv_kernel<T, 4>), grid, dim3(256), 0, st, p);
  } else {
    const dim3 grid((p.T_tot + SC_RUN - 1) / SC_RUN, (c8n + 255) / 256);
    if (KS == 2) hipLaunchKernelGGL((short_conv_bwd_kernel<T, 2>), grid, dim3(256), 0, st, p);
    else if (KS == 3) hipLaunchKernelGGL((short_conv_bwd_kernel<T, 3>), grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL((short_conv_bwd_kernel<T, 4>), grid, dim3(256), 0, st, p);
  }
  return 0;
}

}  // namespace

int layer_prologue_impl(const NhaLayerPrologueArgs* a) {
  LP p = {};
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

int layer_prologue_bwd_impl(const NhaLayerPrologueBwdArgs* a) {
  LP p = {};
  p.q = a->q; p.k = a->k; p.v = a->v; p.f = a->f;
  p.dq_swa = a->dq_swa; p.dk_swa = a->dk_swa;
  p.dq_gsa = a->feature_map ? a->dq_gsa : nullptr;
  p.dk_gsa = a->feature_map ? a->dk_gsa : nullptr;
  p.dv_out = a->dv_out; p.ds = a->ds; p.dg = a->dg;
  p.dq = a->dq; p.dk = a->dk; p.dv = a->dv; p.df = a->df;
  p.inv_freq = a->inv_freq;
  p.cu = a->cu_seqlens;
  p.T_tot = a->T_tot; p.N = a->N; p.T = a->T_tot / a->N;
  p.HQ = a->HQ; p.H = a->H; p.K = a->K; p.V = a->V; p.M = a->M;
  p.fm = a->feature_map; p.off = a->seqlen_offset;
  p.inv_norm = 1.f / a->gate_logit_normalizer;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch_prologue_bwd<bf16_t>(p, st);
  else launch_prologue_bwd<float>(p, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_layer_prologue_bwd: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}

int layer_epilogue_bwd_parts(int rows) { return (rows + BWD_ROWS - 1) / BWD_ROWS; }

int short_conv_bwd_parts(int T_tot) { return (T_tot + SC_RUN - 1) / SC_RUN; }

int short_conv_impl(const NhaShortConvArgs* a) {
  SC p = {};
  p.x = a->x; p.w = a->weight; p.b = a->bias; p.y = a->y; p.cu = a->cu_seqlens;
  p.T_tot = a->T_tot; p.N = a->N; p.T = a->T_tot / a->N; p.C = a->C; p.act = a->activation;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch_short_conv<bf16_t>(p, a->KS, false, st);
  else launch_short_conv<float>(p, a->KS, false, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_short_conv: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}

int short_conv_bwd_impl(const NhaShortConvBwdArgs* a) {
  SC p = {};
  p.x = a->x; p.w = a->weight; p.b = a->bias; p.dy = a->dy; p.dx = a->dx;
  p.dw_part = a->dweight_partial; p.db_part = a->dbias_partial; p.cu = a->cu_seqlens;
  p.T_tot = a->T_tot; p.N = a->N; p.T = a->T_tot / a->N; p.C = a->C; p.act = a->activation;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch_short_conv<bf16_t>(p, a->KS, true, st);
  else launch_short_conv<float>(p, a->KS, true, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_short_conv_bwd: launch failed: %s", hipGetErrorString(e));
    return NHA_ERR_LAUNCH;
  }
  return NHA_OK;
}


int layer_epilogue_bwd_impl(const NhaLayerEpilogueBwdArgs* a) {
  if (a->dim % 8 != 0 || a->dim > 8192) {
    set_error("nha_layer_epilogue_bwd: dim must be a multiple of 8 and <= 8192, got %d", a->dim);
    return NHA_ERR_UNSUPPORTED;
  }
  EPB p;
  p.o = a->o; p.dy = a->dy; p.dout = a->dout; p.w = a->weight; p.dw_part = a->dweight_partial; p.db_part = a->dbias_partial;
  p.rows = a->rows; p.dim = a->dim; p.eps = a->eps;
  hipStream_t st = (hipStream_t)a->stream;
  if (a->dtype == NHA_DTYPE_BF16) launch_epilogue_bwd<bf16_t>(p, st);
  else launch_epilogue_bwd<float>(p, st);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("nha_layer_epilogue_bwd: launch failed: %s", hipGetErrorString(e));
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
