// Shape-generic NHA prefill for gfx950 in fp32 VALU arithmetic (any K, V, M, window, shift; GQA;
// varlen).  It serves the fp32 path (1e-4 relative against the fp64 recurrence), every shape
// the MFMA kernels are not built for, and an independent on-device cross-check of the MFMA
// kernels at sizes a CPU recurrence cannot reach.  Two launches:
//
//   state pass  : per (sequence, kv-head, 16-slot block) a sweep over 64-row chunks: chunk-local
//                 inclusive gate cumsum gc, chunk-start states, h <- h*exp(gc_last) +
//                 K^T (S*exp(gc_last-gc))        (nha_fla/ops/nha/chunk_fused.py:83-107)
//   output pass : per (token, q-head): slot logits from the chunk-start state plus the
//                 intra-chunk terms with the exact decay exp(gc_i-gc_j) <= 1 (chunk_fused.py:186-222),
//                 window logits, ONE softmax over [M | window] (:233-240), slot read + window
//                 read (:242-283), and the two branch LSEs the reference returns
//                 (nha_fla/ops/nha/chunk.py:459-470, :488).
// Rows of the slot branch are read at t - shift (zero rows before the sequence start,
// nha_fla/ops/nha/chunk.py:53-78).
#include "common.h"

namespace nha {
namespace {

constexpr int BT = 64;   // chunk rows
constexpr int BMS = 16;  // slots per state-pass workgroup

struct SP {
  const void *q_swa, *k_swa, *q_gsa, *k_gsa, *v, *s, *g;
  void* o;
  float *lse_swa, *lse_gsa;
  const float *h0k, *h0v;
  float *hkt, *hvt;
  const int32_t *cu, *cidx, *coff;
  float *gc, *hkc, *hvc;  // scratch
  int T_tot, N, NT, HQ, H, K, V, M, wl, shift;
  float scale;
};

template <typename T>
__global__ __launch_bounds__(256) void simple_state_kernel(const SP p) {
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, V = p.V, M = p.M, H = p.H;
  float* hk = lds;              // [K][BMS]
  float* hv = hk + K * BMS;     // [BMS][V]
  float* gcl = hv + BMS * V;    // [BT][BMS]
  float* sd = gcl + BT * BMS;   // [BT][BMS]
  int* src = (int*)(sd + BT * BMS);  // [BT]
  const int tid = threadIdx.x;
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const int mb = blockIdx.y * BMS;
  const int bm = (M - mb) < BMS ? (M - mb) : BMS;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int L = eos - bos;
  const int nchunks = (L + BT - 1) / BT;
  const int c0 = p.coff[n];
  const T* kg = (const T*)p.k_gsa;
  const T* vv_ = (const T*)p.v;
  const T* ss = (const T*)p.s;
  const T* gg = (const T*)p.g;

  for (int e = tid; e < K * bm; e += 256) {
    const int kk = e / bm, m = e - kk * bm;
    hk[kk * BMS + m] = p.h0k ? p.h0k[(((int64_t)n * H + h) * K + kk) * M + mb + m] : 0.f;
  }
  for (int e = tid; e < bm * V; e += 256) {
    const int m = e / V, c = e - m * V;
    hv[m * V + c] = p.h0v ? p.h0v[(((int64_t)n * H + h) * M + mb + m) * V + c] : 0.f;
  }
  __syncthreads();

  for (int it = 0; it < nchunks; ++it) {
    const int rows = (L - it * BT) < BT ? (L - it * BT) : BT;
    if (tid < BT) {
      const int tl = it * BT + tid - p.shift;
      src[tid] = (tid < rows && tl >= 0) ? bos + tl : -1;
    }
    __syncthreads();
    if (tid < bm) {
      float run = 0.f;
      for (int j = 0; j < rows; ++j) {
        const int sj = src[j];
        if (sj >= 0) run += Elem<T>::ld(gg + ((int64_t)sj * H + h) * M + mb + tid);
        gcl[j * BMS + tid] = run;
        p.gc[((int64_t)(bos + it * BT + j) * H + h) * M + mb + tid] = run;
      }
    }
    // chunk-start states
    const int64_t cg = (int64_t)(c0 + it) * H + h;
    for (int e = tid; e < K * bm; e += 256) {
      const int kk = e / bm, m = e - kk * bm;
      p.hkc[(cg * K + kk) * M + mb + m] = hk[kk * BMS + m];
    }
    for (int e = tid; e < bm * V; e += 256) {
      const int m = e / V, c = e - m * V;
      p.hvc[(cg * M + mb + m) * V + c] = hv[m * V + c];
    }
    __syncthreads();
    for (int e = tid; e < rows * bm; e += 256) {
      const int j = e / bm, m = e - j * bm;
      const int sj = src[j];
      const float gl = gcl[(rows - 1) * BMS + m];
      sd[j * BMS + m] = sj >= 0 ? Elem<T>::ld(ss + ((int64_t)sj * H + h) * M + mb + m) * expf(gl - gcl[j * BMS + m]) : 0.f;
    }
    __syncthreads();
    for (int e = tid; e < K * bm; e += 256) {
      const int kk = e / bm, m = e - kk * bm;
      float acc = hk[kk * BMS + m] * expf(gcl[(rows - 1) * BMS + m]);
      for (int j = 0; j < rows; ++j) {
        const int sj = src[j];
        if (sj >= 0) acc += Elem<T>::ld(kg + ((int64_t)sj * H + h) * K + kk) * sd[j * BMS + m];
      }
      hk[kk * BMS + m] = acc;
    }
    for (int e = tid; e < bm * V; e += 256) {
      const int m = e / V, c = e - m * V;
      float acc = hv[m * V + c] * expf(gcl[(rows - 1) * BMS + m]);
      for (int j = 0; j < rows; ++j) {
        const int sj = src[j];
        if (sj >= 0) acc += sd[j * BMS + m] * Elem<T>::ld(vv_ + ((int64_t)sj * H + h) * V + c);
      }
      hv[m * V + c] = acc;
    }
    __syncthreads();
  }
  if (p.hkt)
    for (int e = tid; e < K * bm; e += 256) {
      const int kk = e / bm, m = e - kk * bm;
      p.hkt[(((int64_t)n * H + h) * K + kk) * M + mb + m] = hk[kk * BMS + m];
    }
  if (p.hvt)
    for (int e = tid; e < bm * V; e += 256) {
      const int m = e / V, c = e - m * V;
      p.hvt[(((int64_t)n * H + h) * M + mb + m) * V + c] = hv[m * V + c];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void simple_out_kernel(const SP p) {
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, V = p.V, M = p.M, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  float* qg = lds;            // [K] scaled slot-branch query
  float* qs = qg + K;         // [K] scaled window query
  float* gct = qs + K;        // [M]
  float* okl = gct + M;       // [M] slot logits -> slot probabilities
  float* Aj = okl + M;        // [BT]
  float* Avj = Aj + BT;       // [BT]
  float* pw = Avj + BT;       // [256]
  float* red = pw + 256;      // [4]
  int* src = (int*)(red + 4); // [BT]
  const int tid = threadIdx.x;
  const int chunk = blockIdx.x / BT, r = blockIdx.x % BT;
  const int hq = blockIdx.y, h = hq / NG;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int t = bos + it * BT + r;
  if (t >= eos) return;
  const T* qsw = (const T*)p.q_swa + ((int64_t)t * HQ + hq) * K;
  const T* qgs = (const T*)p.q_gsa + ((int64_t)t * HQ + hq) * K;
  const T* ksw = (const T*)p.k_swa;
  const T* kgs = (const T*)p.k_gsa;
  const T* vv_ = (const T*)p.v;
  const T* ss = (const T*)p.s;
  for (int i = tid; i < K; i += 256) {
    qg[i] = Elem<T>::ld(qgs + i) * p.scale;
    qs[i] = Elem<T>::ld(qsw + i) * p.scale;
  }
  for (int i = tid; i < M; i += 256) gct[i] = p.gc[((int64_t)t * H + h) * M + i];
  if (tid < BT) {
    const int tl = it * BT + tid - p.shift;
    src[tid] = (tid <= r && tl >= 0) ? bos + tl : -1;
  }
  __syncthreads();
  // intra-chunk scores against the slot-branch keys of rows <= r
  if (tid < BT) {
    const int sj = src[tid];
    Aj[tid] = sj >= 0 ? dot_row<T>(qg, kgs + ((int64_t)sj * H + h) * K, K) : 0.f;
  }
  __syncthreads();
  // slot logits
  const float* hk0 = p.hkc + ((int64_t)chunk * H + h) * K * M;
  const float* gcb = p.gc + ((int64_t)(bos + it * BT) * H + h) * M;
  float lmax = -INFINITY;
  for (int m = tid; m < M; m += 256) {
    float acc = 0.f;
    for (int kk = 0; kk < K; ++kk) acc += qg[kk] * hk0[(int64_t)kk * M + m];
    acc *= expf(gct[m]);
    for (int j = 0; j <= r; ++j) {
      const int sj = src[j];
      if (sj >= 0)
        acc += Aj[j] * Elem<T>::ld(ss + ((int64_t)sj * H + h) * M + m) * expf(gct[m] - gcb[(int64_t)j * H * M + m]);
    }
    okl[m] = acc;
    lmax = fmaxf(lmax, acc);
  }
  const float mg = block_max(lmax, red);
  float lsum = 0.f;
  for (int m = tid; m < M; m += 256) lsum += expf(okl[m] - mg);
  const float lg = block_sum(lsum, red);
  // window statistics (pass 1)
  const int lo = p.wl < 0 ? bos : (t - p.wl > bos ? t - p.wl : bos);
  float wm = -INFINITY, wsum = 0.f;
  for (int j = lo + tid; j <= t; j += 256) {
    const float d = dot_row<T>(qs, ksw + ((int64_t)j * H + h) * K, K);
    if (d > wm) {
      wsum = wsum * expf(wm - d) + 1.f;
      wm = d;
    } else {
      wsum += expf(d - wm);
    }
  }
  const float mw = block_max(wm, red);
  const float lw = block_sum(wm == -INFINITY ? 0.f : wsum * expf(wm - mw), red);
  if (tid == 0) {
    if (p.lse_gsa) p.lse_gsa[(int64_t)t * HQ + hq] = mg + logf(lg);
    if (p.lse_swa) p.lse_swa[(int64_t)t * HQ + hq] = mw + logf(lw);
  }
  const float mt = fmaxf(mg, mw);
  const float inv = 1.f / (lg * expf(mg - mt) + lw * expf(mw - mt));
  __syncthreads();
  for (int m = tid; m < M; m += 256) okl[m] = expf(okl[m] - mt) * inv;
  __syncthreads();
  // slot-read weights of the intra-chunk rows
  if (tid < BT) {
    const int sj = src[tid];
    float acc = 0.f;
    if (sj >= 0) {
      const T* srow = ss + ((int64_t)sj * H + h) * M;
      const float* gj = gcb + (int64_t)tid * H * M;
      for (int m = 0; m < M; ++m) acc += okl[m] * Elem<T>::ld(srow + m) * expf(gct[m] - gj[m]);
    }
    Avj[tid] = acc;
  }
  __syncthreads();
  // output: at most 4 value columns per thread per sweep (V <= 1024)
  const float* hv0 = p.hvc + ((int64_t)chunk * H + h) * M * V;
  for (int cb = 0; cb < V; cb += 1024) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int u = 0; u < 4; ++u) {
      const int c = cb + tid + 256 * u;
      if (c < V) {
        float a0 = 0.f;
        for (int m = 0; m < M; ++m) a0 += okl[m] * expf(gct[m]) * hv0[(int64_t)m * V + c];
        for (int j = 0; j <= r; ++j) {
          const int sj = src[j];
          if (sj >= 0) a0 += Avj[j] * Elem<T>::ld(vv_ + ((int64_t)sj * H + h) * V + c);
        }
        acc[u] = a0;
      }
    }
    for (int jb = lo; jb <= t; jb += 256) {
      const int j = jb + tid;
      __syncthreads();
      pw[tid] = j <= t ? expf(dot_row<T>(qs, ksw + ((int64_t)j * H + h) * K, K) - mt) * inv : 0.f;
      __syncthreads();
      const int cnt = (t - jb + 1) < 256 ? (t - jb + 1) : 256;
      for (int u = 0; u < 4; ++u) {
        const int c = cb + tid + 256 * u;
        if (c < V) {
          float a0 = acc[u];
          for (int x = 0; x < cnt; ++x) a0 += pw[x] * Elem<T>::ld(vv_ + ((int64_t)(jb + x) * H + h) * V + c);
          acc[u] = a0;
        }
      }
    }
    for (int u = 0; u < 4; ++u) {
      const int c = cb + tid + 256 * u;
      if (c < V) Elem<T>::st((T*)p.o + ((int64_t)t * HQ + hq) * V + c, acc[u]);
    }
  }
}

static size_t aligned(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

size_t prefill_simple_scratch_bytes(const NhaPrefillArgs* a) {
  const size_t gc = aligned((size_t)a->T_tot * a->H * a->M * 4);
  const size_t hk = aligned((size_t)a->NT * a->H * a->K * a->M * 4);
  const size_t hv = aligned((size_t)a->NT * a->H * a->M * a->V * 4);
  return gc + hk + hv;
}

template <typename T>
static int run_simple(const NhaPrefillArgs* a, int phase) {
  SP p;
  p.q_swa = a->q_swa; p.k_swa = a->k_swa; p.q_gsa = a->q_gsa; p.k_gsa = a->k_gsa;
  p.v = a->v; p.s = a->s; p.g = a->g; p.o = a->o;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa;
  p.h0k = a->h0k; p.h0v = a->h0v; p.hkt = a->hkt; p.hvt = a->hvt;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices; p.coff = a->chunk_offsets;
  char* sc = (char*)a->scratch;
  p.gc = (float*)sc;
  sc += aligned((size_t)a->T_tot * a->H * a->M * 4);
  p.hkc = (float*)sc;
  sc += aligned((size_t)a->NT * a->H * a->K * a->M * 4);
  p.hvc = (float*)sc;
  p.T_tot = a->T_tot; p.N = a->N; p.NT = a->NT; p.HQ = a->HQ; p.H = a->H;
  p.K = a->K; p.V = a->V; p.M = a->M; p.wl = a->wl; p.shift = a->shift; p.scale = a->scale;
  hipStream_t st = (hipStream_t)a->stream;

  const size_t lds1 = ((size_t)a->K * BMS + (size_t)BMS * a->V + 2 * BT * BMS) * 4 + BT * 4;
  const size_t lds2 = ((size_t)2 * a->K + 2 * a->M + 2 * BT + 256 + 4) * 4 + BT * 4;
  if (lds1 > 64 * 1024 || lds2 > 64 * 1024) {
    set_error("nha_prefill_fwd(simple): head dims too large for the generic kernels (K=%d V=%d M=%d)", a->K, a->V, a->M);
    return NHA_ERR_UNSUPPORTED;
  }
  if (phase != 2) {
    hipLaunchKernelGGL((simple_state_kernel<T>), dim3(a->N * a->H, (a->M + BMS - 1) / BMS), dim3(256), lds1, st, p);
    NHA_CHECK_LAUNCH("nha_prefill_fwd(simple state pass)");
  }
  if (phase != 1) {
    hipLaunchKernelGGL((simple_out_kernel<T>), dim3(a->NT * BT, a->HQ), dim3(256), lds2, st, p);
    NHA_CHECK_LAUNCH("nha_prefill_fwd(simple output pass)");
  }
  return NHA_OK;
}

int prefill_simple_impl(const NhaPrefillArgs* a, int phase) {
  if (a->V > 1024 * 64) {
    set_error("nha_prefill_fwd(simple): V too large");
    return NHA_ERR_UNSUPPORTED;
  }
  if (a->dtype == NHA_DTYPE_BF16) return run_simple<bf16_t>(a, phase);
  return run_simple<float>(a, phase);
}

}  // namespace nha
