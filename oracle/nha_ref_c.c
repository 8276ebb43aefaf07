/* CPU restatement in plain C of the NHA prefill: per-token slot recurrence, causal left window, ONE
 * softmax over [M slots | window].  TEST INFRASTRUCTURE ONLY: it is the checker's second,
 * independent implementation (pinned against oracle/nha_ref.py in tests/test_oracle_pins.py) and
 * the timed leg of bench.py's cpu_baseline; nothing in the shipped package loads it.
 *
 * Semantics restated (citations relative to the reference checkout):
 *   slot write  h <- h * exp(g) + k (x) s, hv likewise      scripts/verify_opt_parity.py:76-85
 *   slot read + window under one softmax                    scripts/verify_opt_parity.py:147-191
 *   (window_size_left, gsa_kv_shift) generalisation          nha_fla/ops/nha/chunk.py:53-78, :401-470
 *   q-head hq reads kv-head hq / NG                          scripts/verify_opt_parity.py:43-46
 *
 * Tensors are float32, packed token-major: q_* [T_tot][HQ][K], k_* [T_tot][H][K], v [T_tot][H][V],
 * s, g [T_tot][H][M]; cu [N+1]; optional h0k [N][H][K][M], h0v [N][H][M][V]; outputs o
 * [T_tot][HQ][V], lse_swa / lse_gsa [T_tot][HQ], optional hkt / hvt like h0k / h0v.  Arithmetic in
 * double.  One OpenMP task per (sequence, q-head); each carries its kv-head's recurrence itself.
 * Returns 0, or -1 when memory runs out. */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

int nha_prefill_ref_c(const float* q_swa, const float* k_swa, const float* q_gsa, const float* k_gsa, const float* v,
                      const float* s, const float* g, const int32_t* cu, int N, int HQ, int H, int K, int V, int M, int wl,
                      int shift, double scale, const float* h0k, const float* h0v, float* o, float* lse_swa, float* lse_gsa,
                      float* hkt, float* hvt) {
  const int NG = HQ / H;
  int failed = 0;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int n = 0; n < N; ++n) {
    for (int hq = 0; hq < HQ; ++hq) {
      const int h = hq / NG;
      const int bos = cu[n], eos = cu[n + 1], L = eos - bos;
      const int wmax = (wl < 0 || wl + 1 > L) ? L : wl + 1;
      double* hk = (double*)calloc((size_t)K * M, sizeof(double));   /* [K][M] */
      double* hv = (double*)calloc((size_t)M * V, sizeof(double));   /* [M][V] */
      double* lg = (double*)malloc(((size_t)M + wmax + V + M) * sizeof(double));
      if (!hk || !hv || !lg) {
#pragma omp atomic write
        failed = 1;
        free(hk); free(hv); free(lg);
        continue;
      }
      double* u = lg;            /* [M] slot logits */
      double* w = lg + M;        /* [wmax] window logits */
      double* acc = w + wmax;    /* [V] */
      double* eg = acc + V;      /* [M] */
      if (h0k)
        for (int i = 0; i < K * M; ++i) hk[i] = h0k[((size_t)n * H + h) * K * M + i];
      if (h0v)
        for (int i = 0; i < M * V; ++i) hv[i] = h0v[((size_t)n * H + h) * M * V + i];
      for (int t = bos; t < eos; ++t) {
        const int j = t - shift;   /* the token entering the slots at step t */
        if (j >= bos) {
          const float* gj = g + ((size_t)j * H + h) * M;
          const float* sj = s + ((size_t)j * H + h) * M;
          const float* kj = k_gsa + ((size_t)j * H + h) * K;
          const float* vj = v + ((size_t)j * H + h) * V;
          for (int m = 0; m < M; ++m) eg[m] = exp((double)gj[m]);
          for (int d = 0; d < K; ++d)
            for (int m = 0; m < M; ++m) hk[d * M + m] = hk[d * M + m] * eg[m] + (double)kj[d] * sj[m];
          for (int m = 0; m < M; ++m)
            for (int c = 0; c < V; ++c) hv[m * V + c] = hv[m * V + c] * eg[m] + (double)sj[m] * vj[c];
        }
        const float* qg = q_gsa + ((size_t)t * HQ + hq) * K;
        const float* qs = q_swa + ((size_t)t * HQ + hq) * K;
        for (int m = 0; m < M; ++m) u[m] = 0.0;
        for (int d = 0; d < K; ++d) {
          const double qd = scale * qg[d];
          for (int m = 0; m < M; ++m) u[m] += qd * hk[d * M + m];
        }
        int lo = (wl < 0) ? bos : t - wl;
        if (lo < bos) lo = bos;
        const int nw = t - lo + 1;
        double mu = -INFINITY, mw = -INFINITY;
        for (int m = 0; m < M; ++m) mu = u[m] > mu ? u[m] : mu;
        for (int x = 0; x < nw; ++x) {
          const float* kx = k_swa + ((size_t)(lo + x) * H + h) * K;
          double a = 0.0;
          for (int d = 0; d < K; ++d) a += (double)qs[d] * kx[d];
          w[x] = scale * a;
          mw = w[x] > mw ? w[x] : mw;
        }
        const double mx = mu > mw ? mu : mw;
        double zu = 0.0, zw = 0.0;
        for (int c = 0; c < V; ++c) acc[c] = 0.0;
        for (int m = 0; m < M; ++m) {
          const double p = exp(u[m] - mx);
          zu += p;
          for (int c = 0; c < V; ++c) acc[c] += p * hv[m * V + c];
        }
        for (int x = 0; x < nw; ++x) {
          const double p = exp(w[x] - mx);
          zw += p;
          const float* vx = v + ((size_t)(lo + x) * H + h) * V;
          for (int c = 0; c < V; ++c) acc[c] += p * vx[c];
        }
        const double z = zu + zw;
        float* ot = o + ((size_t)t * HQ + hq) * V;
        for (int c = 0; c < V; ++c) ot[c] = (float)(acc[c] / z);
        lse_gsa[(size_t)t * HQ + hq] = (float)(mx + log(zu));
        lse_swa[(size_t)t * HQ + hq] = (float)(mx + log(zw));
      }
      if (hq % NG == 0) {
        if (hkt)
          for (int i = 0; i < K * M; ++i) hkt[((size_t)n * H + h) * K * M + i] = (float)hk[i];
        if (hvt)
          for (int i = 0; i < M * V; ++i) hvt[((size_t)n * H + h) * M * V + i] = (float)hv[i];
      }
      free(hk); free(hv); free(lg);
    }
  }
  return failed ? -1 : 0;
}
