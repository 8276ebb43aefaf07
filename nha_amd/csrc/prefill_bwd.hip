// Backward of the chunked NHA prefill for gfx950, fp32 VALU arithmetic (any K, V <= 256, M <= 64;
// fp32 or bf16 tensors; GQA; varlen).  Replaces ChunkNativeHybridAttentionFunction.backward
// (nha_fla/ops/nha/chunk.py:490-564): window-branch gradients (:499-511), slot-branch gradients
// with the merged-softmax coupling (:514-530; chunk_gsa.py:52-122), un-shifting (:533-543) and the
// accumulation of dv over both branches (:559) -- as ONE differentiation of the merged softmax
// instead of two branch backwards glued by an LSE correction.
//
// Per token t and q-head a (kv-head h, slot-branch rows read at src = t - shift):
//   u[m] = scale q_gsa . hk_t[:,m]      w[j] = scale q_swa . k_swa_j       lse = log(sum e^u + sum e^w)
//   p = e^(u-lse)   pi = e^(w-lse)      o = p hv_t + pi v
//   delta = do . o      dp[m] = do . hv_t[m,:]      dpi[j] = do . v_j
//   du = p (dp - delta) + dlse_gsa e^(u-lse_gsa)     dw = pi (dpi - delta) + dlse_swa e^(w-lse_swa)
// and the state recurrences hk_t = hk_(t-1) e^g + k' s^T, hv_t = e^g hv_(t-1) + s v'^T run backward
// in chunk form.  With Dh_r the total gradient of the state after row r,
//   dk'_r = Dhk_r s_r     dv'_r = s_r^T Dhv_r     ds_r = k'_r^T Dhk_r + Dhv_r v'_r
//   dg_r  = dg_(r+1) + sum_a (du u + p dp)_r - s_r ds_r        (dg past the end = <dh_T, h_T>)
// (the last line is the usual reverse cumulative sum of gated linear attention: <Dh_r, h_r> telescopes).
//
// Launches: forward state pass (chunk-start states, gate cumsums) -> bwd_q_kernel (per token: the
// vectors du, p) -> bwd_intra_kernel (per chunk: intra-chunk matrices and the intra part of ds)
// -> bwd_dqg_kernel (per token: dq_gsa) -> bwd_state_{direct,scan,inter}_kernel (state gradients as a linear recurrence over
// chunks: dk_gsa, slot-branch dv, inter-chunk part of ds, dh0) -> bwd_gate_*_kernel (reverse scan: ds, dg)
// -> bwd_kv_window_kernel (per key: dk_swa, dv).  For bf16 tensors with K == V in {64,128,256} the
// window parts (dq_swa, dk_swa, dv) run on the matrix cores instead (prefill_bwd_mfma.hip).
#include "common.h"

namespace nha {
namespace {

constexpr int BT = 64;   // chunk rows
constexpr int CB = 32;   // state columns per workgroup of the state-gradient sweep

struct BP {
  const void *q_swa, *k_swa, *q_gsa, *k_gsa, *v, *s, *g, *o, *dout;
  const float *lse_swa, *lse_gsa, *dlse_swa, *dlse_gsa, *dhkt, *dhvt;
  void *dq_swa, *dk_swa, *dq_gsa, *dk_gsa, *dv, *ds, *dg;
  float *dh0k, *dh0v;
  const int32_t *cu, *cidx, *coff;
  // forward recomputation (layout of the generic forward state pass)
  float *gc;          // [T_tot][H][M]      chunk-local inclusive gate cumsum, indexed by row token
  float *hkc, *hvc;   // [NT][H][K][M], [NT][H][M][V]   chunk-start states
  float *hkct, *hvct; // [NT][H][M][K], [NT][H][V][M]   the same, transposed
  float *hkT, *hvT;   // [N][H][K][M], [N][H][M][V]     final states (for the end term of dg)
  // per-token vectors of the slot branch
  float *dus, *pp, *xg;   // [T_tot][HQ][M]   scale*du, p, du*u + p*dp
  float *delta;           // [T_tot][HQ]
  float *ck, *cv;         // [NT][HQ][BT][BT]  sum_m dus_i s_r e^(gc_i-gc_r), same with p   (i >= r)
  float *dsi;             // [T_tot][H][M]     intra-chunk part of ds, indexed by row token
  float *dsp;             // [nbk+nbv][T_tot][H][M]  inter-chunk part of ds per column block
  float *dvs;             // [T_tot][H][V]     slot-branch dv, indexed by SOURCE token
  const bf16_t *ap, *bp;  // [NT][HQ][BT][BT]  q_gsa_i . k'_j and do_i . v'_j from the matrix cores (bf16), or NULL
  const float *ust, *dpst; // [T_tot][HQ][M]    q_gsa_t . hk0[:,m] and do_t . hv0[m,:] (chunk-start states), or NULL
  const int* big;         // [NT][H] chunks the matrix-core slot kernels leave to the VALU kernels, or NULL (all)
  float *gtot;            // [NT][H][M]        chunk sums of the dg summand, then sums of all later chunks
  float *dks;             // [T_tot][H][K]     intra-chunk part of dk_gsa, indexed by SOURCE token
  float *ek, *ev;         // [NT][H][K][M], [NT][H][V][M]  N_c, then E_c (see the state-gradient kernels)
  int T_tot, N, NT, HQ, H, K, V, M, wl, shift, nbk, nbv;
  float scale;
};

// dot product of two global rows of n elements (n a multiple of 8, rows 16-byte aligned)
template <typename T>
__device__ __forceinline__ float dot_rows(const T* a, const T* b, int n) {
  float acc = 0.f;
  for (int i = 0; i < n; i += 8) {
    float x[8], y[8];
    Elem<T>::ld8(a + i, x);
    Elem<T>::ld8(b + i, y);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += x[e] * y[e];
  }
  return acc;
}

__device__ __forceinline__ float logaddexp_f(float a, float b) {
  const float mx = fmaxf(a, b);
  return mx + logf(expf(a - mx) + expf(b - mx));
}

// ------------------------------------------------------------------------------------------
// per (token, q-head), ONE WAVE each (4 tokens per workgroup): the vectors du, p (and du u + p dp)
// the other passes are built from.  Lanes run over the slots m (M <= 64) or over the rows j of
// the chunk, so that every global read of a state is coalesced: hkc [K][M] for u, hvct [V][M] for
// dp (bwd_dqg_kernel reads hkct [M][K]).
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_q_kernel(const BP p) {
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, V = p.V, M = p.M, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  float* qg = lds + wv * (K + V + 2 * BT + M);   // [K] scaled slot-branch query
  float* dov = qg + K;        // [V]
  float* Aj = dov + V;        // [BT] q_gsa . k'_j
  float* Bj = Aj + BT;        // [BT] do . v'_j
  float* gct = Bj + BT;       // [M]
  // Two launch shapes.  Alone (no flags): grid (NT * 16, HQ), one wave per (token, q-head).  Behind
  // the matrix-core kernel: grid (NT, H), a workgroup leaves at once unless its (chunk, kv-head) is
  // flagged and otherwise walks the chunk's 64 * NG (token, q-head) pairs, four at a time.
  const bool looped = p.big != nullptr;
  const int chunk = looped ? blockIdx.x : blockIdx.x / (BT / 4);
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  if (looped && !p.big[(int64_t)chunk * H + blockIdx.y]) return;   // the matrix-core kernel has done this chunk
  const int nit = looped ? BT * NG / 4 : 1;
  for (int itx = 0; itx < nit; ++itx) {
  if (itx) __syncthreads();   // the previous pair's vectors in LDS are no longer read
  const int item = 4 * itx + wv;
  const int r = looped ? item % BT : (blockIdx.x % (BT / 4)) * 4 + wv;
  const int hq = looped ? blockIdx.y * NG + item / BT : blockIdx.y;
  const int h = hq / NG;
  const bool valid = bos + it * BT + r < eos;   // waves past the end compute on row 0 and write nothing
  const int rr = valid ? r : 0;
  const int t = bos + it * BT + rr;
  const T* kgs = (const T*)p.k_gsa;
  const T* vv_ = (const T*)p.v;
  const T* ss = (const T*)p.s;
  const int64_t tq = (int64_t)t * HQ + hq;
  float dl = 0.f;
  for (int i = lane; i < K; i += 64) qg[i] = Elem<T>::ld((const T*)p.q_gsa + tq * K + i) * p.scale;
  for (int i = lane; i < V; i += 64) {
    const float d = Elem<T>::ld((const T*)p.dout + tq * V + i);
    dov[i] = d;
    dl += d * Elem<T>::ld((const T*)p.o + tq * V + i);
  }
  if (lane < M) gct[lane] = p.gc[((int64_t)t * H + h) * M + lane];
  const float delta = wave_sum(dl);
  __syncthreads();
  const int tl0 = it * BT - p.shift;   // sequence-local source index of row 0 (negative: no source)
  {
    const int j = lane;
    const bool has = j <= rr && tl0 + j >= 0;
    const int64_t sj = (int64_t)bos + tl0 + j;
    if (p.ap) {
      const int64_t pi = (((int64_t)chunk * HQ + hq) * BT + rr) * BT + j;
      Aj[j] = has ? bf16_to_f32(p.ap[pi]) * p.scale : 0.f;
      Bj[j] = has ? bf16_to_f32(p.bp[pi]) : 0.f;
    } else {
      Aj[j] = has ? dot_row<T>(qg, kgs + (sj * H + h) * K, K) : 0.f;
      Bj[j] = has ? dot_row<T>(dov, vv_ + (sj * H + h) * V, V) : 0.f;
    }
  }
  __syncthreads();
  const float* hk0 = p.hkc + ((int64_t)chunk * H + h) * K * M;
  const float* hv0t = p.hvct + ((int64_t)chunk * H + h) * V * M;
  const float* gcb = p.gc + ((int64_t)(bos + it * BT) * H + h) * M;
  const float ls = p.lse_swa[tq], lg = p.lse_gsa[tq];
  const float lt = logaddexp_f(ls, lg);
  const float dlg = p.dlse_gsa ? p.dlse_gsa[tq] : 0.f;
  if (lane < M) {
    const int m = lane;
    float au = 0.f, ad = 0.f;
    if (p.ust) {
      au = p.ust[tq * M + m] * p.scale;
      ad = p.dpst[tq * M + m];
    } else {
#pragma unroll 8
      for (int kk = 0; kk < K; ++kk) au += qg[kk] * hk0[(int64_t)kk * M + m];
#pragma unroll 8
      for (int c = 0; c < V; ++c) ad += dov[c] * hv0t[(int64_t)c * M + m];
    }
    const float gm = gct[m];
    const float e = expf(gm);
    au *= e;
    ad *= e;
    const int jlo = tl0 < 0 ? -tl0 : 0;
    for (int j = jlo; j <= rr; ++j) {
      const int64_t sj = (int64_t)bos + tl0 + j;
      const float w = Elem<T>::ld(ss + (sj * H + h) * M + m) * expf(gm - gcb[(int64_t)j * H * M + m]);
      au += Aj[j] * w;
      ad += Bj[j] * w;
    }
    const float pm = expf(au - lt);
    const float du = pm * (ad - delta) + dlg * expf(au - lg);
    if (valid) {
      p.dus[tq * M + m] = p.scale * du;
      p.pp[tq * M + m] = pm;
      p.xg[tq * M + m] = du * au + pm * ad;
    }
  }
  if (lane == 0 && valid) p.delta[tq] = delta;
  }
}

// ------------------------------------------------------------------------------------------
// per (token, q-head), one wave each, after bwd_intra_kernel:
//   dq_gsa[d] = sum_m scale du[m] hk_t[d][m]
//             = sum_m (scale du[m] e^(gc_r[m])) hk0[d][m] + sum_(j<=r) ck[r][j] k'_j[d]
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_dqg_kernel(const BP p) {
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, M = p.M, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  float* due = lds + wv * (M + BT);   // [M] scale * du * e^(gc_r)
  float* Wj = due + M;                // [BT] row r of ck
  const int chunk = blockIdx.x / (BT / 4), r = (blockIdx.x % (BT / 4)) * 4 + wv;
  const int hq = blockIdx.y, h = hq / NG;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const bool valid = bos + it * BT + r < eos;
  const int rr = valid ? r : 0;
  const int t = bos + it * BT + rr;
  const int64_t tq = (int64_t)t * HQ + hq;
  if (lane < M) due[lane] = p.dus[tq * M + lane] * expf(p.gc[((int64_t)t * H + h) * M + lane]);
  Wj[lane] = lane <= rr ? p.ck[(((int64_t)chunk * HQ + hq) * BT + rr) * BT + lane] : 0.f;
  __syncthreads();
  const float* hk0t = p.hkct + ((int64_t)chunk * H + h) * M * K;
  const T* kgs = (const T*)p.k_gsa;
  const int tl0 = it * BT - p.shift;
  const int jlo = tl0 < 0 ? -tl0 : 0;
  for (int d = lane; d < K; d += 64) {
    float acc = 0.f;
#pragma unroll 8
    for (int m = 0; m < M; ++m) acc += due[m] * hk0t[(int64_t)m * K + d];
    for (int j = jlo; j <= rr; ++j) acc += Wj[j] * Elem<T>::ld(kgs + (((int64_t)bos + tl0 + j) * H + h) * K + d);
    if (valid) Elem<T>::st((T*)p.dq_gsa + tq * K + d, acc);
  }
}

// chunk-start states in the transposed layouts bwd_q_kernel reads (generic state pass only; the
// matrix-core state pass exports them directly): hkct [NT][H][M][K], hvct [NT][H][V][M]
__global__ __launch_bounds__(256) void bwd_transpose_states_kernel(const BP p) {
  const int K = p.K, V = p.V, M = p.M;
  const int64_t cg = blockIdx.x;
  const float* hk = p.hkc + cg * K * M;
  const float* hv = p.hvc + cg * M * V;
  for (int e = threadIdx.x; e < K * M; e += 256) {
    const int m = e / K, d = e - m * K;
    p.hkct[cg * M * K + e] = hk[(int64_t)d * M + m];
  }
  for (int e = threadIdx.x; e < V * M; e += 256) {
    const int c = e / M, m = e - c * M;
    p.hvct[cg * V * M + e] = hv[(int64_t)m * V + c];
  }
}

// ------------------------------------------------------------------------------------------
// per (token, q-head): dq_swa in fp32 VALU arithmetic (tensors the matrix-core kernels do not take)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_q_window_kernel(const BP p) {
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, V = p.V, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  float* qs = lds;         // [K] scaled window query
  float* dov = qs + K;     // [V]
  float* pw = dov + V;     // [256]
  const int tid = threadIdx.x;
  const int chunk = blockIdx.x / BT, r = blockIdx.x % BT;
  const int hq = blockIdx.y, h = hq / NG;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int t = bos + it * BT + r;
  if (t >= eos) return;
  const T* ksw = (const T*)p.k_swa;
  const T* vv_ = (const T*)p.v;
  const int64_t tq = (int64_t)t * HQ + hq;
  for (int i = tid; i < K; i += 256) qs[i] = Elem<T>::ld((const T*)p.q_swa + tq * K + i) * p.scale;
  for (int i = tid; i < V; i += 256) dov[i] = Elem<T>::ld((const T*)p.dout + tq * V + i);
  const float ls = p.lse_swa[tq];
  const float lt = logaddexp_f(ls, p.lse_gsa[tq]);
  const float dls = p.dlse_swa ? p.dlse_swa[tq] : 0.f;
  const float delta = p.delta[tq];
  // dq_swa[d] = scale sum_j dw[j] k_swa_j[d]   (K <= 256: one column per thread)
  const int lo = p.wl < 0 ? bos : (t - p.wl > bos ? t - p.wl : bos);
  float acc = 0.f;
  for (int jb = lo; jb <= t; jb += 256) {
    const int j = jb + tid;
    __syncthreads();
    float val = 0.f;
    if (j <= t) {
      const float w = dot_row<T>(qs, ksw + ((int64_t)j * H + h) * K, K);
      const float pi = expf(w - lt);
      const float dpi = dot_row<T>(dov, vv_ + ((int64_t)j * H + h) * V, V);
      val = p.scale * (pi * (dpi - delta) + dls * expf(w - ls));
    }
    pw[tid] = val;
    __syncthreads();
    const int cnt = (t - jb + 1) < 256 ? (t - jb + 1) : 256;
    if (tid < K)
      for (int x = 0; x < cnt; ++x) acc += pw[x] * Elem<T>::ld(ksw + ((int64_t)(jb + x) * H + h) * K + tid);
  }
  if (tid < K) Elem<T>::st((T*)p.dq_swa + tq * K + tid, acc);
}

// ------------------------------------------------------------------------------------------
// per (chunk, kv-head): intra-chunk matrices ck, cv and the intra-chunk part of ds
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(512) void bwd_intra_kernel(const BP p) {
  constexpr int NTHR = 512;   // 8 waves: the tables fill most of the LDS, so one workgroup per CU
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, V = p.V, M = p.M, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  const int LM = M + 1;
  float* gcl = lds;              // [BT][LM]
  float* sl = gcl + BT * LM;     // [BT][LM]
  float* du = sl + BT * LM;      // [BT][LM]
  float* pl = du + BT * LM;      // [BT][LM]
  float* dsl = pl + BT * LM;     // [BT][LM]
  float* Am = dsl + BT * LM;     // [BT][BT+1]  q_gsa_i . k'_r
  float* Bm = Am + BT * (BT + 1);   // [BT][BT+1]  do_i . v'_r
  int* src = (int*)(Bm + BT * (BT + 1));   // [BT]
  const int tid = threadIdx.x;
  const int chunk = blockIdx.x, h = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const T* ss = (const T*)p.s;
  if (p.big && !p.big[(int64_t)chunk * H + h]) return;   // the matrix-core kernel has done this chunk
  if (tid < BT) {
    const int tl = it * BT + tid - p.shift;
    src[tid] = (tid < R && tl >= 0) ? bos + tl : -1;
  }
  __syncthreads();
  for (int e = tid; e < R * M; e += NTHR) {
    const int r = e / M, m = e - r * M;
    gcl[r * LM + m] = p.gc[((int64_t)(c0 + r) * H + h) * M + m];
    const int sj = src[r];
    sl[r * LM + m] = sj >= 0 ? Elem<T>::ld(ss + ((int64_t)sj * H + h) * M + m) : 0.f;
    dsl[r * LM + m] = 0.f;
  }
  for (int a = 0; a < NG; ++a) {
    const int hq = h * NG + a;
    __syncthreads();
    for (int e = tid; e < R * M; e += NTHR) {
      const int r = e / M, m = e - r * M;
      du[r * LM + m] = p.dus[((int64_t)(c0 + r) * HQ + hq) * M + m];
      pl[r * LM + m] = p.pp[((int64_t)(c0 + r) * HQ + hq) * M + m];
    }
    for (int e = tid; e < R * R; e += NTHR) {
      const int i = e / R, r = e - i * R;
      if (i < r) continue;
      const int sj = src[r];
      float av = 0.f, bv = 0.f;
      if (sj >= 0 && p.ap) {
        av = bf16_to_f32(p.ap[(((int64_t)chunk * HQ + hq) * BT + i) * BT + r]);
        bv = bf16_to_f32(p.bp[(((int64_t)chunk * HQ + hq) * BT + i) * BT + r]);
      } else if (sj >= 0) {
        const T* qrow = (const T*)p.q_gsa + ((int64_t)(c0 + i) * HQ + hq) * K;
        const T* krow = (const T*)p.k_gsa + ((int64_t)sj * H + h) * K;
        av = dot_rows<T>(qrow, krow, K);
        const T* drow = (const T*)p.dout + ((int64_t)(c0 + i) * HQ + hq) * V;
        const T* vrow = (const T*)p.v + ((int64_t)sj * H + h) * V;
        bv = dot_rows<T>(drow, vrow, V);
      }
      Am[i * (BT + 1) + r] = av;
      Bm[i * (BT + 1) + r] = bv;
    }
    __syncthreads();
    float* ckp = p.ck + ((int64_t)chunk * HQ + hq) * BT * BT;
    float* cvp = p.cv + ((int64_t)chunk * HQ + hq) * BT * BT;
    for (int e = tid; e < R * R; e += NTHR) {
      const int i = e / R, r = e - i * R;
      if (i < r) continue;
      float a1 = 0.f, a2 = 0.f;
      for (int m = 0; m < M; ++m) {
        const float w = sl[r * LM + m] * expf(gcl[i * LM + m] - gcl[r * LM + m]);
        a1 += du[i * LM + m] * w;
        a2 += pl[i * LM + m] * w;
      }
      ckp[i * BT + r] = a1;
      cvp[i * BT + r] = a2;
    }
    if (M == 64) {
      // a thread's BT*64/NTHR outputs share the slot m (rows rb, rb + 8, ...): du_i[m], p_i[m] and
      // gc_i[m] are read once per i
      const int rb = tid >> 6, m = tid & 63;
      float acc[BT * 64 / NTHR], gr[BT * 64 / NTHR];
#pragma unroll
      for (int u = 0; u < BT * 64 / NTHR; ++u) {
        acc[u] = 0.f;
        const int r = rb + (NTHR / 64) * u;
        gr[u] = r < R ? gcl[r * LM + m] : 0.f;
      }
      for (int i = rb; i < R; ++i) {
        const float dui = du[i * LM + m], pli = pl[i * LM + m], gi = gcl[i * LM + m];
#pragma unroll
        for (int u = 0; u < BT * 64 / NTHR; ++u) {
          const int r = rb + (NTHR / 64) * u;
          if (i >= r) acc[u] += (Am[i * (BT + 1) + r] * dui + Bm[i * (BT + 1) + r] * pli) * expf(gi - gr[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < BT * 64 / NTHR; ++u) {
        const int r = rb + (NTHR / 64) * u;
        if (r < R) dsl[r * LM + m] += acc[u];
      }
    } else {
      for (int e = tid; e < R * M; e += NTHR) {
        const int r = e / M, m = e - r * M;
        float acc = 0.f;
        const float gr = gcl[r * LM + m];
        for (int i = r; i < R; ++i)
          acc += (Am[i * (BT + 1) + r] * du[i * LM + m] + Bm[i * (BT + 1) + r] * pl[i * LM + m]) * expf(gcl[i * LM + m] - gr);
        dsl[r * LM + m] += acc;
      }
    }
  }
  __syncthreads();
  for (int e = tid; e < R * M; e += NTHR) {
    const int r = e / M, m = e - r * M;
    p.dsi[((int64_t)(c0 + r) * H + h) * M + m] = dsl[r * LM + m];
  }
}

// ------------------------------------------------------------------------------------------
// State gradients.  E_c[x][m], the gradient of the state at the END of chunk c that comes from
// later chunks, obeys a linear recurrence over the chunks of a sequence,
//   E_(c-1) = e^(gl_c)[m] E_c + N_c,    N_c[x][m] = sum_i sum_a x_i^a[x] w_i^a[m] e^(gc_i[m])
// (x = rows of q_gsa with weights scale*du for the k-state, rows of do with weights p for the
// v-state), whose inhomogeneous term N_c does not depend on E.  Three launches, the first and
// the last parallel over chunks:
//   bwd_state_direct_kernel   N_c and the intra-chunk part of dk' / dv'   (per chunk, CB columns)
//   bwd_state_scan_kernel     the recurrence, element-wise over chunks (E_c replaces N_c; dh0)
//   bwd_state_inter_kernel    the parts of dk' / dv' / ds that involve E_c (per chunk, CB columns)
// blockIdx.z = 0: k-state (columns d; q_gsa / k_gsa rows, weights dus, matrix ck, output dk_gsa);
// 1: v-state (columns c; do / v rows, weights p, matrix cv, output dvs).  eg holds N then E as
// [NT][H][X][M] per state.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_state_direct_kernel(const BP p) {
  extern __shared__ __align__(16) float lds[];
  const int M = p.M, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  const int LM = M + 1;
  const bool isv = blockIdx.z != 0;
  const int X = isv ? p.V : p.K;
  const int nbmax = p.nbk > p.nbv ? p.nbk : p.nbv;
  const int h = blockIdx.y / nbmax, blk = blockIdx.y % nbmax;
  if (blk >= (isv ? p.nbv : p.nbk)) return;
  const int x0 = blk * CB;
  float* gcl = lds;                  // [BT][LM]
  float* Lw = gcl + BT * LM;         // [BT][LM]  per head: weight_i[m] e^(gc_i[m])
  float* Cm = Lw + BT * LM;          // [BT][BT+1] per head
  float* xq = Cm + BT * (BT + 1);    // [BT][CB+1] per head: q_gsa / do columns
  int* src = (int*)(xq + BT * (CB + 1));   // [BT]
  const int tid = threadIdx.x;
  const int chunk = blockIdx.x;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const T* qrow_src = isv ? (const T*)p.dout : (const T*)p.q_gsa;  // [T_tot][HQ][X]
  const float* wsrc = isv ? p.pp : p.dus;
  const float* csrc = isv ? p.cv : p.ck;
  if (tid < BT) {
    const int tl = it * BT + tid - p.shift;
    src[tid] = (tid < R && tl >= 0) ? bos + tl : -1;
  }
  for (int e = tid; e < R * M; e += 256) {
    const int r = e / M, m = e - r * M;
    gcl[r * LM + m] = p.gc[((int64_t)(c0 + r) * H + h) * M + m];
  }
  // this thread's outputs: 8 of the R x CB intra sums, CB*M/256 of the CB x M elements of N
  float acc[BT * CB / 256];
  float en[CB * 64 / 256];
#pragma unroll
  for (int u = 0; u < BT * CB / 256; ++u) acc[u] = 0.f;
#pragma unroll
  for (int u = 0; u < CB * 64 / 256; ++u) en[u] = 0.f;
  for (int a = 0; a < NG; ++a) {
    const int hq = h * NG + a;
    __syncthreads();
    const float* cp = csrc + ((int64_t)chunk * HQ + hq) * BT * BT;
    for (int e = tid; e < R * R; e += 256) {
      const int i = e / R, r = e - i * R;
      Cm[i * (BT + 1) + r] = i >= r ? cp[i * BT + r] : 0.f;
    }
    for (int e = tid; e < R * CB; e += 256) {
      const int i = e / CB, x = e - i * CB;
      xq[i * (CB + 1) + x] = (x0 + x < X) ? Elem<T>::ld(qrow_src + ((int64_t)(c0 + i) * HQ + hq) * X + x0 + x) : 0.f;
    }
    for (int e = tid; e < R * M; e += 256) {
      const int i = e / M, m = e - i * M;
      Lw[i * LM + m] = wsrc[((int64_t)(c0 + i) * HQ + hq) * M + m] * expf(gcl[i * LM + m]);
    }
    __syncthreads();
    // a thread's BT*CB/256 intra sums share the column x (rows rb, rb + 256/CB, ...): one read of
    // x_i[x] serves all of them (Cm is zero above the diagonal)
    {
      const int rb = tid / CB, x = tid % CB;
      for (int i = rb; i < R; ++i) {
        const float xv = xq[i * (CB + 1) + x];
#pragma unroll
        for (int u = 0; u < BT * CB / 256; ++u) acc[u] += xv * Cm[i * (BT + 1) + rb + (256 / CB) * u];
      }
    }
    if (M == 64) {
      // likewise its CB*64/256 elements of N share the slot m (columns xb, xb + 4, ...)
      const int xb = tid >> 6, m = tid & 63;
      for (int i = 0; i < R; ++i) {
        const float lw = Lw[i * LM + m];
#pragma unroll
        for (int u = 0; u < CB * 64 / 256; ++u) en[u] += xq[i * (CB + 1) + xb + 4 * u] * lw;
      }
    } else {
#pragma unroll
      for (int u = 0; u < CB * 64 / 256; ++u) {
        const int e = tid + 256 * u;
        const int x = e / M, m = e - x * M;
        if (e < CB * M) {
          float s2 = 0.f;
          for (int i = 0; i < R; ++i) s2 += xq[i * (CB + 1) + x] * Lw[i * LM + m];
          en[u] += s2;
        }
      }
    }
  }
  float* outp = isv ? p.dvs : p.dks;
#pragma unroll
  for (int u = 0; u < BT * CB / 256; ++u) {
    const int e = tid + 256 * u;
    const int r = e / CB, x = e - r * CB;
    if (r >= R) continue;
    const int sj = src[r];
    if (sj >= 0 && x0 + x < X) outp[((int64_t)sj * H + h) * X + x0 + x] = acc[u];
  }
  float* ep = (isv ? p.ev : p.ek) + ((int64_t)chunk * H + h) * X * M;
#pragma unroll
  for (int u = 0; u < CB * 64 / 256; ++u) {
    const int e = tid + 256 * u;
    const int x = e / M, m = e - x * M;
    if (e < CB * M && x0 + x < X) ep[(int64_t)(x0 + x) * M + m] = en[u];
  }
}

// grid (N*H, ceil((K+V)*M / 256)): one thread per state element, sequential over the chunks
__global__ __launch_bounds__(256) void bwd_state_scan_kernel(const BP p) {
  const int K = p.K, V = p.V, M = p.M, H = p.H;
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const int e = blockIdx.y * 256 + threadIdx.x;
  if (e >= (K + V) * M) return;
  const bool isv = e >= K * M;
  const int em = isv ? e - K * M : e;
  const int X = isv ? V : K;
  const int x = em / M, m = em % M;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int L = eos - bos;
  const int nchunks = (L + BT - 1) / BT;
  float* eb = isv ? p.ev : p.ek;
  const float* dht = isv ? p.dhvt : p.dhkt;
  float E = 0.f;
  if (dht) E = isv ? dht[(((int64_t)n * H + h) * M + m) * X + x] : dht[(((int64_t)n * H + h) * X + x) * M + m];
  // the recurrence is sequential, its operands are not: four chunks' loads are in flight together
  const int64_t cstride = (int64_t)H * X * M;
  float* ebn = eb + (((int64_t)p.coff[n] * H + h) * X + x) * M + m;
  auto gl_of = [&](int it) {
    const int R = (L - it * BT) < BT ? (L - it * BT) : BT;
    return p.gc[((int64_t)(bos + it * BT + R - 1) * H + h) * M + m];
  };
  int it = nchunks - 1;
  for (; it >= 3; it -= 4) {
    float nc[4], gl[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      nc[u] = ebn[(it - u) * cstride];
      gl[u] = gl_of(it - u);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      ebn[(it - u) * cstride] = E;
      E = E * expf(gl[u]) + nc[u];
    }
  }
  for (; it >= 0; --it) {
    const float nc = ebn[it * cstride];
    ebn[it * cstride] = E;
    E = E * expf(gl_of(it)) + nc;
  }
  float* dh0 = isv ? p.dh0v : p.dh0k;
  if (dh0) {
    if (isv) dh0[(((int64_t)n * H + h) * M + m) * X + x] = E;
    else dh0[(((int64_t)n * H + h) * X + x) * M + m] = E;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bwd_state_inter_kernel(const BP p) {
  extern __shared__ __align__(16) float lds[];
  const int M = p.M, H = p.H;
  const int LM = M + 1;
  const bool isv = blockIdx.z != 0;
  const int X = isv ? p.V : p.K;
  const int nbmax = p.nbk > p.nbv ? p.nbk : p.nbv;
  const int h = blockIdx.y / nbmax, blk = blockIdx.y % nbmax;
  if (blk >= (isv ? p.nbv : p.nbk)) return;
  const int slab = isv ? p.nbk + blk : blk;
  const int x0 = blk * CB;
  float* E = lds;                    // [CB][LM]
  float* gcl = E + CB * LM;          // [BT][LM]
  float* dec = gcl + BT * LM;        // [BT][LM]  e^(gl - gc_r)
  float* sE = dec + BT * LM;         // [BT][LM]  s_r e^(gl - gc_r)
  float* xk = sE + BT * LM;          // [BT][CB+1] k' / v' columns
  int* src = (int*)(xk + BT * (CB + 1));   // [BT]
  const int tid = threadIdx.x;
  const int chunk = blockIdx.x;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const T* xrow_src = isv ? (const T*)p.v : (const T*)p.k_gsa;     // [T_tot][H][X]
  const float* ep = (isv ? p.ev : p.ek) + ((int64_t)chunk * H + h) * X * M;
  if (tid < BT) {
    const int tl = it * BT + tid - p.shift;
    src[tid] = (tid < R && tl >= 0) ? bos + tl : -1;
  }
  for (int e = tid; e < R * M; e += 256) {
    const int r = e / M, m = e - r * M;
    gcl[r * LM + m] = p.gc[((int64_t)(c0 + r) * H + h) * M + m];
  }
  for (int e = tid; e < CB * M; e += 256) {
    const int x = e / M, m = e - x * M;
    E[x * LM + m] = (x0 + x < X) ? ep[(int64_t)(x0 + x) * M + m] : 0.f;
  }
  __syncthreads();
  for (int e = tid; e < R * M; e += 256) {
    const int r = e / M, m = e - r * M;
    const float d = expf(gcl[(R - 1) * LM + m] - gcl[r * LM + m]);
    const int sj = src[r];
    dec[r * LM + m] = d;
    sE[r * LM + m] = sj >= 0 ? d * Elem<T>::ld((const T*)p.s + ((int64_t)sj * H + h) * M + m) : 0.f;
  }
  for (int e = tid; e < R * CB; e += 256) {
    const int r = e / CB, x = e - r * CB;
    const int sj = src[r];
    xk[r * (CB + 1) + x] = (sj >= 0 && x0 + x < X) ? Elem<T>::ld(xrow_src + ((int64_t)sj * H + h) * X + x0 + x) : 0.f;
  }
  __syncthreads();
  // dk'_r[x] = intra part + sum_m sE_r[m] E[x][m];  ds part = dec_r[m] sum_x k'_r[x] E[x][m].
  // A thread's outputs share x (resp. m), so every E element it reads serves all of them.
  float* part = isv ? p.dvs : p.dks;
  {
    const int rb = tid / CB, x = tid % CB;
    float a[BT * CB / 256];
#pragma unroll
    for (int u = 0; u < BT * CB / 256; ++u) a[u] = 0.f;
    for (int m = 0; m < M; ++m) {
      const float ev = E[x * LM + m];
#pragma unroll
      for (int u = 0; u < BT * CB / 256; ++u) a[u] += sE[(rb + (256 / CB) * u) * LM + m] * ev;
    }
#pragma unroll
    for (int u = 0; u < BT * CB / 256; ++u) {
      const int r = rb + (256 / CB) * u;
      if (r >= R) continue;
      const int sj = src[r];
      if (sj < 0 || x0 + x >= X) continue;
      const int64_t oi = ((int64_t)sj * H + h) * X + x0 + x;
      const float val = part[oi] + a[u];
      if (isv) p.dvs[oi] = val;
      else Elem<T>::st((T*)p.dk_gsa + oi, val);
    }
  }
  if (M == 64) {
    const int rb = tid >> 6, m = tid & 63;
    float a[BT * 64 / 256];
#pragma unroll
    for (int u = 0; u < BT * 64 / 256; ++u) a[u] = 0.f;
    for (int x = 0; x < CB; ++x) {
      const float ev = E[x * LM + m];
#pragma unroll
      for (int u = 0; u < BT * 64 / 256; ++u) a[u] += xk[(rb + 4 * u) * (CB + 1) + x] * ev;
    }
#pragma unroll
    for (int u = 0; u < BT * 64 / 256; ++u) {
      const int r = rb + 4 * u;
      if (r < R) p.dsp[(((int64_t)slab * p.T_tot + c0 + r) * H + h) * M + m] = a[u] * dec[r * LM + m];
    }
  } else {
    for (int e = tid; e < R * M; e += 256) {
      const int r = e / M, m = e - r * M;
      float a = 0.f;
      for (int x = 0; x < CB; ++x) a += xk[r * (CB + 1) + x] * E[x * LM + m];
      p.dsp[(((int64_t)slab * p.T_tot + c0 + r) * H + h) * M + m] = a * dec[r * LM + m];
    }
  }
}

// ------------------------------------------------------------------------------------------
// ds and dg.  dg is a reverse cumulative sum over the rows of a sequence; three small launches:
// per chunk the summand, ds and the chunk-local sums (bwd_gate_local_kernel), per sequence the
// sums of all later chunks plus the end term (bwd_gate_scan_kernel), per chunk the final values
// (bwd_gate_final_kernel, which also zeroes the gradients of the tokens that never reach the
// slots: the last `shift` of a sequence).
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_gate_local_kernel(const BP p) {
  // M == 64 (the matrix-core path): thread = (group rg of 4 consecutive rows, 4 consecutive slots), 16-byte
  // reads, all of a thread's rows requested together; the reverse cumulative sum is a suffix sum over the
  // thread's rows plus the sums of the later groups through LDS.  Other M: thread = (group of 16 rows, slot).
  __shared__ float gs[16][BT];
  const int M = p.M, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  const int chunk = blockIdx.x, h = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  const int nslab = p.nbk + p.nbv;
  if (M == BT) {
    const int rg = threadIdx.x >> 4, m = (threadIdx.x & 15) * 4;
    float z[4][4], dst[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 4 * rg + q, t = c0 + r, sj = t - p.shift;
#pragma unroll
      for (int e = 0; e < 4; ++e) z[q][e] = dst[q][e] = 0.f;
      if (r < R && sj >= bos) {
        const int64_t rt = ((int64_t)t * H + h) * M + m;
        float4 ds4 = *reinterpret_cast<const float4*>(p.dsi + rt);
        for (int b = 0; b < nslab; ++b) {
          const float4 a = *reinterpret_cast<const float4*>(p.dsp + (int64_t)b * p.T_tot * H * M + rt);
          ds4.x += a.x; ds4.y += a.y; ds4.z += a.z; ds4.w += a.w;
        }
        float4 x4 = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int a = 0; a < NG; ++a) {
          const float4 v = *reinterpret_cast<const float4*>(p.xg + ((int64_t)t * HQ + h * NG + a) * M + m);
          x4.x += v.x; x4.y += v.y; x4.z += v.z; x4.w += v.w;
        }
        float sv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) sv[e] = Elem<T>::ld((const T*)p.s + ((int64_t)sj * H + h) * M + m + e);
        const float d4[4] = {ds4.x, ds4.y, ds4.z, ds4.w}, xx[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          z[q][e] = xx[e] - sv[e] * d4[e];
          dst[q][e] = d4[e];
        }
      }
    }
    float run[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 3; q >= 0; --q)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        run[e] += z[q][e];
        z[q][e] = run[e];   // suffix sum inside the group
      }
    *reinterpret_cast<float4*>(&gs[rg][m]) = make_float4(run[0], run[1], run[2], run[3]);
    __syncthreads();
    float later[4] = {0.f, 0.f, 0.f, 0.f};
    for (int g2 = 15; g2 > rg; --g2) {
      const float4 a = *reinterpret_cast<const float4*>(&gs[g2][m]);
      later[0] += a.x; later[1] += a.y; later[2] += a.z; later[3] += a.w;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = 4 * rg + q, t = c0 + r, sj = t - p.shift;
      if (r < R && sj >= bos) {
        const int64_t rt = ((int64_t)t * H + h) * M + m;
#pragma unroll
        for (int e = 0; e < 4; ++e) Elem<T>::st((T*)p.ds + ((int64_t)sj * H + h) * M + m + e, dst[q][e]);
        *reinterpret_cast<float4*>(p.dsi + rt) = make_float4(z[q][0] + later[0], z[q][1] + later[1], z[q][2] + later[2], z[q][3] + later[3]);   // chunk-local reverse cumulative sum
      }
    }
    if (rg == 0) *reinterpret_cast<float4*>(p.gtot + ((int64_t)chunk * H + h) * M + m) = make_float4(run[0] + later[0], run[1] + later[1], run[2] + later[2], run[3] + later[3]);
    return;
  }
  const int m = threadIdx.x & 63, g = threadIdx.x >> 6;
  float z[16], dst[16];
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int r = 16 * g + q, t = c0 + r, sj = t - p.shift;
    z[q] = dst[q] = 0.f;
    if (m < M && r < R && sj >= bos) {
      const int64_t rt = ((int64_t)t * H + h) * M + m;
      float dstot = p.dsi[rt];
      for (int b = 0; b < nslab; ++b) dstot += p.dsp[(int64_t)b * p.T_tot * H * M + rt];
      float x = 0.f;
      for (int a = 0; a < NG; ++a) x += p.xg[((int64_t)t * HQ + h * NG + a) * M + m];
      const float sval = Elem<T>::ld((const T*)p.s + ((int64_t)sj * H + h) * M + m);
      z[q] = x - sval * dstot;
      dst[q] = dstot;
    }
  }
  float run = 0.f;
#pragma unroll
  for (int q = 15; q >= 0; --q) {
    run += z[q];
    z[q] = run;   // suffix sum inside the group
  }
  gs[g][m] = run;
  __syncthreads();
  float later = 0.f;
  for (int g2 = 3; g2 > g; --g2) later += gs[g2][m];
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int r = 16 * g + q, t = c0 + r, sj = t - p.shift;
    if (m < M && r < R && sj >= bos) {
      const int64_t rt = ((int64_t)t * H + h) * M + m;
      Elem<T>::st((T*)p.ds + ((int64_t)sj * H + h) * M + m, dst[q]);
      p.dsi[rt] = z[q] + later;   // chunk-local reverse cumulative sum
    }
  }
  if (g == 0 && m < M) p.gtot[((int64_t)chunk * H + h) * M + m] = run + later;
}

template <typename T>
__global__ void bwd_gate_scan_kernel(const BP p) {
  const int K = p.K, V = p.V, M = p.M, H = p.H;
  const int n = blockIdx.x / H, h = blockIdx.x % H;
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int tid = threadIdx.x;
  const int m = tid;
  if (m >= M) return;
  float run = 0.f;   // <dh_T, h_T>: what the gates past the end of the sequence would receive
  if (p.dhkt) {
    const float* a = p.dhkt + ((int64_t)n * H + h) * K * M;
    const float* b = p.hkT + ((int64_t)n * H + h) * K * M;
    for (int d = 0; d < K; ++d) run += a[d * M + m] * b[d * M + m];
  }
  if (p.dhvt) {
    const float* a = p.dhvt + (((int64_t)n * H + h) * M + m) * V;
    const float* b = p.hvT + (((int64_t)n * H + h) * M + m) * V;
    for (int c = 0; c < V; ++c) run += a[c] * b[c];
  }
  // sixteen chunk sums are fetched before the first is consumed, so the loads overlap
  const int nchunks = (eos - bos + BT - 1) / BT;
  float* gt = p.gtot + ((int64_t)p.coff[n] * H + h) * M + m;
  const int64_t cs = (int64_t)H * M;
  int it = nchunks - 1;
  constexpr int NB = 16;
  for (; it >= NB - 1; it -= NB) {
    float t[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) t[u] = gt[(it - u) * cs];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      gt[(it - u) * cs] = run;
      run += t[u];
    }
  }
  for (; it >= 0; --it) {
    const float tot = gt[it * cs];
    gt[it * cs] = run;
    run += tot;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bwd_gate_final_kernel(const BP p) {
  const int M = p.M, H = p.H;
  const int chunk = blockIdx.x, h = blockIdx.y;
  const int n = p.cidx[2 * chunk], it = p.cidx[2 * chunk + 1];
  const int bos = p.cu[n], eos = p.cu[n + 1];
  const int c0 = bos + it * BT;
  const int R = (eos - c0) < BT ? (eos - c0) : BT;
  if (M == BT) {
    // four consecutive slots of four rows per thread, their 16-byte reads requested together
    const int m = (threadIdx.x & 15) * 4, r0 = threadIdx.x >> 4;
    const float4 gt = *reinterpret_cast<const float4*>(p.gtot + ((int64_t)chunk * H + h) * M + m);
    float4 v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = r0 + 16 * q, t = c0 + r;
      v[q] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r < R && t - p.shift >= bos) v[q] = *reinterpret_cast<const float4*>(p.dsi + ((int64_t)t * H + h) * M + m);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = r0 + 16 * q, sj = c0 + r - p.shift;
      if (r < R && sj >= bos) {
        T* dst = (T*)p.dg + ((int64_t)sj * H + h) * M + m;
        Elem<T>::st(dst, v[q].x + gt.x);
        Elem<T>::st(dst + 1, v[q].y + gt.y);
        Elem<T>::st(dst + 2, v[q].z + gt.z);
        Elem<T>::st(dst + 3, v[q].w + gt.w);
      }
    }
  } else {
    for (int e = threadIdx.x; e < R * M; e += 256) {
      const int r = e / M, m = e - r * M;
      const int t = c0 + r, sj = t - p.shift;
      if (sj < bos) continue;
      const float val = p.dsi[((int64_t)t * H + h) * M + m] + p.gtot[((int64_t)chunk * H + h) * M + m];
      Elem<T>::st((T*)p.dg + ((int64_t)sj * H + h) * M + m, val);
    }
  }
  // tokens of this chunk that never reach the slots (the last `shift` of the sequence): zero gradients
  const int K = p.K, V = p.V;
  int r0 = eos - p.shift - c0;
  r0 = r0 < 0 ? 0 : r0;
  if (r0 >= R) return;
  const int nr = R - r0;
  if (M % 8 == 0 && K % 8 == 0 && V % 8 == 0) {
    // 16-byte stores, the rows of the chunk side by side (M, K, V multiples of 8: every row start is 16-byte aligned)
    constexpr int EPV = 16 / (int)sizeof(T);   // elements of T per 16 bytes
    const uint4 zero = make_uint4(0, 0, 0, 0);
    for (int i = threadIdx.x; i < nr * (M / EPV); i += 256) {
      const int r = r0 + i / (M / EPV), e = (i % (M / EPV)) * EPV;
      const int64_t jh = (int64_t)(c0 + r) * H + h;
      *reinterpret_cast<uint4*>((T*)p.ds + jh * M + e) = zero;
      *reinterpret_cast<uint4*>((T*)p.dg + jh * M + e) = zero;
    }
    for (int i = threadIdx.x; i < nr * (K / EPV); i += 256) {
      const int r = r0 + i / (K / EPV), e = (i % (K / EPV)) * EPV;
      *reinterpret_cast<uint4*>((T*)p.dk_gsa + ((int64_t)(c0 + r) * H + h) * K + e) = zero;
    }
    for (int i = threadIdx.x; i < nr * (V / 4); i += 256) {
      const int r = r0 + i / (V / 4), e = (i % (V / 4)) * 4;
      *reinterpret_cast<uint4*>(p.dvs + ((int64_t)(c0 + r) * H + h) * V + e) = zero;
    }
    return;
  }
  for (int r = r0; r < R; ++r) {
    const int64_t jh = (int64_t)(c0 + r) * H + h;
    for (int e = threadIdx.x; e < M; e += 256) {
      Elem<T>::st((T*)p.ds + jh * M + e, 0.f);
      Elem<T>::st((T*)p.dg + jh * M + e, 0.f);
    }
    for (int e = threadIdx.x; e < K; e += 256) Elem<T>::st((T*)p.dk_gsa + jh * K + e, 0.f);
    for (int e = threadIdx.x; e < V; e += 256) p.dvs[jh * V + e] = 0.f;
  }
}

// ------------------------------------------------------------------------------------------
// per (key token, kv-head): dk_swa and dv (window part + slot-branch part)
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_kv_window_kernel(const BP p) {
  extern __shared__ __align__(16) float lds[];
  const int K = p.K, V = p.V, H = p.H, HQ = p.HQ;
  const int NG = HQ / H;
  float* kj = lds;          // [K] scale * k_swa_j
  float* vj = kj + K;       // [V]
  float* pwk = vj + V;      // [256] scale * dw
  float* ppi = pwk + 256;   // [256] pi
  const int tid = threadIdx.x;
  const int j = blockIdx.x, h = blockIdx.y;
  int n = 0;
  {
    int lo = 0, hi = p.N - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p.cu[mid] <= j) lo = mid; else hi = mid - 1;
    }
    n = lo;
  }
  const int eos = p.cu[n + 1];
  int tmax = eos - 1;
  if (p.wl >= 0 && j + p.wl < tmax) tmax = j + p.wl;
  for (int i = tid; i < K; i += 256) kj[i] = Elem<T>::ld((const T*)p.k_swa + ((int64_t)j * H + h) * K + i) * p.scale;
  for (int i = tid; i < V; i += 256) vj[i] = Elem<T>::ld((const T*)p.v + ((int64_t)j * H + h) * V + i);
  __syncthreads();
  const int npairs = (tmax - j + 1) * NG;
  float acck = 0.f, accv = 0.f;
  for (int pb = 0; pb < npairs; pb += 256) {
    const int x = pb + tid;
    float dwv = 0.f, piv = 0.f;
    if (x < npairs) {
      const int t = j + x / NG, hq = h * NG + x % NG;
      const int64_t tq = (int64_t)t * HQ + hq;
      const float w = dot_row<T>(kj, (const T*)p.q_swa + tq * K, K);
      const float ls = p.lse_swa[tq];
      const float lt = logaddexp_f(ls, p.lse_gsa[tq]);
      piv = expf(w - lt);
      const float dpi = dot_row<T>(vj, (const T*)p.dout + tq * V, V);
      dwv = p.scale * (piv * (dpi - p.delta[tq]) + (p.dlse_swa ? p.dlse_swa[tq] * expf(w - ls) : 0.f));
    }
    __syncthreads();
    pwk[tid] = dwv;
    ppi[tid] = piv;
    __syncthreads();
    const int cnt = (npairs - pb) < 256 ? (npairs - pb) : 256;
    if (tid < K)
      for (int y = 0; y < cnt; ++y) {
        const int t = j + (pb + y) / NG, hq = h * NG + (pb + y) % NG;
        acck += pwk[y] * Elem<T>::ld((const T*)p.q_swa + ((int64_t)t * HQ + hq) * K + tid);
      }
    if (tid < V)
      for (int y = 0; y < cnt; ++y) {
        const int t = j + (pb + y) / NG, hq = h * NG + (pb + y) % NG;
        accv += ppi[y] * Elem<T>::ld((const T*)p.dout + ((int64_t)t * HQ + hq) * V + tid);
      }
  }
  if (tid < K) Elem<T>::st((T*)p.dk_swa + ((int64_t)j * H + h) * K + tid, acck);
  if (tid < V) Elem<T>::st((T*)p.dv + ((int64_t)j * H + h) * V + tid, accv + p.dvs[((int64_t)j * H + h) * V + tid]);
}

size_t aligned(size_t x) { return (x + 255) & ~(size_t)255; }

struct BwdPlan {
  size_t fwd, mfma, hkct, hvct, hkb, hvb, hkl, hvl, ap, bp, ust, dpst, big, hkT, hvT, dus, pp, xg, delta, ld, ck, cv, dsi, dsp, dvs, gtot, dks, ek, ev, total;
  bool use_mfma;
  int nbk, nbv;
};
BwdPlan plan_bwd(const NhaPrefillBwdArgs* a, const NhaPrefillArgs& f) {
  BwdPlan s;
  s.nbk = (a->K + CB - 1) / CB;
  s.nbv = (a->V + CB - 1) / CB;
  size_t off = 0;
  s.fwd = off; off += aligned(prefill_simple_scratch_bytes(&f));
  // bf16 shapes the matrix-core state pass covers: recompute the states with it and convert
  s.use_mfma = prefill_mfma_supported(&f);
  s.mfma = off;
  if (s.use_mfma) off += aligned(prefill_mfma_scratch_bytes(&f));
  s.hkct = off; off += aligned((size_t)a->NT * a->H * a->K * a->M * 4);
  s.hvct = off; off += aligned((size_t)a->NT * a->H * a->V * a->M * 4);
  s.hkb = s.hvb = s.hkl = s.hvl = s.ap = s.bp = s.ust = s.dpst = s.big = off;
  if (s.use_mfma) {
    s.hkb = off; off += aligned((size_t)a->NT * a->H * a->M * a->K * 2);
    s.hvb = off; off += aligned((size_t)a->NT * a->H * a->M * a->V * 2);
    s.hkl = off; off += aligned((size_t)a->NT * a->H * a->M * a->K * 2);
    s.hvl = off; off += aligned((size_t)a->NT * a->H * a->M * a->V * 2);
    s.ap = off; off += aligned((size_t)a->NT * a->HQ * BT * BT * 2);
    s.bp = off; off += aligned((size_t)a->NT * a->HQ * BT * BT * 2);
    s.ust = off; off += aligned((size_t)a->T_tot * a->HQ * a->M * 4);
    s.dpst = off; off += aligned((size_t)a->T_tot * a->HQ * a->M * 4);
    s.big = off; off += aligned((size_t)a->NT * a->H * 4);
  }
  s.hkT = off; off += aligned((size_t)a->N * a->H * a->K * a->M * 4);
  s.hvT = off; off += aligned((size_t)a->N * a->H * a->M * a->V * 4);
  const size_t tqm = aligned((size_t)a->T_tot * a->HQ * a->M * 4);
  s.dus = off; off += tqm;
  s.pp = off; off += tqm;
  s.xg = off; off += tqm;
  s.delta = off; off += aligned((size_t)a->T_tot * a->HQ * 4);
  s.ld = off; off += aligned((size_t)a->T_tot * a->HQ * 8);   // (-lse / scale, -delta) pairs of the LDS-direct window kernels
  const size_t cc = aligned((size_t)a->NT * a->HQ * BT * BT * 4);
  s.ck = off; off += cc;
  s.cv = off; off += cc;
  const size_t thm = (size_t)a->T_tot * a->H * a->M * 4;
  s.dsi = off; off += aligned(thm);
  s.dsp = off; off += aligned(thm * (s.nbk + s.nbv));
  s.dvs = off; off += aligned((size_t)a->T_tot * a->H * a->V * 4);
  s.gtot = off; off += aligned((size_t)a->NT * a->H * a->M * 4);
  s.dks = off; off += aligned((size_t)a->T_tot * a->H * a->K * 4);
  s.ek = off; off += aligned((size_t)a->NT * a->H * a->K * a->M * 4);
  s.ev = off; off += aligned((size_t)a->NT * a->H * a->V * a->M * 4);
  s.total = off;
  return s;
}

NhaPrefillArgs forward_args(const NhaPrefillBwdArgs* a) {
  NhaPrefillArgs f = {};
  f.q_swa = a->q_swa; f.k_swa = a->k_swa; f.q_gsa = a->q_gsa; f.k_gsa = a->k_gsa;
  f.v = a->v; f.s = a->s; f.g = a->g;
  f.h0k = a->h0k; f.h0v = a->h0v;
  f.cu_seqlens = a->cu_seqlens; f.chunk_indices = a->chunk_indices; f.chunk_offsets = a->chunk_offsets;
  f.T_tot = a->T_tot; f.N = a->N; f.NT = a->NT; f.HQ = a->HQ; f.H = a->H; f.K = a->K; f.V = a->V; f.M = a->M;
  f.wl = a->wl; f.shift = a->shift; f.dtype = a->dtype; f.impl = NHA_IMPL_SIMPLE;
  f.scale = a->scale; f.stream = a->stream;
  return f;
}

template <typename T>
int run_bwd(const NhaPrefillBwdArgs* a) {
  NhaPrefillArgs f = forward_args(a);
  const BwdPlan sp = plan_bwd(a, f);
  char* sc = (char*)a->scratch;
  f.hkt = (float*)(sc + sp.hkT);
  f.hvt = (float*)(sc + sp.hvT);
  // layout of the generic forward state pass: gc | hkc | hvc, each aligned to 256 bytes
  char* fs = sc + sp.fwd;
  float* gc = (float*)fs;
  fs += aligned((size_t)a->T_tot * a->H * a->M * 4);
  float* hkc = (float*)fs;
  fs += aligned((size_t)a->NT * a->H * a->K * a->M * 4);
  float* hvc = (float*)fs;
#ifdef NHA_AB_SWITCHES   // measurement builds only (-DNHA_AB_SWITCHES)
  static const bool intra_mfma = getenv("NHA_BWD_INTRA_VALU") == nullptr;
#else
  constexpr bool intra_mfma = true;
#endif
  int rc;
  if (sp.use_mfma) {
    f.impl = NHA_IMPL_MFMA;
    f.scratch = sc + sp.mfma;
    f.scratch_bytes = prefill_mfma_scratch_bytes(&f);
    // state pass (segment form) and its export; every consumer of the states on this path reads
    // the bf16 copies
    rc = prefill_mfma_export_states(&f, gc, nullptr, nullptr, nullptr, sc + sp.hkb, sc + sp.hvb, sc + sp.hkl, sc + sp.hvl, (int*)(sc + sp.big));
    // the decay-free products of the slot branch on the matrix cores
    // (with the decay-coupled terms on the matrix cores too, the per-token stage rides along)
    if (rc == NHA_OK) rc = bwd_slot_products(a, sc + sp.hkb, sc + sp.hvb, sc + sp.hkl, sc + sp.hvl, (bf16_t*)(sc + sp.ap), (bf16_t*)(sc + sp.bp), (float*)(sc + sp.ust), (float*)(sc + sp.dpst),
                                             (float*)(sc + sp.delta), intra_mfma ? (const int*)(sc + sp.big) : nullptr, gc,
                                             (float*)(sc + sp.dus), (float*)(sc + sp.pp), (float*)(sc + sp.xg));
  } else {
    f.scratch = sc + sp.fwd;
    f.scratch_bytes = prefill_simple_scratch_bytes(&f);
    rc = prefill_simple_impl(&f, 1);   // the state pass only
  }
  if (rc != NHA_OK) return rc;

  BP p;
  p.q_swa = a->q_swa; p.k_swa = a->k_swa; p.q_gsa = a->q_gsa; p.k_gsa = a->k_gsa;
  p.v = a->v; p.s = a->s; p.g = a->g; p.o = a->o; p.dout = a->dout;
  p.lse_swa = a->lse_swa; p.lse_gsa = a->lse_gsa; p.dlse_swa = a->dlse_swa; p.dlse_gsa = a->dlse_gsa;
  p.dhkt = a->dhkt; p.dhvt = a->dhvt;
  p.dq_swa = a->dq_swa; p.dk_swa = a->dk_swa; p.dq_gsa = a->dq_gsa; p.dk_gsa = a->dk_gsa;
  p.dv = a->dv; p.ds = a->ds; p.dg = a->dg; p.dh0k = a->dh0k; p.dh0v = a->dh0v;
  p.cu = a->cu_seqlens; p.cidx = a->chunk_indices; p.coff = a->chunk_offsets;
  p.gc = gc; p.hkc = hkc; p.hvc = hvc;
  p.hkct = (float*)(sc + sp.hkct); p.hvct = (float*)(sc + sp.hvct);
  p.ap = p.bp = nullptr;
  p.ust = p.dpst = nullptr;
  p.big = nullptr;
  if (sp.use_mfma) {
    if (intra_mfma) p.big = (const int*)(sc + sp.big);
    p.ap = (const bf16_t*)(sc + sp.ap); p.bp = (const bf16_t*)(sc + sp.bp);
    p.ust = (float*)(sc + sp.ust); p.dpst = (float*)(sc + sp.dpst);
  }
  p.hkT = (float*)(sc + sp.hkT); p.hvT = (float*)(sc + sp.hvT);
  p.dus = (float*)(sc + sp.dus); p.pp = (float*)(sc + sp.pp); p.xg = (float*)(sc + sp.xg);
  p.delta = (float*)(sc + sp.delta);
  p.ck = (float*)(sc + sp.ck); p.cv = (float*)(sc + sp.cv);
  p.dsi = (float*)(sc + sp.dsi); p.dsp = (float*)(sc + sp.dsp); p.dvs = (float*)(sc + sp.dvs);
  p.gtot = (float*)(sc + sp.gtot);
  p.dks = (float*)(sc + sp.dks); p.ek = (float*)(sc + sp.ek); p.ev = (float*)(sc + sp.ev);
  p.T_tot = a->T_tot; p.N = a->N; p.NT = a->NT; p.HQ = a->HQ; p.H = a->H; p.K = a->K; p.V = a->V; p.M = a->M;
  p.wl = a->wl; p.shift = a->shift; p.nbk = sp.nbk; p.nbv = sp.nbv; p.scale = a->scale;
  hipStream_t st = (hipStream_t)a->stream;
  const int K = a->K, V = a->V, M = a->M, LM = M + 1;

  const size_t lds_q = (size_t)4 * (K + V + 2 * BT + M) * 4;
  const size_t lds_qw = ((size_t)K + V + 256) * 4;
  const size_t lds_i = ((size_t)5 * BT * LM + 2 * BT * (BT + 1)) * 4 + BT * 4;
  const size_t lds_s1 = ((size_t)2 * BT * LM + BT * (BT + 1) + BT * (CB + 1)) * 4 + BT * 4;
  const size_t lds_s3 = ((size_t)CB * LM + 3 * BT * LM + BT * (CB + 1)) * 4 + BT * 4;
  const size_t lds_w = ((size_t)K + V + 512) * 4;
  static std::atomic<bool> configured{false};   // the attribute call is idempotent: a second thread may repeat it
  if (!configured) {
    hipError_t e1 = hipFuncSetAttribute((const void*)bwd_intra_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipError_t e2 = hipFuncSetAttribute((const void*)bwd_state_inter_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e1 != hipSuccess || e2 != hipSuccess) {
      set_error("nha_prefill_bwd: cannot reserve LDS: %s", hipGetErrorString(e1 != hipSuccess ? e1 : e2));
      return NHA_ERR_LAUNCH;
    }
    configured = true;
  }
  const bool wmfma = bwd_window_mfma_supported(a);
  if (!sp.use_mfma) hipLaunchKernelGGL(bwd_transpose_states_kernel, dim3(a->NT * a->H), dim3(256), 0, st, p);
  if (sp.use_mfma && intra_mfma && !bwd_slot_products_fuses_q(a)) {
    rc = bwd_slot_products3(a, 0, p.big, p.ap, p.bp, p.ust, p.dpst, p.gc, p.delta, p.dus, p.pp, p.xg, p.ck, p.cv, p.dsi);
    if (rc != NHA_OK) return rc;
  }
  hipLaunchKernelGGL((bwd_q_kernel<T>), p.big ? dim3(a->NT, a->H) : dim3(a->NT * (BT / 4), a->HQ), dim3(256), lds_q, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(query pass)");
  if (wmfma) {
    rc = bwd_window_mfma_dq(a, p.delta, sc + sp.ld);
    if (rc != NHA_OK) return rc;
  } else {
    hipLaunchKernelGGL((bwd_q_window_kernel<T>), dim3(a->NT * BT, a->HQ), dim3(256), lds_qw, st, p);
    NHA_CHECK_LAUNCH("nha_prefill_bwd(window query pass)");
  }
  if (sp.use_mfma && intra_mfma) {
    rc = bwd_slot_products3(a, 1, p.big, p.ap, p.bp, p.ust, p.dpst, p.gc, p.delta, p.dus, p.pp, p.xg, p.ck, p.cv, p.dsi);
    if (rc != NHA_OK) return rc;
  }
  hipLaunchKernelGGL((bwd_intra_kernel<T>), dim3(a->NT, a->H), dim3(512), lds_i, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(intra-chunk pass)");
  if (sp.use_mfma) {
    rc = bwd_slot_products2(a, 0, sc + sp.hkb, p.dus, p.pp, p.ck, p.cv, p.gc, p.ek, p.ev, p.dks, p.dvs, p.dsp);
    if (rc != NHA_OK) return rc;
  } else {
    hipLaunchKernelGGL((bwd_dqg_kernel<T>), dim3(a->NT * (BT / 4), a->HQ), dim3(256), (size_t)4 * (M + BT) * 4, st, p);
    NHA_CHECK_LAUNCH("nha_prefill_bwd(dq_gsa pass)");
  }
  const int nbmax = sp.nbk > sp.nbv ? sp.nbk : sp.nbv;
  if (sp.use_mfma) {
    rc = bwd_slot_products2(a, 1, sc + sp.hkb, p.dus, p.pp, p.ck, p.cv, p.gc, p.ek, p.ev, p.dks, p.dvs, p.dsp);
    if (rc != NHA_OK) return rc;
  } else {
    hipLaunchKernelGGL((bwd_state_direct_kernel<T>), dim3(a->NT, a->H * nbmax, 2), dim3(256), lds_s1, st, p);
  }
  hipLaunchKernelGGL(bwd_state_scan_kernel, dim3(a->N * a->H, ((K + V) * M + 255) / 256), dim3(256), 0, st, p);
  if (sp.use_mfma) {
    // one partial-ds slab per state and column range of a workgroup instead of one per 32-column block
    p.nbk = p.nbv = bwd_slot_inter_slabs(a);
    rc = bwd_slot_products2(a, 2, sc + sp.hkb, p.dus, p.pp, p.ck, p.cv, p.gc, p.ek, p.ev, p.dks, p.dvs, p.dsp);
    if (rc != NHA_OK) return rc;
  } else {
    hipLaunchKernelGGL((bwd_state_inter_kernel<T>), dim3(a->NT, a->H * nbmax, 2), dim3(256), lds_s3, st, p);
  }
  NHA_CHECK_LAUNCH("nha_prefill_bwd(state gradients)");
  hipLaunchKernelGGL((bwd_gate_local_kernel<T>), dim3(a->NT, a->H), dim3(256), 0, st, p);
  hipLaunchKernelGGL((bwd_gate_scan_kernel<T>), dim3(a->N * a->H), dim3(64), 0, st, p);
  hipLaunchKernelGGL((bwd_gate_final_kernel<T>), dim3(a->NT, a->H), dim3(256), 0, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(gate scan)");
  if (wmfma) return bwd_window_mfma_dkv(a, p.delta, p.dvs, sc + sp.ld);
  hipLaunchKernelGGL((bwd_kv_window_kernel<T>), dim3(a->T_tot, a->H), dim3(256), lds_w, st, p);
  NHA_CHECK_LAUNCH("nha_prefill_bwd(key pass)");
  return NHA_OK;
}

}  // namespace

size_t prefill_bwd_scratch_bytes(const NhaPrefillBwdArgs* a) {
  NhaPrefillArgs f = forward_args(a);
  return plan_bwd(a, f).total;
}

bool prefill_bwd_supported(const NhaPrefillBwdArgs* a) { return a->K <= 256 && a->V <= 256 && a->M <= 64 && a->K % 8 == 0 && a->V % 8 == 0; }

int prefill_bwd_impl(const NhaPrefillBwdArgs* a) {
  if (a->dtype == NHA_DTYPE_BF16) return run_bwd<bf16_t>(a);
  return run_bwd<float>(a);
}

}  // namespace nha
