/*
 * nha_hip.h -- C ABI of libnha_hip.so: the MI355X (gfx950) implementation of NHA's fused
 * hybrid-attention hot path (gated-slot memory + sliding window under ONE softmax).
 *
 * The reference (JusenD/NHA) has no FFI layer: its boundary is the Python op API
 *   nha_fla/ops/nha/chunk.py:568-585            chunk_nha
 *   nha_fla/ops/nha/chunk_fused.py:291-303      fused_chunk_nha_prefill
 *   nha_fla/ops/nha/fused_recurrent.py:431-445  fused_recurrent_nha_decode
 *   nha_fla/ops/nha/fused_recurrent.py:588-598  fused_recurrent_nha
 * and, one level up, the layer nha_fla/layers/nha.py:147-282, whose elementwise glue around the
 * op (lines 214-237 and 278) has entry points here too.
 * Each entry point below states which of those it sits behind.  The host-side mirror of that
 * Python API (same names, argument meaning and error behaviour) is nha_amd/ops.py, which binds
 * this library with ctypes; no torch type crosses this boundary.
 *
 * Conventions: every pointer is a DEVICE pointer unless marked "host"; the caller owns every
 * buffer (the library never allocates or frees device memory); tensors are dense row-major in
 * the stated shape; functions return NHA_OK or a negative NHA_ERR_* code and never throw;
 * nha_last_error() gives the message of the calling thread's last failure.  Work is enqueued on
 * `stream` (a hipStream_t, may be NULL for the default stream) and is asynchronous.
 */
#ifndef NHA_HIP_H
#define NHA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NHA_ABI_VERSION 9

enum { NHA_DTYPE_F32 = 0, NHA_DTYPE_BF16 = 1 };
enum {
  NHA_OK = 0,
  NHA_ERR_INVALID = -1,      /* bad argument (null pointer, non-positive dim, HQ % H != 0 ...) */
  NHA_ERR_UNSUPPORTED = -2,  /* valid call the kernels cannot serve (shape outside the built set) */
  NHA_ERR_SCRATCH = -3,      /* scratch buffer smaller than nha_prefill_scratch_bytes() */
  NHA_ERR_LAUNCH = -4        /* HIP reported an error at launch */
};
enum { NHA_IMPL_AUTO = 0, NHA_IMPL_SIMPLE = 1, NHA_IMPL_MFMA = 2 };

/* ------------------------------------------------------------------------------------------
 * Chunked prefill forward.  Replaces ChunkNativeHybridAttentionFunction.forward
 * (nha_fla/ops/nha/chunk.py:367-488: optional slot-branch shift :401-420, SWA branch :423-431,
 * GSA branch :437-445, LSE merge :459-470) and the two kernels of fused_chunk_nha_prefill
 * (nha_fla/ops/nha/chunk_fused.py:30-283), GQA-native.
 *
 * Packed token-major layout (the reference's flattened '(b t) h d', chunk.py:665-671):
 *   q_swa, q_gsa [T_tot, HQ, K]   k_swa, k_gsa [T_tot, H, K]   v [T_tot, H, V]   s, g [T_tot, H, M]
 *   o [T_tot, HQ, V] (input dtype)   lse_swa, lse_gsa [T_tot, HQ] fp32 (either may be NULL)
 *   h0k [N,H,K,M], h0v [N,H,M,V] fp32 or NULL;  hkt, hvt same shapes, or NULL when not wanted
 *   cu_seqlens int32 [N+1] (batched mode: arange(0,(B+1)T,T), chunk.py:660)
 *   chunk_indices int32 [NT,2] rows (sequence, chunk-in-sequence), chunk_offsets int32 [N+1]:
 *     as produced by nha_varlen_indices() with chunk size 64.
 * Semantics per token t of a sequence [bos,eos): window keys j in [max(bos, t-wl), t] (wl < 0:
 * unbounded); the slots have absorbed tokens bos .. t-shift (shift >= 0); one softmax over
 * [M slot logits | window logits]; q-head hq reads kv-head hq / (HQ/H).
 * ------------------------------------------------------------------------------------------ */
typedef struct NhaPrefillArgs {
  const void* q_swa;
  const void* k_swa;
  const void* q_gsa;
  const void* k_gsa;
  const void* v;
  const void* s;
  const void* g;
  void* o;
  float* lse_swa;
  float* lse_gsa;
  const float* h0k;
  const float* h0v;
  float* hkt;
  float* hvt;
  const int32_t* cu_seqlens;
  const int32_t* chunk_indices;
  const int32_t* chunk_offsets;
  void* scratch;
  size_t scratch_bytes;
  int32_t T_tot, N, NT, HQ, H, K, V, M;
  int32_t wl;     /* window_size_left; < 0 = unbounded */
  int32_t shift;  /* gsa_kv_shift */
  int32_t dtype;  /* NHA_DTYPE_* of q/k/v/s/g/o */
  int32_t impl;   /* NHA_IMPL_* */
  float scale;
  void* stream;
} NhaPrefillArgs;

/* Bytes of device scratch nha_prefill_fwd needs for these dims (chunk-start slot states, gate
 * cumsums, staging).  Only the integer/dtype/impl fields of `a` are read. */
size_t nha_prefill_scratch_bytes(const NhaPrefillArgs* a);
int nha_prefill_fwd(const NhaPrefillArgs* a);

/* nha_prefill_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same arguments, kernels and results, but
 * `scratch` / `scratch_bytes` are ignored and the workspace is an array of
 * NHA_NOALLOC_SCRATCH_BYTES that is part of the loaded library (one per GPU, held until the process
 * ends).  The call allocates and frees nothing.  It returns NHA_ERR_SCRATCH when
 * nha_prefill_scratch_bytes(a) exceeds NHA_NOALLOC_SCRATCH_BYTES (bf16, D = 128: about 400 chunks x
 * kv-heads, e.g. 3200 tokens at 8 kv-heads).  Every call on a GPU shares that GPU's array: calls
 * that overlap on one GPU (different streams or threads) race and must be serialised by the
 * caller; successive calls on one stream are ordered by the stream.  No counterpart in the
 * reference, whose ops allocate their intermediates through torch. */
#define NHA_NOALLOC_SCRATCH_BYTES (32u << 20)
int nha_prefill_fwd_noalloc(const NhaPrefillArgs* a);

/* ------------------------------------------------------------------------------------------
 * Chunked prefill backward.  Replaces ChunkNativeHybridAttentionFunction.backward
 * (nha_fla/ops/nha/chunk.py:490-564: window-branch backward :499-511, slot-branch backward with
 * the LSE coupling of the merged softmax :514-530 and nha_fla/ops/nha/chunk_gsa.py:52-122,
 * un-shifting of the slot-branch gradients :533-543, dv accumulated over both branches :559).
 *
 * Inputs: the forward's inputs (same layouts and dims as NhaPrefillArgs), its outputs o, lse_swa,
 * lse_gsa (all three required), the initial states if the forward had them, and the cotangents
 * dout [T_tot,HQ,V] (input dtype; required), dlse_swa / dlse_gsa [T_tot,HQ] fp32 and dhkt
 * [N,H,K,M] / dhvt [N,H,M,V] fp32 (each NULL = zero).  Outputs: dq_swa, dq_gsa [T_tot,HQ,K],
 * dk_swa, dk_gsa [T_tot,H,K], dv [T_tot,H,V], ds, dg [T_tot,H,M] in the input dtype (all
 * required, fully written), and dh0k / dh0v fp32 (NULL = not wanted).  fp32 arithmetic
 * throughout; K, V <= 256 (multiples of 8), M <= 64.  The slot states are recomputed from the
 * inputs into the scratch, nothing else is kept from the forward.
 * ------------------------------------------------------------------------------------------ */
typedef struct NhaPrefillBwdArgs {
  const void* q_swa;
  const void* k_swa;
  const void* q_gsa;
  const void* k_gsa;
  const void* v;
  const void* s;
  const void* g;
  const void* o;
  const float* lse_swa;
  const float* lse_gsa;
  const float* h0k;
  const float* h0v;
  const void* dout;
  const float* dlse_swa;
  const float* dlse_gsa;
  const float* dhkt;
  const float* dhvt;
  void* dq_swa;
  void* dk_swa;
  void* dq_gsa;
  void* dk_gsa;
  void* dv;
  void* ds;
  void* dg;
  float* dh0k;
  float* dh0v;
  const int32_t* cu_seqlens;
  const int32_t* chunk_indices;
  const int32_t* chunk_offsets;
  void* scratch;
  size_t scratch_bytes;
  int32_t T_tot, N, NT, HQ, H, K, V, M;
  int32_t wl;
  int32_t shift;
  int32_t dtype;
  float scale;
  void* stream;
} NhaPrefillBwdArgs;

size_t nha_prefill_bwd_scratch_bytes(const NhaPrefillBwdArgs* a);
int nha_prefill_bwd(const NhaPrefillBwdArgs* a);

/* ------------------------------------------------------------------------------------------
 * Single-token decode step.  Replaces the k/v kernel pair of fused_recurrent_nha_decode
 * (nha_fla/ops/nha/fused_recurrent.py:228-428, host :431-584) and, with `win_logits`, the
 * kernel pair + host softmax of fused_recurrent_nha (:47-225).  One launch; a workgroup owns a
 * (sequence, kv-head) and serves all HQ/H query heads, so state and window are read once.
 *
 * mode NHA_DECODE_WINDOW: explicit popped entry k_pop/v_pop/g_pop [B,H,*] (s_pop optional,
 *   else 1-exp(g), :282-285) and a time-ordered window win_k/win_v [B,W,H,*], all W rows valid
 *   (:287-288).  Either `sq` (pre-rotated query, pre-rotated win_k) or cos/sin tables
 *   [B|1, W, K] (row stride cos_sw, batch stride cos_sb = 0 to broadcast; row W-1 is the query
 *   position) for in-kernel rotate-half RoPE of raw q / win_k (:309-329).
 * mode NHA_DECODE_LOGITS: explicit popped entry and caller-supplied window logits
 *   win_logits [B,HQ,W] (input dtype); writes the window probabilities win_probs [B,HQ,W] fp32
 *   and the slot part of the output only (:200-205, :143-145).
 * mode NHA_DECODE_RING: W-slot ring buffers ring_k (window keys), ring_kg (slot-branch keys),
 *   ring_v, ring_g [B,W,H,*] resident in HBM and count[b] = tokens cached so far.  The step
 *   pops slot count%W into the slots when count >= W, stores the new token (k_new, kg_new,
 *   v_new, g_new [B,H,*]) there, and attends over the min(count+1, W) valid entries.  The
 *   counters advance either in the same launch, into a second array (count_next[b] = count[b]+1;
 *   the caller then swaps the two arrays), or by nha_decode_advance after the step; count itself
 *   is never written by nha_decode_step.  No reference counterpart: it
 *   replaces the cat-shift cache of nha_fla/models/nha_cache.py:105-131, :143-154.
 * State hk [B,H,K,M], hv [B,H,M,V] fp32: read from hk_in/hv_in (NULL = zeros), written to
 * hk_out/hv_out (NULL = not written; may alias the inputs, fused_recurrent.py:541-545).
 * o [B,HQ,V] in the input dtype.
 * ------------------------------------------------------------------------------------------ */
enum { NHA_DECODE_WINDOW = 0, NHA_DECODE_LOGITS = 1, NHA_DECODE_RING = 2 };

typedef struct NhaDecodeArgs {
  int32_t mode;
  int32_t dtype;
  int32_t B, HQ, H, K, V, M, W;
  float scale;
  const void* q;   /* [B,HQ,K] raw query: slot logits (and the rotated window query when cos/sin) */
  const void* sq;  /* [B,HQ,K] pre-rotated window query, or NULL */
  const void* k_pop;
  const void* v_pop;
  const void* g_pop;
  const void* s_pop;
  const void* win_k;
  const void* win_v;
  const void* cos;
  const void* sin;
  int64_t cos_sb, cos_sw;
  const void* win_logits;
  float* win_probs;
  void* ring_k;
  void* ring_kg;
  void* ring_v;
  void* ring_g;
  const void* k_new;
  const void* kg_new;
  const void* v_new;
  const void* g_new;
  const int32_t* count;
  const float* hk_in;
  const float* hv_in;
  float* hk_out;
  float* hv_out;
  void* o;
  void* stream;
  int32_t* count_next; /* ring mode, optional: receives count[b] + 1 (must not alias count) */
} NhaDecodeArgs;

int nha_decode_step(const NhaDecodeArgs* a);
/* count[b] += 1 for b < B (ring mode bookkeeping between steps). */
int nha_decode_advance(int32_t* count, int32_t B, void* stream);

/* ------------------------------------------------------------------------------------------
 * Varlen chunk tables (HOST pointers, pure integer, no GPU).  Replaces fla's
 * prepare_chunk_indices / prepare_chunk_offsets as consumed at
 * nha_fla/ops/nha_naive/chunk.py:59-64, :557-558: rows (i_n, i_t) in sequence-major order,
 * NT = sum_n ceil(L_n / BT); chunk_off is the exclusive prefix sum of ceil(L_n / BT).
 * nha_varlen_num_chunks returns NT (or a negative error for a non-increasing cu_seqlens).
 * ------------------------------------------------------------------------------------------ */
int32_t nha_varlen_num_chunks(const int32_t* cu_seqlens_host, int32_t N, int32_t BT);
int nha_varlen_indices(const int32_t* cu_seqlens_host, int32_t N, int32_t BT,
                       int32_t* chunk_idx_host /* [NT,2] */, int32_t* chunk_off_host /* [N+1] */);

/* ------------------------------------------------------------------------------------------
 * Layer glue on either side of the fused op, one launch each (device pointers, contiguous,
 * 16-byte aligned, all tensors in `dtype`).
 *
 * nha_layer_prologue replaces the chain of elementwise tensor ops at
 * nha_fla/layers/nha.py:214-237: from the raw projections q [T_tot,HQ,K], k [T_tot,H,K],
 * v [T_tot,H,V], f [T_tot,H,M] it writes
 *   q_swa, k_swa  rotate-half RoPE over the whole head dim (:237); the position of token t is
 *                 t - cu_seqlens[n] + seqlen_offset inside its sequence n, or (t mod T_tot/N) +
 *                 seqlen_offset when cu_seqlens is NULL; angle = position * inv_freq[i], i < K/2;
 *   q_gsa, k_gsa  the feature map of q, k (:219-222): NHA_FMAP_SWISH x*sigmoid(x), NHA_FMAP_RELU;
 *                 with NHA_FMAP_NONE they are not written (the caller passes q, k themselves);
 *   v_out         silu(v) (:223);
 *   g             logsigmoid(f) / gate_logit_normalizer, s = 1 - exp(g) (:225-227), each step
 *                 rounded to `dtype` as the reference's tensor ops round it.
 * k, v, s, g stay at the kv-head count H: the op reads them per group, the reference's repeat
 * (:229-230) is not materialised.
 *
 * nha_layer_epilogue replaces the normalisation half of rms_norm_linear(silu(o), ...) at
 * nha_fla/layers/nha.py:278: y[r,:] = silu(o[r,:]) * rsqrt(mean(silu(o[r,:])^2) + eps) * weight
 * (+ bias), rows of `dim` = HQ*V elements; weight and bias are fp32 [dim] or NULL.  The output
 * projection itself stays a library GEMM on the caller's side.
 * ------------------------------------------------------------------------------------------ */
#define NHA_FMAP_NONE 0
#define NHA_FMAP_SWISH 1
#define NHA_FMAP_RELU 2

typedef struct NhaLayerPrologueArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* f;
  void* q_swa;
  void* k_swa;
  void* q_gsa;
  void* k_gsa;
  void* v_out;
  void* s;
  void* g;
  const float* inv_freq;     /* [K/2] fp32 */
  const int32_t* cu_seqlens; /* device [N+1], or NULL */
  int32_t T_tot, N, HQ, H, K, V, M;
  int32_t feature_map;
  int32_t seqlen_offset;
  int32_t dtype;
  float gate_logit_normalizer;
  void* stream;
} NhaLayerPrologueArgs;

typedef struct NhaLayerEpilogueArgs {
  const void* o;
  void* y;
  const float* weight;
  const float* bias;
  int32_t rows, dim, dtype;
  float eps;
  void* stream;
} NhaLayerEpilogueArgs;

int nha_layer_prologue(const NhaLayerPrologueArgs* a);
int nha_layer_epilogue(const NhaLayerEpilogueArgs* a);

/* ------------------------------------------------------------------------------------------
 * Glue of the hybrid decoder models' attention blocks in one launch (inference): from the raw
 * projections of a block -- which may be column slices of one fused projection output: `*_stride`
 * is the number of elements between the rows of two tokens -- it writes the contiguous operands of
 * the prefill op and of the decode step.  Replaces the tensor-op chain of
 * nha_fla/models/qwen3_moe_nha/qwennha.py:103-106 (per-head RMSNorm of q and k: x * rsqrt(mean(x^2) +
 * eps) in fp32, rounded, times `q_weight` / `k_weight` [D]; NULL weights = the dense flavour,
 * nha_fla/models/llama3_nha/llamanha.py:79-81), :117-128 (g = logsigmoid(f) / normalizer,
 * s = 1 - exp(g), each step rounded to the tensor dtype), :133-144 (v and s times the padding mask
 * of the token, `mask` [B*T] in the tensor dtype or NULL), :240-247 (rotate-half rotary embedding with
 * cos / sin [B or 1, T, D] in the tensor dtype, `cs_batch_stride` = T*D or 0 -- or with `positions` and
 * `inv_freq`, from which the kernel forms the same table rows itself; the rotation is evaluated in fp32 and
 * rounded once).  Outputs: q_out / sq_out [B,T,HQ,D] (normed, and normed + rotated), k_out / sk_out [B,T,H,D],
 * v_out [B,T,H,D], g_out and s_out [B,T,H,M] (s_out may be NULL: a decode step does not read it).
 * f == NULL writes g = s = 0 (the layers whose slots never absorb anything).  D in {64, 128, 256},
 * M a multiple of 8, every pointer and stride 16-byte aligned. */
typedef struct NhaHybridPrologueArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* f;
  int64_t q_stride, k_stride, v_stride, f_stride;
  const void* q_weight;
  const void* k_weight;
  const void* cos;
  const void* sin;
  int64_t cs_batch_stride;
  const int64_t* positions; /* [B*T] token positions, with inv_freq [D/2] fp32: cos / sin of position * inv_freq are */
  const float* inv_freq;    /* formed in the kernel (fp32, rounded to the tensor dtype) and cos / sin are not read   */
  const void* mask;
  void* q_out;
  void* sq_out;
  void* k_out;
  void* sk_out;
  void* v_out;
  void* g_out;
  void* s_out;
  int32_t B, T, HQ, H, D, M;
  int32_t dtype;
  float eps;
  float gate_logit_normalizer;
  void* stream;
} NhaHybridPrologueArgs;

int nha_hybrid_prologue(const NhaHybridPrologueArgs* a);

/* ------------------------------------------------------------------------------------------
 * Sliding-window attention with zero sinks: the "full attention" layers of the hybrid models
 * (nha_fla/models/qwen3_moe_nha/qwennha.py:323-336 with naive_swa, :400-413;
 * nha_fla/models/llama3_nha/llamanha.py:204-216).  `sinks` all-zero key / value rows precede every
 * sequence; query t (position in its sequence) attends the keys j with t - window < j <= t and the
 * clamp(window - 1 - t, 0, sinks) sinks its window still covers, each with logit 0 and value 0:
 *   o_t = sum_j e^(scale q_t.k_j) v_j / (sum_j e^(scale q_t.k_j) + sinks_in_view(t)).
 * q [T_tot,HQ,D] and k, v [T_tot,H,D] packed as for nha_prefill_fwd (q and k already rotated), with the
 * same three index tables; o [T_tot,HQ,D]; lse [T_tot,HQ] fp32 or NULL: the log of the denominator.
 * One launch of the prefill's window loop (no slot branch, no state pass) + an exact pass for rows whose
 * sums leave the range of the fixed softmax reference.  Served: bf16, D = 64 or 128, HQ / H a
 * multiple of four; other shapes return NHA_ERR_UNSUPPORTED (callers then run nha_prefill_fwd with
 * zero slot writes and nha_zero_sink_rescale).  scratch: nha_sink_window_scratch_bytes(a) bytes. */
typedef struct NhaSinkWindowArgs {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  float* lse;
  const int32_t* cu_seqlens;
  const int32_t* chunk_indices;
  const int32_t* chunk_offsets;
  void* scratch;
  size_t scratch_bytes;
  int32_t T_tot, N, NT, HQ, H, D;
  int32_t window;
  int32_t sinks;
  int32_t dtype;
  float scale;
  void* stream;
} NhaSinkWindowArgs;

size_t nha_sink_window_scratch_bytes(const NhaSinkWindowArgs* a);
int nha_sink_window_fwd(const NhaSinkWindowArgs* a);

/* The "full attention" layers of the hybrid models (window 2048: a sliding-window softmax preceded by M all-zero
 * key / value rows, nha_fla/models/qwen3_moe_nha/qwennha.py:323-336, :400-413;
 * nha_fla/models/llama3_nha/llamanha.py:204-216) run through nha_prefill_fwd with slot states that stay zero, which
 * puts M zero-logit, zero-value keys into every query's softmax; the reference's window still covers
 * n0(t) = clamp(W - 1 - t, 0, M) of them at position t of its sequence.  This call multiplies row (b, t, head) of
 * o [B,T,HQ,D] in place by (e^lse + M) / (e^lse + n0(t)), lse = lse_swa [B,T,HQ] of that prefill call.
 * D in {64, 128, 256}; o 16-byte aligned. */
int nha_zero_sink_rescale(void* o, const float* lse_swa, int32_t B, int32_t T, int32_t HQ, int32_t D, int32_t W, int32_t M,
                          int32_t dtype, void* stream);

/* Backward of the two launches above (what autograd derives from the tensor-op chain of
 * nha_fla/layers/nha.py:214-237, :278; the reference has no hand-written counterpart).
 *
 * nha_layer_prologue_bwd: from the raw projections and the cotangents of the seven outputs it
 * writes dq, dk, dv, df: the rotation by the opposite angle of dq_swa / dk_swa plus the feature
 * map's derivative times dq_gsa / dk_gsa (not read with NHA_FMAP_NONE: the caller adds the slot
 * cotangent itself, q_gsa being q), dv_out * silu'(v), and
 * df = (dg - ds * exp(g)) / normalizer * sigmoid(-f).
 *
 * nha_layer_epilogue_bwd: dout = d silu(o) of the RMS-norm backward; the weight and bias
 * gradients leave as partial sums dweight_partial / dbias_partial [parts, dim] fp32 with
 * parts = nha_layer_epilogue_bwd_parts(rows), which the caller adds up over the first axis
 * (fixed order: run-to-run identical).  Either may be NULL.  dim: multiple of 8, <= 8192. */
typedef struct NhaLayerPrologueBwdArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* f;
  const void* dq_swa;
  const void* dk_swa;
  const void* dq_gsa;
  const void* dk_gsa;
  const void* dv_out;
  const void* ds;
  const void* dg;
  void* dq;
  void* dk;
  void* dv;
  void* df;
  const float* inv_freq;
  const int32_t* cu_seqlens;
  int32_t T_tot, N, HQ, H, K, V, M;
  int32_t feature_map;
  int32_t seqlen_offset;
  int32_t dtype;
  float gate_logit_normalizer;
  void* stream;
} NhaLayerPrologueBwdArgs;

typedef struct NhaLayerEpilogueBwdArgs {
  const void* o;
  const void* dy;
  void* dout;
  const float* weight;
  float* dweight_partial;
  float* dbias_partial;
  int32_t rows, dim, dtype;
  float eps;
  void* stream;
} NhaLayerEpilogueBwdArgs;

int nha_layer_prologue_bwd(const NhaLayerPrologueBwdArgs* a);
int32_t nha_layer_epilogue_bwd_parts(int32_t rows);
int nha_layer_epilogue_bwd(const NhaLayerEpilogueBwdArgs* a);

/* Depthwise causal short convolution with optional SiLU over packed tokens: what the layer applies to its
 * q / k / v projections when use_short_conv is set (nha_fla/layers/nha.py:121-140, :186-206; the module
 * itself, fla.modules.ShortConvolution, is a dependency outside the reference tree):
 *   y[t][c] = act(bias[c] + sum_{j < KS} weight[c][j] * x[t - (KS-1) + j][c])
 * with the taps that would reach before the first token of t's sequence taken as zero.  x, y [T_tot, C];
 * weight [C, KS] (the module's [C, 1, KS] parameter) and bias [C] (or NULL) in the dtype of x; cu_seqlens
 * [N+1] on the device, or NULL for N sequences of T_tot / N tokens.  KS in {2, 3, 4}, C a multiple of 8,
 * activation 0 (none) or 1 (SiLU).  fp32 arithmetic, rounded once.
 *
 * nha_short_conv_bwd: dx, and the weight / bias gradients as partial sums dweight_partial [parts, C, KS],
 * dbias_partial [parts, C] fp32 with parts = nha_short_conv_bwd_parts(T_tot), which the caller adds up over
 * the first axis (fixed order: run-to-run identical).  Either may be NULL. */
typedef struct NhaShortConvArgs {
  const void* x;
  const void* weight;
  const void* bias;
  void* y;
  const int32_t* cu_seqlens;
  int32_t T_tot, N, C, KS;
  int32_t activation;
  int32_t dtype;
  void* stream;
} NhaShortConvArgs;

typedef struct NhaShortConvBwdArgs {
  const void* x;
  const void* weight;
  const void* bias;
  const void* dy;
  void* dx;
  float* dweight_partial;
  float* dbias_partial;
  const int32_t* cu_seqlens;
  int32_t T_tot, N, C, KS;
  int32_t activation;
  int32_t dtype;
  void* stream;
} NhaShortConvBwdArgs;

int nha_short_conv(const NhaShortConvArgs* a);
int32_t nha_short_conv_bwd_parts(int32_t T_tot);
int nha_short_conv_bwd(const NhaShortConvBwdArgs* a);

const char* nha_last_error(void);
int nha_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* NHA_HIP_H */
