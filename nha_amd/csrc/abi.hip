// extern "C" surface of libnha_hip.so (declared in include/nha_hip.h): argument validation,
// implementation choice, the host-side varlen chunk tables and the error string.
#include "common.h"

#include <string.h>

#include <mutex>

namespace nha {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

static int check_prefill(const NhaPrefillArgs* a, bool pointers, bool own_scratch = false) {
  NHA_CHECK_ARG(a != nullptr, "nha_prefill: null args");
  NHA_CHECK_ARG(a->T_tot > 0 && a->N > 0 && a->NT > 0 && a->HQ > 0 && a->H > 0 && a->K > 0 && a->V > 0 && a->M > 0,
                "nha_prefill: non-positive dimension");
  NHA_CHECK_ARG(a->HQ % a->H == 0, "nha_prefill: HQ (%d) must be a multiple of H (%d)", a->HQ, a->H);
  NHA_CHECK_ARG(a->shift >= 0, "nha_prefill: gsa_kv_shift must be >= 0, got %d", a->shift);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_prefill: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->impl >= NHA_IMPL_AUTO && a->impl <= NHA_IMPL_MFMA, "nha_prefill: bad impl %d", a->impl);
  if (pointers) {
    NHA_CHECK_ARG(a->q_swa && a->k_swa && a->q_gsa && a->k_gsa && a->v && a->s && a->g && a->o,
                  "nha_prefill_fwd: q_swa, k_swa, q_gsa, k_gsa, v, s, g, o are required");
    NHA_CHECK_ARG(a->cu_seqlens && a->chunk_indices && a->chunk_offsets,
                  "nha_prefill_fwd: cu_seqlens, chunk_indices and chunk_offsets are required");
    NHA_CHECK_ARG((a->h0k == nullptr) == (a->h0v == nullptr), "nha_prefill_fwd: pass both initial states or neither");
    NHA_CHECK_ARG((a->hkt == nullptr) == (a->hvt == nullptr), "nha_prefill_fwd: pass both final states or neither");
    NHA_CHECK_ARG(own_scratch || a->scratch != nullptr, "nha_prefill_fwd: scratch is required");
  }
  return NHA_OK;
}

// Scratch of nha_prefill_fwd_noalloc: device memory that is part of the loaded library, one copy per
// GPU at its own address, held until the process ends.  The name is a host-side handle only; host code
// uses the address hipGetSymbolAddress reports for the current device.
static __device__ __align__(256) unsigned char scratch[NHA_NOALLOC_SCRATCH_BYTES];

static int noalloc_scratch(void** out) {
  constexpr int MAX_DEV = 64;
  static std::mutex mu;
  static void* addr[MAX_DEV];
  static bool known[MAX_DEV];
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEV) {
    set_error("nha_prefill_fwd_noalloc: no usable current device (%s, ordinal %d)", hipGetErrorString(e), dev);
    return NHA_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!known[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("nha_prefill_fwd_noalloc: cannot locate the library's scratch array on device %d: %s", dev, hipGetErrorString(e));
      return NHA_ERR_LAUNCH;
    }
    addr[dev] = ptr;
    known[dev] = true;
  }
  *out = addr[dev];
  return NHA_OK;
}

static int check_prefill_bwd(const NhaPrefillBwdArgs* a, bool pointers) {
  NHA_CHECK_ARG(a != nullptr, "nha_prefill_bwd: null args");
  NHA_CHECK_ARG(a->T_tot > 0 && a->N > 0 && a->NT > 0 && a->HQ > 0 && a->H > 0 && a->K > 0 && a->V > 0 && a->M > 0,
                "nha_prefill_bwd: non-positive dimension");
  NHA_CHECK_ARG(a->HQ % a->H == 0, "nha_prefill_bwd: HQ (%d) must be a multiple of H (%d)", a->HQ, a->H);
  NHA_CHECK_ARG(a->shift >= 0, "nha_prefill_bwd: gsa_kv_shift must be >= 0, got %d", a->shift);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_prefill_bwd: bad dtype %d", a->dtype);
  if (pointers) {
    NHA_CHECK_ARG(a->q_swa && a->k_swa && a->q_gsa && a->k_gsa && a->v && a->s && a->g,
                  "nha_prefill_bwd: q_swa, k_swa, q_gsa, k_gsa, v, s, g are required");
    NHA_CHECK_ARG(a->o && a->lse_swa && a->lse_gsa && a->dout, "nha_prefill_bwd: o, lse_swa, lse_gsa and dout are required");
    NHA_CHECK_ARG(a->dq_swa && a->dk_swa && a->dq_gsa && a->dk_gsa && a->dv && a->ds && a->dg,
                  "nha_prefill_bwd: dq_swa, dk_swa, dq_gsa, dk_gsa, dv, ds, dg are required");
    NHA_CHECK_ARG(a->cu_seqlens && a->chunk_indices && a->chunk_offsets,
                  "nha_prefill_bwd: cu_seqlens, chunk_indices and chunk_offsets are required");
    NHA_CHECK_ARG((a->h0k == nullptr) == (a->h0v == nullptr), "nha_prefill_bwd: pass both initial states or neither");
    NHA_CHECK_ARG((a->dhkt == nullptr) == (a->dhvt == nullptr), "nha_prefill_bwd: pass both final-state cotangents or neither");
    NHA_CHECK_ARG((a->dh0k == nullptr) == (a->dh0v == nullptr), "nha_prefill_bwd: pass both initial-state gradients or neither");
    NHA_CHECK_ARG(a->scratch != nullptr, "nha_prefill_bwd: scratch is required");
  }
  return NHA_OK;
}

static bool use_mfma(const NhaPrefillArgs* a) {
  if (a->impl == NHA_IMPL_SIMPLE) return false;
  return prefill_mfma_supported(a);
}

}  // namespace nha

using namespace nha;

extern "C" {

size_t nha_prefill_scratch_bytes(const NhaPrefillArgs* a) {
  if (check_prefill(a, false) != NHA_OK) return 0;
  return use_mfma(a) ? prefill_mfma_scratch_bytes(a) : prefill_simple_scratch_bytes(a);
}

// The forward in parts, for measurements (bench.py times the state pass and the output pass apart): phase 1 = the
// state pass only (fills the scratch, writes the final states), 2 = the output pass only (the scratch must hold a
// state pass of the same inputs), 0 = the whole op.  Exported, but no part of the public header: a user's call is
// nha_prefill_fwd.
static int prefill_fwd_phase(const NhaPrefillArgs* a, int phase);

int nha_internal_prefill_fwd_phase(const NhaPrefillArgs* a, int phase) {
  if (phase < 0 || phase > 2) {
    set_error("nha_internal_prefill_fwd_phase: bad phase %d", phase);
    return NHA_ERR_INVALID;
  }
  return prefill_fwd_phase(a, phase);
}

int nha_prefill_fwd(const NhaPrefillArgs* a) { return prefill_fwd_phase(a, 0); }

static int prefill_fwd_phase(const NhaPrefillArgs* a, int phase) {
  int rc = check_prefill(a, true);
  if (rc != NHA_OK) return rc;
  const bool mfma = use_mfma(a);
  if (a->impl == NHA_IMPL_MFMA && !mfma) {
    set_error("nha_prefill_fwd: the MFMA kernels are not built for dtype=%d K=%d V=%d M=%d HQ/H=%d", a->dtype, a->K,
              a->V, a->M, a->HQ / a->H);
    return NHA_ERR_UNSUPPORTED;
  }
  const size_t need = mfma ? prefill_mfma_scratch_bytes(a) : prefill_simple_scratch_bytes(a);
  if (a->scratch_bytes < need) {
    set_error("nha_prefill_fwd: scratch has %zu bytes, %zu needed", a->scratch_bytes, need);
    return NHA_ERR_SCRATCH;
  }
  return mfma ? prefill_mfma_impl(a, phase) : prefill_simple_impl(a, phase);
}

int nha_prefill_fwd_noalloc(const NhaPrefillArgs* a) {
  int rc = check_prefill(a, true, true);
  if (rc != NHA_OK) return rc;
  const bool mfma = use_mfma(a);
  if (a->impl == NHA_IMPL_MFMA && !mfma) {
    set_error("nha_prefill_fwd_noalloc: the MFMA kernels are not built for dtype=%d K=%d V=%d M=%d HQ/H=%d", a->dtype, a->K,
              a->V, a->M, a->HQ / a->H);
    return NHA_ERR_UNSUPPORTED;
  }
  const size_t need = mfma ? prefill_mfma_scratch_bytes(a) : prefill_simple_scratch_bytes(a);
  if (need > (size_t)NHA_NOALLOC_SCRATCH_BYTES) {
    set_error("nha_prefill_fwd_noalloc: this call needs %zu bytes of scratch, the library's array holds %zu "
              "(use nha_prefill_fwd with a workspace of nha_prefill_scratch_bytes() bytes)", need, (size_t)NHA_NOALLOC_SCRATCH_BYTES);
    return NHA_ERR_SCRATCH;
  }
  void* ptr = nullptr;
  rc = noalloc_scratch(&ptr);
  if (rc != NHA_OK) return rc;
  // nothing in the scratch has to start at zero: the state pass writes every table the output pass
  // reads (rows past a sequence's end are never read), so the previous call's contents are harmless
  NhaPrefillArgs b = *a;
  b.scratch = ptr;
  b.scratch_bytes = (size_t)NHA_NOALLOC_SCRATCH_BYTES;
  return mfma ? prefill_mfma_impl(&b, 0) : prefill_simple_impl(&b, 0);
}

size_t nha_prefill_bwd_scratch_bytes(const NhaPrefillBwdArgs* a) {
  if (check_prefill_bwd(a, false) != NHA_OK) return 0;
  return prefill_bwd_scratch_bytes(a);
}

int nha_prefill_bwd(const NhaPrefillBwdArgs* a) {
  int rc = check_prefill_bwd(a, true);
  if (rc != NHA_OK) return rc;
  if (!prefill_bwd_supported(a)) {
    set_error("nha_prefill_bwd: built for K, V <= 256 (multiples of 8) and M <= 64, got K=%d V=%d M=%d", a->K, a->V, a->M);
    return NHA_ERR_UNSUPPORTED;
  }
  const size_t need = prefill_bwd_scratch_bytes(a);
  if (a->scratch_bytes < need) {
    set_error("nha_prefill_bwd: scratch has %zu bytes, %zu needed", a->scratch_bytes, need);
    return NHA_ERR_SCRATCH;
  }
  return prefill_bwd_impl(a);
}

int nha_decode_step(const NhaDecodeArgs* a) { return decode_step_impl(a); }

int nha_decode_advance(int32_t* count, int32_t B, void* stream) { return decode_advance_impl(count, B, stream); }

int nha_layer_prologue(const NhaLayerPrologueArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_layer_prologue: null args");
  NHA_CHECK_ARG(a->T_tot > 0 && a->N > 0 && a->HQ > 0 && a->H > 0 && a->K > 0 && a->V > 0 && a->M > 0,
                "nha_layer_prologue: non-positive dimension");
  NHA_CHECK_ARG(a->K % 2 == 0 && a->K <= 1024, "nha_layer_prologue: K must be even and <= 1024, got %d", a->K);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_layer_prologue: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->feature_map >= NHA_FMAP_NONE && a->feature_map <= NHA_FMAP_RELU,
                "nha_layer_prologue: bad feature_map %d", a->feature_map);
  NHA_CHECK_ARG(a->q && a->k && a->v && a->f && a->q_swa && a->k_swa && a->v_out && a->s && a->g && a->inv_freq,
                "nha_layer_prologue: q, k, v, f, q_swa, k_swa, v_out, s, g, inv_freq are required");
  NHA_CHECK_ARG(a->feature_map == NHA_FMAP_NONE || (a->q_gsa && a->k_gsa),
                "nha_layer_prologue: q_gsa and k_gsa are required with a feature map");
  NHA_CHECK_ARG(a->cu_seqlens != nullptr || a->T_tot % a->N == 0,
                "nha_layer_prologue: T_tot (%d) must be a multiple of N (%d) without cu_seqlens", a->T_tot, a->N);
  NHA_CHECK_ARG(a->gate_logit_normalizer != 0.f, "nha_layer_prologue: gate_logit_normalizer must not be 0");
  const void* ptrs[] = {a->q, a->k, a->v, a->f, a->q_swa, a->k_swa, a->q_gsa, a->k_gsa, a->v_out, a->s, a->g};
  for (const void* p : ptrs)
    NHA_CHECK_ARG((reinterpret_cast<uintptr_t>(p) & 15) == 0, "nha_layer_prologue: tensors must be 16-byte aligned");
  return layer_prologue_impl(a);
}

int nha_hybrid_prologue(const NhaHybridPrologueArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_hybrid_prologue: null args");
  NHA_CHECK_ARG(a->B > 0 && a->T > 0 && a->HQ > 0 && a->H > 0 && a->M > 0, "nha_hybrid_prologue: non-positive dimension");
  NHA_CHECK_ARG(a->D == 64 || a->D == 128 || a->D == 256, "nha_hybrid_prologue: head size must be 64, 128 or 256, got %d", a->D);
  NHA_CHECK_ARG(a->M % 8 == 0, "nha_hybrid_prologue: M must be a multiple of 8, got %d", a->M);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_hybrid_prologue: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->q && a->k && a->v, "nha_hybrid_prologue: q, k, v are required");
  NHA_CHECK_ARG((a->cos && a->sin) || (a->positions && a->inv_freq),
                "nha_hybrid_prologue: pass cos and sin, or positions and inv_freq");
  NHA_CHECK_ARG(a->q_out && a->sq_out && a->k_out && a->sk_out && a->v_out && a->g_out,
                "nha_hybrid_prologue: q_out, sq_out, k_out, sk_out, v_out, g_out are required");
  NHA_CHECK_ARG((a->q_weight == nullptr) == (a->k_weight == nullptr), "nha_hybrid_prologue: pass both norm weights or neither");
  NHA_CHECK_ARG(a->gate_logit_normalizer != 0.f, "nha_hybrid_prologue: gate_logit_normalizer must not be 0");
  const int64_t esz = a->dtype == NHA_DTYPE_BF16 ? 2 : 4;
  NHA_CHECK_ARG(a->q_stride >= (int64_t)a->HQ * a->D && a->k_stride >= (int64_t)a->H * a->D && a->v_stride >= (int64_t)a->H * a->D &&
                    (a->f == nullptr || a->f_stride >= (int64_t)a->H * a->M),
                "nha_hybrid_prologue: a row stride is shorter than its row");
  NHA_CHECK_ARG(a->cs_batch_stride == 0 || a->cs_batch_stride >= (int64_t)a->T * a->D, "nha_hybrid_prologue: bad cos / sin batch stride");
  const int64_t strides[] = {a->q_stride, a->k_stride, a->v_stride, a->f ? a->f_stride : 0, a->cs_batch_stride};
  for (int64_t s : strides) NHA_CHECK_ARG((s * esz) % 16 == 0, "nha_hybrid_prologue: strides must be multiples of 16 bytes");
  const void* ptrs[] = {a->q, a->k, a->v, a->f, a->q_weight, a->k_weight, a->cos, a->sin, a->q_out, a->sq_out, a->k_out, a->sk_out,
                        a->v_out, a->g_out, a->s_out};
  for (const void* p : ptrs)
    NHA_CHECK_ARG((reinterpret_cast<uintptr_t>(p) & 15) == 0, "nha_hybrid_prologue: tensors must be 16-byte aligned");
  return hybrid_prologue_impl(a);
}

int nha_zero_sink_rescale(void* o, const float* lse_swa, int32_t B, int32_t T, int32_t HQ, int32_t D, int32_t W, int32_t M,
                          int32_t dtype, void* stream) {
  NHA_CHECK_ARG(o && lse_swa, "nha_zero_sink_rescale: o and lse_swa are required");
  NHA_CHECK_ARG(B > 0 && T > 0 && HQ > 0 && W > 0 && M >= 0, "nha_zero_sink_rescale: bad dimension");
  NHA_CHECK_ARG(D == 64 || D == 128 || D == 256, "nha_zero_sink_rescale: head size must be 64, 128 or 256, got %d", D);
  NHA_CHECK_ARG(dtype == NHA_DTYPE_F32 || dtype == NHA_DTYPE_BF16, "nha_zero_sink_rescale: bad dtype %d", dtype);
  NHA_CHECK_ARG((reinterpret_cast<uintptr_t>(o) & 15) == 0, "nha_zero_sink_rescale: o must be 16-byte aligned");
  NHA_CHECK_ARG((int64_t)B * T * HQ < ((int64_t)1 << 31), "nha_zero_sink_rescale: too many rows");
  return zero_sink_rescale_impl(o, lse_swa, B, T, HQ, D, W, M, dtype, stream);
}

static int check_sink_window(const NhaSinkWindowArgs* a, bool pointers) {
  NHA_CHECK_ARG(a != nullptr, "nha_sink_window_fwd: null args");
  NHA_CHECK_ARG(a->T_tot > 0 && a->N > 0 && a->NT > 0 && a->HQ > 0 && a->H > 0 && a->D > 0, "nha_sink_window_fwd: non-positive dimension");
  NHA_CHECK_ARG(a->HQ % a->H == 0, "nha_sink_window_fwd: HQ (%d) must be a multiple of H (%d)", a->HQ, a->H);
  NHA_CHECK_ARG(a->window >= 1 && a->sinks >= 0, "nha_sink_window_fwd: window must be >= 1 and sinks >= 0, got %d / %d", a->window, a->sinks);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_sink_window_fwd: bad dtype %d", a->dtype);
  if (pointers) {
    NHA_CHECK_ARG(a->q && a->k && a->v && a->o, "nha_sink_window_fwd: q, k, v, o are required");
    NHA_CHECK_ARG(a->cu_seqlens && a->chunk_indices && a->chunk_offsets,
                  "nha_sink_window_fwd: cu_seqlens, chunk_indices and chunk_offsets are required");
    NHA_CHECK_ARG(a->scratch != nullptr, "nha_sink_window_fwd: scratch is required");
  }
  return NHA_OK;
}

size_t nha_sink_window_scratch_bytes(const NhaSinkWindowArgs* a) {
  if (check_sink_window(a, false) != NHA_OK) return 0;
  return sink_window_scratch_bytes(a);
}

int nha_sink_window_fwd(const NhaSinkWindowArgs* a) {
  const int rc = check_sink_window(a, true);
  if (rc != NHA_OK) return rc;
  const size_t need = sink_window_scratch_bytes(a);
  if (a->scratch_bytes < need) {
    set_error("nha_sink_window_fwd: scratch has %zu bytes, %zu needed", a->scratch_bytes, need);
    return NHA_ERR_SCRATCH;
  }
  return sink_window_impl(a);
}

int nha_layer_epilogue(const NhaLayerEpilogueArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_layer_epilogue: null args");
  NHA_CHECK_ARG(a->rows > 0 && a->dim > 0, "nha_layer_epilogue: non-positive dimension");
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_layer_epilogue: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->o && a->y, "nha_layer_epilogue: o and y are required");
  NHA_CHECK_ARG(((reinterpret_cast<uintptr_t>(a->o) | reinterpret_cast<uintptr_t>(a->y)) & 15) == 0,
                "nha_layer_epilogue: tensors must be 16-byte aligned");
  return layer_epilogue_impl(a);
}

int nha_layer_prologue_bwd(const NhaLayerPrologueBwdArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_layer_prologue_bwd: null args");
  NHA_CHECK_ARG(a->T_tot > 0 && a->N > 0 && a->HQ > 0 && a->H > 0 && a->K > 0 && a->V > 0 && a->M > 0,
                "nha_layer_prologue_bwd: non-positive dimension");
  NHA_CHECK_ARG(a->K % 2 == 0 && a->K <= 1024, "nha_layer_prologue_bwd: K must be even and <= 1024, got %d", a->K);
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_layer_prologue_bwd: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->feature_map >= NHA_FMAP_NONE && a->feature_map <= NHA_FMAP_RELU,
                "nha_layer_prologue_bwd: bad feature_map %d", a->feature_map);
  NHA_CHECK_ARG(a->q && a->k && a->v && a->f && a->dq_swa && a->dk_swa && a->dv_out && a->ds && a->dg && a->dq && a->dk &&
                    a->dv && a->df && a->inv_freq,
                "nha_layer_prologue_bwd: q, k, v, f, dq_swa, dk_swa, dv_out, ds, dg, dq, dk, dv, df, inv_freq are required");
  NHA_CHECK_ARG(a->feature_map == NHA_FMAP_NONE || (a->dq_gsa && a->dk_gsa),
                "nha_layer_prologue_bwd: dq_gsa and dk_gsa are required with a feature map");
  NHA_CHECK_ARG(a->cu_seqlens != nullptr || a->T_tot % a->N == 0,
                "nha_layer_prologue_bwd: T_tot (%d) must be a multiple of N (%d) without cu_seqlens", a->T_tot, a->N);
  NHA_CHECK_ARG(a->gate_logit_normalizer != 0.f, "nha_layer_prologue_bwd: gate_logit_normalizer must not be 0");
  const void* ptrs[] = {a->q, a->k, a->v, a->f, a->dq_swa, a->dk_swa, a->dq_gsa, a->dk_gsa, a->dv_out, a->ds, a->dg,
                        a->dq, a->dk, a->dv, a->df};
  for (const void* p : ptrs)
    NHA_CHECK_ARG((reinterpret_cast<uintptr_t>(p) & 15) == 0, "nha_layer_prologue_bwd: tensors must be 16-byte aligned");
  return layer_prologue_bwd_impl(a);
}

int32_t nha_layer_epilogue_bwd_parts(int32_t rows) { return rows > 0 ? layer_epilogue_bwd_parts(rows) : 0; }

int nha_layer_epilogue_bwd(const NhaLayerEpilogueBwdArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_layer_epilogue_bwd: null args");
  NHA_CHECK_ARG(a->rows > 0 && a->dim > 0, "nha_layer_epilogue_bwd: non-positive dimension");
  NHA_CHECK_ARG(a->dtype == NHA_DTYPE_F32 || a->dtype == NHA_DTYPE_BF16, "nha_layer_epilogue_bwd: bad dtype %d", a->dtype);
  NHA_CHECK_ARG(a->o && a->dy && a->dout, "nha_layer_epilogue_bwd: o, dy and dout are required");
  const void* ptrs[] = {a->o, a->dy, a->dout, a->weight, a->dweight_partial, a->dbias_partial};
  for (const void* p : ptrs)
    NHA_CHECK_ARG((reinterpret_cast<uintptr_t>(p) & 15) == 0, "nha_layer_epilogue_bwd: tensors must be 16-byte aligned");
  return layer_epilogue_bwd_impl(a);
}

static int check_short_conv(const char* who, const void* x, const void* w, int T_tot, int N, int C, int KS, int act, int dtype) {
  NHA_CHECK_ARG(T_tot > 0 && N > 0 && C > 0, "%s: non-positive dimension", who);
  NHA_CHECK_ARG(dtype == NHA_DTYPE_F32 || dtype == NHA_DTYPE_BF16, "%s: bad dtype %d", who, dtype);
  NHA_CHECK_ARG(x && w, "%s: x and weight are required", who);
  NHA_CHECK_ARG(act == 0 || act == 1, "%s: activation must be 0 (none) or 1 (SiLU), got %d", who, act);
  if (KS < 2 || KS > 4 || C % 8 != 0) {
    nha::set_error("%s: kernel size must be 2, 3 or 4 and C a multiple of 8 (got KS = %d, C = %d)", who, KS, C);
    return NHA_ERR_UNSUPPORTED;
  }
  NHA_CHECK_ARG((reinterpret_cast<uintptr_t>(x) & 15) == 0, "%s: tensors must be 16-byte aligned", who);
  return NHA_OK;
}

int nha_short_conv(const NhaShortConvArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_short_conv: null args");
  const int rc = check_short_conv("nha_short_conv", a->x, a->weight, a->T_tot, a->N, a->C, a->KS, a->activation, a->dtype);
  if (rc != NHA_OK) return rc;
  NHA_CHECK_ARG(a->y != nullptr && (reinterpret_cast<uintptr_t>(a->y) & 15) == 0, "nha_short_conv: y is required, 16-byte aligned");
  NHA_CHECK_ARG(a->cu_seqlens || a->T_tot % a->N == 0, "nha_short_conv: T_tot must be a multiple of N without cu_seqlens");
  return short_conv_impl(a);
}

int32_t nha_short_conv_bwd_parts(int32_t T_tot) { return T_tot > 0 ? short_conv_bwd_parts(T_tot) : 0; }

int nha_short_conv_bwd(const NhaShortConvBwdArgs* a) {
  NHA_CHECK_ARG(a != nullptr, "nha_short_conv_bwd: null args");
  const int rc = check_short_conv("nha_short_conv_bwd", a->x, a->weight, a->T_tot, a->N, a->C, a->KS, a->activation, a->dtype);
  if (rc != NHA_OK) return rc;
  NHA_CHECK_ARG(a->dy && a->dx, "nha_short_conv_bwd: dy and dx are required");
  NHA_CHECK_ARG(((reinterpret_cast<uintptr_t>(a->dy) | reinterpret_cast<uintptr_t>(a->dx)) & 15) == 0,
                "nha_short_conv_bwd: tensors must be 16-byte aligned");
  NHA_CHECK_ARG(a->cu_seqlens || a->T_tot % a->N == 0, "nha_short_conv_bwd: T_tot must be a multiple of N without cu_seqlens");
  return short_conv_bwd_impl(a);
}

int32_t nha_varlen_num_chunks(const int32_t* cu, int32_t N, int32_t BT) {
  if (!cu || N <= 0 || BT <= 0) {
    set_error("nha_varlen_num_chunks: bad arguments");
    return NHA_ERR_INVALID;
  }
  if (cu[0] != 0) {
    set_error("nha_varlen_num_chunks: cu_seqlens[0] must be 0, got %d", cu[0]);
    return NHA_ERR_INVALID;
  }
  int64_t nt = 0;
  for (int n = 0; n < N; ++n) {
    const int64_t len = (int64_t)cu[n + 1] - cu[n];
    if (len <= 0) {
      set_error("nha_varlen_num_chunks: cu_seqlens must be strictly increasing (sequence %d has length %lld)", n,
                (long long)len);
      return NHA_ERR_INVALID;
    }
    nt += (len + BT - 1) / BT;
  }
  if (nt > INT32_MAX) {
    set_error("nha_varlen_num_chunks: too many chunks");
    return NHA_ERR_INVALID;
  }
  return (int32_t)nt;
}

int nha_varlen_indices(const int32_t* cu, int32_t N, int32_t BT, int32_t* chunk_idx, int32_t* chunk_off) {
  const int32_t nt = nha_varlen_num_chunks(cu, N, BT);
  if (nt < 0) return nt;
  if (!chunk_idx || !chunk_off) {
    set_error("nha_varlen_indices: null output");
    return NHA_ERR_INVALID;
  }
  int32_t row = 0;
  for (int32_t n = 0; n < N; ++n) {
    chunk_off[n] = row;
    const int32_t nc = (int32_t)(((int64_t)cu[n + 1] - cu[n] + BT - 1) / BT);
    for (int32_t i = 0; i < nc; ++i) {
      chunk_idx[2 * row] = n;
      chunk_idx[2 * row + 1] = i;
      ++row;
    }
  }
  chunk_off[N] = row;
  return NHA_OK;
}

const char* nha_last_error(void) { return g_err; }

int nha_abi_version(void) { return NHA_ABI_VERSION; }

}  // extern "C"
