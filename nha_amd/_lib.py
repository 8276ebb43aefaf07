"""ctypes binding of libnha_hip.so (C ABI declared in include/nha_hip.h).

The library is built in-tree by nha_amd/build.py.  There is no CPU fallback: if the shared
object is missing or a call fails, the error is raised to the caller."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnha_hip.so")

NHA_DTYPE_F32, NHA_DTYPE_BF16 = 0, 1
NHA_IMPL_AUTO, NHA_IMPL_SIMPLE, NHA_IMPL_MFMA = 0, 1, 2
NHA_DECODE_WINDOW, NHA_DECODE_LOGITS, NHA_DECODE_RING = 0, 1, 2
NHA_OK, NHA_ERR_INVALID, NHA_ERR_UNSUPPORTED, NHA_ERR_SCRATCH, NHA_ERR_LAUNCH = 0, -1, -2, -3, -4
ABI_VERSION = 9
NHA_NOALLOC_SCRATCH_BYTES = 32 << 20   # workspace of nha_prefill_fwd_noalloc (include/nha_hip.h)
NHA_FMAP_NONE, NHA_FMAP_SWISH, NHA_FMAP_RELU = 0, 1, 2

EXPORTS = (
    "nha_prefill_scratch_bytes", "nha_prefill_fwd", "nha_prefill_fwd_noalloc", "nha_prefill_bwd_scratch_bytes", "nha_prefill_bwd",
    "nha_decode_step", "nha_decode_advance", "nha_layer_prologue", "nha_layer_epilogue",
    "nha_layer_prologue_bwd", "nha_layer_epilogue_bwd", "nha_layer_epilogue_bwd_parts",
    "nha_short_conv", "nha_short_conv_bwd", "nha_short_conv_bwd_parts", "nha_hybrid_prologue", "nha_zero_sink_rescale", "nha_sink_window_fwd", "nha_sink_window_scratch_bytes",
    "nha_varlen_num_chunks", "nha_varlen_indices", "nha_last_error", "nha_abi_version",
)


class NhaPrefillArgs(C.Structure):
    _fields_ = [
        ("q_swa", C.c_void_p), ("k_swa", C.c_void_p), ("q_gsa", C.c_void_p), ("k_gsa", C.c_void_p),
        ("v", C.c_void_p), ("s", C.c_void_p), ("g", C.c_void_p), ("o", C.c_void_p),
        ("lse_swa", C.c_void_p), ("lse_gsa", C.c_void_p),
        ("h0k", C.c_void_p), ("h0v", C.c_void_p), ("hkt", C.c_void_p), ("hvt", C.c_void_p),
        ("cu_seqlens", C.c_void_p), ("chunk_indices", C.c_void_p), ("chunk_offsets", C.c_void_p),
        ("scratch", C.c_void_p), ("scratch_bytes", C.c_size_t),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("NT", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32),
        ("K", C.c_int32), ("V", C.c_int32), ("M", C.c_int32),
        ("wl", C.c_int32), ("shift", C.c_int32), ("dtype", C.c_int32), ("impl", C.c_int32),
        ("scale", C.c_float), ("stream", C.c_void_p),
    ]


class NhaPrefillBwdArgs(C.Structure):
    _fields_ = [
        ("q_swa", C.c_void_p), ("k_swa", C.c_void_p), ("q_gsa", C.c_void_p), ("k_gsa", C.c_void_p),
        ("v", C.c_void_p), ("s", C.c_void_p), ("g", C.c_void_p),
        ("o", C.c_void_p), ("lse_swa", C.c_void_p), ("lse_gsa", C.c_void_p),
        ("h0k", C.c_void_p), ("h0v", C.c_void_p),
        ("dout", C.c_void_p), ("dlse_swa", C.c_void_p), ("dlse_gsa", C.c_void_p),
        ("dhkt", C.c_void_p), ("dhvt", C.c_void_p),
        ("dq_swa", C.c_void_p), ("dk_swa", C.c_void_p), ("dq_gsa", C.c_void_p), ("dk_gsa", C.c_void_p),
        ("dv", C.c_void_p), ("ds", C.c_void_p), ("dg", C.c_void_p),
        ("dh0k", C.c_void_p), ("dh0v", C.c_void_p),
        ("cu_seqlens", C.c_void_p), ("chunk_indices", C.c_void_p), ("chunk_offsets", C.c_void_p),
        ("scratch", C.c_void_p), ("scratch_bytes", C.c_size_t),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("NT", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32),
        ("K", C.c_int32), ("V", C.c_int32), ("M", C.c_int32),
        ("wl", C.c_int32), ("shift", C.c_int32), ("dtype", C.c_int32),
        ("scale", C.c_float), ("stream", C.c_void_p),
    ]


class NhaDecodeArgs(C.Structure):
    _fields_ = [
        ("mode", C.c_int32), ("dtype", C.c_int32),
        ("B", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32), ("K", C.c_int32), ("V", C.c_int32),
        ("M", C.c_int32), ("W", C.c_int32), ("scale", C.c_float),
        ("q", C.c_void_p), ("sq", C.c_void_p),
        ("k_pop", C.c_void_p), ("v_pop", C.c_void_p), ("g_pop", C.c_void_p), ("s_pop", C.c_void_p),
        ("win_k", C.c_void_p), ("win_v", C.c_void_p),
        ("cos", C.c_void_p), ("sin", C.c_void_p), ("cos_sb", C.c_int64), ("cos_sw", C.c_int64),
        ("win_logits", C.c_void_p), ("win_probs", C.c_void_p),
        ("ring_k", C.c_void_p), ("ring_kg", C.c_void_p), ("ring_v", C.c_void_p), ("ring_g", C.c_void_p),
        ("k_new", C.c_void_p), ("kg_new", C.c_void_p), ("v_new", C.c_void_p), ("g_new", C.c_void_p),
        ("count", C.c_void_p),
        ("hk_in", C.c_void_p), ("hv_in", C.c_void_p), ("hk_out", C.c_void_p), ("hv_out", C.c_void_p),
        ("o", C.c_void_p), ("stream", C.c_void_p), ("count_next", C.c_void_p),
    ]


class NhaLayerPrologueArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("f", C.c_void_p),
        ("q_swa", C.c_void_p), ("k_swa", C.c_void_p), ("q_gsa", C.c_void_p), ("k_gsa", C.c_void_p),
        ("v_out", C.c_void_p), ("s", C.c_void_p), ("g", C.c_void_p),
        ("inv_freq", C.c_void_p), ("cu_seqlens", C.c_void_p),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32),
        ("K", C.c_int32), ("V", C.c_int32), ("M", C.c_int32),
        ("feature_map", C.c_int32), ("seqlen_offset", C.c_int32), ("dtype", C.c_int32),
        ("gate_logit_normalizer", C.c_float), ("stream", C.c_void_p),
    ]


class NhaHybridPrologueArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("f", C.c_void_p),
        ("q_stride", C.c_int64), ("k_stride", C.c_int64), ("v_stride", C.c_int64), ("f_stride", C.c_int64),
        ("q_weight", C.c_void_p), ("k_weight", C.c_void_p), ("cos", C.c_void_p), ("sin", C.c_void_p),
        ("cs_batch_stride", C.c_int64), ("positions", C.c_void_p), ("inv_freq", C.c_void_p), ("mask", C.c_void_p),
        ("q_out", C.c_void_p), ("sq_out", C.c_void_p), ("k_out", C.c_void_p), ("sk_out", C.c_void_p),
        ("v_out", C.c_void_p), ("g_out", C.c_void_p), ("s_out", C.c_void_p),
        ("B", C.c_int32), ("T", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32), ("D", C.c_int32), ("M", C.c_int32),
        ("dtype", C.c_int32), ("eps", C.c_float), ("gate_logit_normalizer", C.c_float), ("stream", C.c_void_p),
    ]


class NhaSinkWindowArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("lse", C.c_void_p),
        ("cu_seqlens", C.c_void_p), ("chunk_indices", C.c_void_p), ("chunk_offsets", C.c_void_p),
        ("scratch", C.c_void_p), ("scratch_bytes", C.c_size_t),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("NT", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
        ("window", C.c_int32), ("sinks", C.c_int32), ("dtype", C.c_int32), ("scale", C.c_float), ("stream", C.c_void_p),
    ]


class NhaLayerEpilogueArgs(C.Structure):
    _fields_ = [
        ("o", C.c_void_p), ("y", C.c_void_p), ("weight", C.c_void_p), ("bias", C.c_void_p),
        ("rows", C.c_int32), ("dim", C.c_int32), ("dtype", C.c_int32), ("eps", C.c_float), ("stream", C.c_void_p),
    ]


class NhaLayerPrologueBwdArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("f", C.c_void_p),
        ("dq_swa", C.c_void_p), ("dk_swa", C.c_void_p), ("dq_gsa", C.c_void_p), ("dk_gsa", C.c_void_p),
        ("dv_out", C.c_void_p), ("ds", C.c_void_p), ("dg", C.c_void_p),
        ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p), ("df", C.c_void_p),
        ("inv_freq", C.c_void_p), ("cu_seqlens", C.c_void_p),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("HQ", C.c_int32), ("H", C.c_int32),
        ("K", C.c_int32), ("V", C.c_int32), ("M", C.c_int32),
        ("feature_map", C.c_int32), ("seqlen_offset", C.c_int32), ("dtype", C.c_int32),
        ("gate_logit_normalizer", C.c_float), ("stream", C.c_void_p),
    ]


class NhaLayerEpilogueBwdArgs(C.Structure):
    _fields_ = [
        ("o", C.c_void_p), ("dy", C.c_void_p), ("dout", C.c_void_p), ("weight", C.c_void_p),
        ("dweight_partial", C.c_void_p), ("dbias_partial", C.c_void_p),
        ("rows", C.c_int32), ("dim", C.c_int32), ("dtype", C.c_int32), ("eps", C.c_float), ("stream", C.c_void_p),
    ]


class NhaShortConvArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("weight", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p), ("cu_seqlens", C.c_void_p),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("C", C.c_int32), ("KS", C.c_int32),
        ("activation", C.c_int32), ("dtype", C.c_int32), ("stream", C.c_void_p),
    ]


class NhaShortConvBwdArgs(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("weight", C.c_void_p), ("bias", C.c_void_p), ("dy", C.c_void_p), ("dx", C.c_void_p),
        ("dweight_partial", C.c_void_p), ("dbias_partial", C.c_void_p), ("cu_seqlens", C.c_void_p),
        ("T_tot", C.c_int32), ("N", C.c_int32), ("C", C.c_int32), ("KS", C.c_int32),
        ("activation", C.c_int32), ("dtype", C.c_int32), ("stream", C.c_void_p),
    ]


class NhaError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"libnha_hip error {code}: {msg}")
        self.code = code


_lib = None


def load() -> C.CDLL:
    """Load libnha_hip.so once; raises if it has not been built (python -m nha_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m nha_amd.build` "
                           "(the NHA ops have no CPU or eager fallback)")
    lib = C.CDLL(LIB_PATH)
    lib.nha_prefill_scratch_bytes.restype = C.c_size_t
    lib.nha_prefill_scratch_bytes.argtypes = [C.POINTER(NhaPrefillArgs)]
    lib.nha_prefill_fwd.restype = C.c_int
    lib.nha_prefill_fwd.argtypes = [C.POINTER(NhaPrefillArgs)]
    lib.nha_prefill_fwd_noalloc.restype = C.c_int
    lib.nha_prefill_fwd_noalloc.argtypes = [C.POINTER(NhaPrefillArgs)]
    lib.nha_prefill_bwd_scratch_bytes.restype = C.c_size_t
    lib.nha_prefill_bwd_scratch_bytes.argtypes = [C.POINTER(NhaPrefillBwdArgs)]
    lib.nha_prefill_bwd.restype = C.c_int
    lib.nha_prefill_bwd.argtypes = [C.POINTER(NhaPrefillBwdArgs)]
    lib.nha_decode_step.restype = C.c_int
    lib.nha_decode_step.argtypes = [C.POINTER(NhaDecodeArgs)]
    lib.nha_decode_advance.restype = C.c_int
    lib.nha_decode_advance.argtypes = [C.c_void_p, C.c_int32, C.c_void_p]
    lib.nha_layer_prologue.restype = C.c_int
    lib.nha_layer_prologue.argtypes = [C.POINTER(NhaLayerPrologueArgs)]
    lib.nha_layer_epilogue.restype = C.c_int
    lib.nha_layer_epilogue.argtypes = [C.POINTER(NhaLayerEpilogueArgs)]
    lib.nha_layer_prologue_bwd.restype = C.c_int
    lib.nha_layer_prologue_bwd.argtypes = [C.POINTER(NhaLayerPrologueBwdArgs)]
    lib.nha_layer_epilogue_bwd.restype = C.c_int
    lib.nha_layer_epilogue_bwd.argtypes = [C.POINTER(NhaLayerEpilogueBwdArgs)]
    lib.nha_layer_epilogue_bwd_parts.restype = C.c_int32
    lib.nha_layer_epilogue_bwd_parts.argtypes = [C.c_int32]
    lib.nha_hybrid_prologue.restype = C.c_int
    lib.nha_hybrid_prologue.argtypes = [C.POINTER(NhaHybridPrologueArgs)]
    lib.nha_zero_sink_rescale.restype = C.c_int
    lib.nha_zero_sink_rescale.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int32] * 7 + [C.c_void_p]
    lib.nha_sink_window_scratch_bytes.restype = C.c_size_t
    lib.nha_sink_window_scratch_bytes.argtypes = [C.POINTER(NhaSinkWindowArgs)]
    lib.nha_sink_window_fwd.restype = C.c_int
    lib.nha_sink_window_fwd.argtypes = [C.POINTER(NhaSinkWindowArgs)]
    lib.nha_short_conv.restype = C.c_int
    lib.nha_short_conv.argtypes = [C.POINTER(NhaShortConvArgs)]
    lib.nha_short_conv_bwd.restype = C.c_int
    lib.nha_short_conv_bwd.argtypes = [C.POINTER(NhaShortConvBwdArgs)]
    lib.nha_short_conv_bwd_parts.restype = C.c_int32
    lib.nha_short_conv_bwd_parts.argtypes = [C.c_int32]
    lib.nha_varlen_num_chunks.restype = C.c_int32
    lib.nha_varlen_num_chunks.argtypes = [C.c_void_p, C.c_int32, C.c_int32]
    lib.nha_varlen_indices.restype = C.c_int
    lib.nha_varlen_indices.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.nha_last_error.restype = C.c_char_p
    lib.nha_last_error.argtypes = []
    lib.nha_abi_version.restype = C.c_int
    lib.nha_abi_version.argtypes = []
    if lib.nha_abi_version() != ABI_VERSION:
        raise RuntimeError(f"libnha_hip.so ABI {lib.nha_abi_version()} != binding {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != NHA_OK:
        raise NhaError(rc, load().nha_last_error().decode("utf-8", "replace"))
