"""ctypes front of oracle/nha_ref_c.c (plain-C restatement of the prefill).  TEST INFRASTRUCTURE ONLY:
used by tests/ and by bench.py's cpu_baseline, never by the shipped package."""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional, Sequence

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(_HERE, "libnha_ref_c.so")
_lib = None


def build() -> str:
    """gcc -O3 -fopenmp through oracle/Makefile; returns the path of the shared object."""
    subprocess.run(["make", "-C", _HERE, "-B", "libnha_ref_c.so"], check=True, capture_output=True)
    return LIB


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
        _lib.nha_prefill_ref_c.restype = C.c_int
        _lib.nha_prefill_ref_c.argtypes = [C.c_void_p] * 8 + [C.c_int] * 8 + [C.c_double] + [C.c_void_p] * 7
    return _lib


def prefill_ref_c(q_swa, k_swa, q_gsa, k_gsa, v, s, g, *, window_size_left: int, gsa_kv_shift: int = 0,
                  cu_seqlens: Optional[Sequence[int]] = None, initial_state=None, scale: Optional[float] = None):
    """Same contract as oracle.nha_ref.prefill_ref, computed by the C restatement (float32 in and
    out, double arithmetic).  Returns (o, lse_swa, lse_gsa, hkt, hvt) as float32 tensors."""
    lib = load()
    B, T, HQ, K = q_swa.shape
    H, V, M = k_swa.shape[2], v.shape[-1], s.shape[-1]
    if scale is None:
        scale = K ** -0.5
    if cu_seqlens is None:
        cu = np.arange(0, (B + 1) * T, T, dtype=np.int32)
    else:
        assert B == 1, "varlen packing requires B == 1"
        cu = np.asarray([int(c) for c in cu_seqlens], dtype=np.int32)
    N = len(cu) - 1
    f32 = lambda x: np.ascontiguousarray(x.detach().to("cpu", torch.float32).numpy())
    a = [f32(x).reshape(B * T, *x.shape[2:]) for x in (q_swa, k_swa, q_gsa, k_gsa, v, s, g)]
    h0k = h0v = None
    if initial_state is not None:
        h0k, h0v = f32(initial_state[0]), f32(initial_state[1])
    o = np.empty((B * T, HQ, V), np.float32)
    ls = np.empty((B * T, HQ), np.float32)
    lg = np.empty((B * T, HQ), np.float32)
    hkt = np.empty((N, H, K, M), np.float32)
    hvt = np.empty((N, H, M, V), np.float32)
    ptr = lambda x: None if x is None else x.ctypes.data_as(C.c_void_p)
    rc = lib.nha_prefill_ref_c(*[ptr(x) for x in a], ptr(cu), N, HQ, H, K, V, M, int(window_size_left), int(gsa_kv_shift),
                               float(scale), ptr(h0k), ptr(h0v), ptr(o), ptr(ls), ptr(lg), ptr(hkt), ptr(hvt))
    if rc != 0:
        raise MemoryError("nha_prefill_ref_c ran out of memory")
    t = torch.from_numpy
    return t(o).reshape(B, T, HQ, V), t(ls).reshape(B, T, HQ), t(lg).reshape(B, T, HQ), t(hkt), t(hvt)
