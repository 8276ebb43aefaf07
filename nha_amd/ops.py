"""Host-side mirror of the reference op API for the NHA hot path, bound to libnha_hip.so.

Same names, argument meaning, return tuples and error behaviour as
  nha_fla/ops/nha/chunk.py:568-690            chunk_nha
  nha_fla/ops/nha/chunk_fused.py:291-380      fused_chunk_nha_prefill
  nha_fla/ops/nha/fused_recurrent.py:431-584  fused_recurrent_nha_decode
  nha_fla/ops/nha/fused_recurrent.py:588-682  fused_recurrent_nha
Differences, all widening: k/v/s/g may carry fewer (kv) heads than q in chunk_nha (the reference
needs them pre-expanded); window and head-dim limits of the fused prefill are lifted.  chunk_nha
is differentiable (nha_prefill_bwd behind nha_fla/ops/nha/chunk.py:490-564); the inference ops
reject inputs that require grad, as the reference's do.
PyTorch is used for device memory and the current stream only; every tensor op on the hot path
is a HIP kernel behind the C ABI.  There is no CPU / eager fallback.
"""
from __future__ import annotations

import ctypes as C
import weakref
from typing import Optional, Tuple

import numpy as np
import torch

from . import _lib
from .varlen import CHUNK, chunk_tables

__all__ = ["chunk_nha", "fused_chunk_nha_prefill", "fused_recurrent_nha", "fused_recurrent_nha_decode",
           "prefill_tables", "nha_prefill", "nha_prefill_bwd", "nha_layer_prologue", "nha_layer_epilogue"]

_DT = {torch.float32: _lib.NHA_DTYPE_F32, torch.bfloat16: _lib.NHA_DTYPE_BF16}
_IMPL = {None: _lib.NHA_IMPL_AUTO, "auto": _lib.NHA_IMPL_AUTO, "simple": _lib.NHA_IMPL_SIMPLE,
         "mfma": _lib.NHA_IMPL_MFMA}


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(dev) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise TypeError(f"NHA HIP kernels take bfloat16 or float32 tensors, got {t.dtype}")
    return _DT[t.dtype]


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("NHA ops run on the GPU only (tensor on %s); there is no CPU fallback" % t.device)


# ---------------------------------------------------------------------------------------------
# varlen tables, cached per cu_seqlens content
# ---------------------------------------------------------------------------------------------
_TABLE_CACHE: dict = {}


def prefill_tables(cu_host: np.ndarray, device) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]:
    """(cu_seqlens, chunk_indices [NT,2], chunk_offsets [N+1]) as int32 device tensors + NT."""
    key = (cu_host.tobytes(), str(device))
    hit = _TABLE_CACHE.get(key)
    if hit is not None:
        return hit
    idx, off = chunk_tables(cu_host, CHUNK)
    out = (torch.from_numpy(cu_host.astype(np.int32)).to(device), torch.from_numpy(idx).to(device),
           torch.from_numpy(off).to(device), int(idx.shape[0]))
    if len(_TABLE_CACHE) > 64:
        _TABLE_CACHE.pop(next(iter(_TABLE_CACHE)))      # oldest entry
    _TABLE_CACHE[key] = out
    return out


# ---------------------------------------------------------------------------------------------
# forward workspace: one buffer per (device, stream), grown when a call needs more.  Calls on one
# stream are ordered by the stream, so they can share it; another stream gets its own.
# ---------------------------------------------------------------------------------------------
_WORKSPACE: dict = {}
_WORKSPACE_MAX_STREAMS = 16      # entries kept; the one used longest ago leaves first (streams come and go)


def _workspace(nbytes: int, dev, stream: int) -> torch.Tensor:
    key = (str(dev), stream)
    ws = _WORKSPACE.pop(key, None)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
    _WORKSPACE[key] = ws             # re-inserted: the dict's order is the order of last use
    while len(_WORKSPACE) > _WORKSPACE_MAX_STREAMS:
        _WORKSPACE.pop(next(iter(_WORKSPACE)))
    return ws


def release_workspaces() -> int:
    """Drop the cached prefill workspaces (forward and backward) of every device and stream and return
    the bytes they held.  The buffers are grow-only: one large prefill otherwise keeps its scratch for the life of the
    process, out of reach of `torch.cuda.empty_cache()`.  Work already queued keeps its buffer alive through the
    caching allocator's stream ordering, so this is safe to call between steps."""
    held = sum(ws.numel() for ws in _WORKSPACE.values())
    _WORKSPACE.clear()
    return held


# host copies of cu_seqlens tensors, keyed by the tensor OBJECT (weakly) and its version counter, so that
# the layers of a model, which all receive the same tensor, wait for one device-to-host copy, not one each
_CU_HOST: dict = {}      # id(tensor) -> (weak reference, version, host copy)


def _cu_to_host(cu: torch.Tensor) -> np.ndarray:
    if not cu.is_cuda:
        return cu.detach().to(torch.int32).numpy()
    key = id(cu)
    hit = _CU_HOST.get(key)
    if hit is not None and hit[0]() is cu and hit[1] == cu._version:
        return hit[2]
    host = cu.detach().to("cpu", torch.int32).numpy()
    _CU_HOST[key] = (weakref.ref(cu, lambda _, k=key: _CU_HOST.pop(k, None)), cu._version, host)
    return host


def nha_prefill(q_swa, k_swa, q_gsa, k_gsa, v, s, g, cu_host: np.ndarray, *, wl: int, shift: int, scale: float,
                h0=None, want_state: bool = False, want_lse: bool = True, impl=None):
    """Packed prefill on token-major tensors ``[T_tot, heads, dim]`` (one nha_prefill_fwd call).
    Returns (o, lse_swa, lse_gsa, hkt, hvt)."""
    lib = _lib.load()
    T_tot, HQ, K = q_swa.shape
    H, V, M = k_swa.shape[1], v.shape[-1], s.shape[-1]
    dev = q_swa.device
    N = cu_host.size - 1
    cu_d, idx_d, off_d, NT = prefill_tables(cu_host, dev)
    o = torch.empty(T_tot, HQ, V, dtype=q_swa.dtype, device=dev)
    lse_swa = torch.empty(T_tot, HQ, dtype=torch.float32, device=dev) if want_lse else None
    lse_gsa = torch.empty(T_tot, HQ, dtype=torch.float32, device=dev) if want_lse else None
    hkt = torch.empty(N, H, K, M, dtype=torch.float32, device=dev) if want_state else None
    hvt = torch.empty(N, H, M, V, dtype=torch.float32, device=dev) if want_state else None
    h0k = h0v = None
    if h0 is not None and h0[0] is not None:
        h0k = h0[0].to(torch.float32).contiguous()
        h0v = h0[1].to(torch.float32).contiguous()
        if tuple(h0k.shape) != (N, H, K, M) or tuple(h0v.shape) != (N, H, M, V):
            raise ValueError(f"initial_state must be ([{N},{H},{K},{M}], [{N},{H},{M},{V}]) (kv-head count), "
                             f"got {tuple(h0k.shape)} / {tuple(h0v.shape)}")
    a = _lib.NhaPrefillArgs()
    a.q_swa, a.k_swa, a.q_gsa, a.k_gsa = _ptr(q_swa), _ptr(k_swa), _ptr(q_gsa), _ptr(k_gsa)
    a.v, a.s, a.g, a.o = _ptr(v), _ptr(s), _ptr(g), _ptr(o)
    a.lse_swa, a.lse_gsa = _ptr(lse_swa), _ptr(lse_gsa)
    a.h0k, a.h0v, a.hkt, a.hvt = _ptr(h0k), _ptr(h0v), _ptr(hkt), _ptr(hvt)
    a.cu_seqlens, a.chunk_indices, a.chunk_offsets = _ptr(cu_d), _ptr(idx_d), _ptr(off_d)
    a.T_tot, a.N, a.NT, a.HQ, a.H, a.K, a.V, a.M = T_tot, N, NT, HQ, H, K, V, M
    a.wl, a.shift = int(wl), int(shift)
    a.dtype = _dtype_code(q_swa)
    a.impl = _IMPL[impl]
    a.scale = float(scale)
    a.stream = _stream(dev)
    nbytes = lib.nha_prefill_scratch_bytes(C.byref(a))
    if nbytes == 0:
        _lib.check(_lib.NHA_ERR_INVALID)
    scratch = _workspace(nbytes, dev, a.stream or 0)
    a.scratch, a.scratch_bytes = _ptr(scratch), scratch.numel()
    _lib.check(lib.nha_prefill_fwd(C.byref(a)))
    return o, lse_swa, lse_gsa, hkt, hvt


def nha_prefill_bwd(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, dout, cu_host: np.ndarray, *,
                    wl: int, shift: int, scale: float, h0=None, dlse_swa=None, dlse_gsa=None, dht=None,
                    want_dh0: bool = False):
    """Packed prefill backward on token-major tensors (one nha_prefill_bwd call).  Returns
    (dq_swa, dk_swa, dq_gsa, dk_gsa, dv, ds, dg, dh0k, dh0v) -- the last two None unless wanted."""
    lib = _lib.load()
    T_tot, HQ, K = q_swa.shape
    H, V, M = k_swa.shape[1], v.shape[-1], s.shape[-1]
    dev = q_swa.device
    N = cu_host.size - 1
    cu_d, idx_d, off_d, NT = prefill_tables(cu_host, dev)
    f32 = lambda x: None if x is None else x.to(torch.float32).contiguous()
    h0k, h0v = (None, None) if h0 is None or h0[0] is None else (f32(h0[0]), f32(h0[1]))
    dhkt, dhvt = (None, None) if dht is None else dht
    if (dhkt is None) != (dhvt is None):      # one final state unused downstream: its cotangent is zero
        dhkt = torch.zeros(N, H, K, M, dtype=torch.float32, device=dev) if dhkt is None else dhkt
        dhvt = torch.zeros(N, H, M, V, dtype=torch.float32, device=dev) if dhvt is None else dhvt
    dhkt, dhvt, dlse_swa, dlse_gsa = f32(dhkt), f32(dhvt), f32(dlse_swa), f32(dlse_gsa)
    dout = dout.to(q_swa.dtype).contiguous()
    outs = [torch.empty_like(x) for x in (q_swa, k_swa, q_gsa, k_gsa, v, s, g)]
    dh0k = torch.empty(N, H, K, M, dtype=torch.float32, device=dev) if want_dh0 else None
    dh0v = torch.empty(N, H, M, V, dtype=torch.float32, device=dev) if want_dh0 else None
    a = _lib.NhaPrefillBwdArgs()
    a.q_swa, a.k_swa, a.q_gsa, a.k_gsa = _ptr(q_swa), _ptr(k_swa), _ptr(q_gsa), _ptr(k_gsa)
    a.v, a.s, a.g = _ptr(v), _ptr(s), _ptr(g)
    a.o, a.lse_swa, a.lse_gsa = _ptr(o), _ptr(lse_swa), _ptr(lse_gsa)
    a.h0k, a.h0v = _ptr(h0k), _ptr(h0v)
    a.dout, a.dlse_swa, a.dlse_gsa, a.dhkt, a.dhvt = _ptr(dout), _ptr(dlse_swa), _ptr(dlse_gsa), _ptr(dhkt), _ptr(dhvt)
    a.dq_swa, a.dk_swa, a.dq_gsa, a.dk_gsa, a.dv, a.ds, a.dg = [_ptr(x) for x in outs]
    a.dh0k, a.dh0v = _ptr(dh0k), _ptr(dh0v)
    a.cu_seqlens, a.chunk_indices, a.chunk_offsets = _ptr(cu_d), _ptr(idx_d), _ptr(off_d)
    a.T_tot, a.N, a.NT, a.HQ, a.H, a.K, a.V, a.M = T_tot, N, NT, HQ, H, K, V, M
    a.wl, a.shift = int(wl), int(shift)
    a.dtype = _dtype_code(q_swa)
    a.scale = float(scale)
    a.stream = _stream(dev)
    nbytes = lib.nha_prefill_bwd_scratch_bytes(C.byref(a))
    if nbytes == 0:
        _lib.check(_lib.NHA_ERR_INVALID)
    scratch = _workspace(nbytes, dev, a.stream or 0)     # shared with the forward: calls on one stream are ordered
    a.scratch, a.scratch_bytes = _ptr(scratch), nbytes
    _lib.check(lib.nha_prefill_bwd(C.byref(a)))
    return (*outs, dh0k, dh0v)


_FMAP = {None: _lib.NHA_FMAP_NONE, "none": _lib.NHA_FMAP_NONE, "swish": _lib.NHA_FMAP_SWISH, "relu": _lib.NHA_FMAP_RELU}


def _prologue_dims(q, k, v, f, inv_freq, cu):
    B, T, HQ, K = q.shape
    H, V, M = k.shape[2], v.shape[3], f.shape[3]
    if cu is not None and B != 1:
        raise ValueError("cu_seqlens needs the packed layout [1, T_tot, ...]")
    for x in (k, v, f):
        if x.dtype != q.dtype:
            raise TypeError("q, k, v, f must share one dtype")
    if inv_freq.numel() != K // 2:
        raise ValueError(f"inv_freq must hold K/2 = {K // 2} entries, got {inv_freq.numel()}")
    return dict(T_tot=B * T, N=(cu.numel() - 1) if cu is not None else B, HQ=HQ, H=H, K=K, V=V, M=M)


def _prologue_fwd(q, k, v, f, inv_freq, fm: int, normalizer: float, offset: int, cu):
    lib = _lib.load()
    dims = _prologue_dims(q, k, v, f, inv_freq, cu)
    q_swa, k_swa, v_out = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    s, g = torch.empty_like(f), torch.empty_like(f)
    q_gsa = torch.empty_like(q) if fm else None
    k_gsa = torch.empty_like(k) if fm else None
    a = _lib.NhaLayerPrologueArgs(
        q=_ptr(q), k=_ptr(k), v=_ptr(v), f=_ptr(f), q_swa=_ptr(q_swa), k_swa=_ptr(k_swa), q_gsa=_ptr(q_gsa),
        k_gsa=_ptr(k_gsa), v_out=_ptr(v_out), s=_ptr(s), g=_ptr(g), inv_freq=_ptr(inv_freq), cu_seqlens=_ptr(cu),
        feature_map=fm, seqlen_offset=int(offset), dtype=_dtype_code(q), gate_logit_normalizer=float(normalizer),
        stream=_stream(q.device), **dims)
    _lib.check(lib.nha_layer_prologue(C.byref(a)))
    return q_swa, k_swa, q_gsa, k_gsa, v_out, s, g


def _prologue_bwd(q, k, v, f, inv_freq, fm: int, normalizer: float, offset: int, cu, dq_swa, dk_swa, dq_gsa, dk_gsa,
                  dv_out, ds, dg):
    lib = _lib.load()
    dims = _prologue_dims(q, k, v, f, inv_freq, cu)
    dq, dk, dv, df = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(f)
    a = _lib.NhaLayerPrologueBwdArgs(
        q=_ptr(q), k=_ptr(k), v=_ptr(v), f=_ptr(f), dq_swa=_ptr(dq_swa), dk_swa=_ptr(dk_swa), dq_gsa=_ptr(dq_gsa),
        dk_gsa=_ptr(dk_gsa), dv_out=_ptr(dv_out), ds=_ptr(ds), dg=_ptr(dg), dq=_ptr(dq), dk=_ptr(dk), dv=_ptr(dv),
        df=_ptr(df), inv_freq=_ptr(inv_freq), cu_seqlens=_ptr(cu), feature_map=fm, seqlen_offset=int(offset),
        dtype=_dtype_code(q), gate_logit_normalizer=float(normalizer), stream=_stream(q.device), **dims)
    _lib.check(lib.nha_layer_prologue_bwd(C.byref(a)))
    return dq, dk, dv, df


class _LayerPrologueFunction(torch.autograd.Function):
    """Autograd node of the fused prologue: both directions are one HIP launch."""

    @staticmethod
    def forward(ctx, q, k, v, f, inv_freq, fm, normalizer, offset, cu):
        outs = _prologue_fwd(q, k, v, f, inv_freq, fm, normalizer, offset, cu)
        ctx.save_for_backward(q, k, v, f, inv_freq)
        ctx.cu, ctx.meta = cu, (fm, normalizer, offset)
        return outs if fm else (outs[0], outs[1], outs[4], outs[5], outs[6])

    @staticmethod
    def backward(ctx, *grads):
        q, k, v, f, inv_freq = ctx.saved_tensors
        fm, normalizer, offset = ctx.meta
        shapes = (q, k, q, k, v, f, f) if fm else (q, k, v, f, f)
        grads = [torch.zeros_like(x) if gr is None else gr.contiguous() for gr, x in zip(grads, shapes)]
        if fm:
            dq_swa, dk_swa, dq_gsa, dk_gsa, dv_out, ds, dg = grads
        else:
            (dq_swa, dk_swa, dv_out, ds, dg), dq_gsa, dk_gsa = grads, None, None
        dq, dk, dv, df = _prologue_bwd(q, k, v, f, inv_freq, fm, normalizer, offset, ctx.cu, dq_swa, dk_swa, dq_gsa,
                                       dk_gsa, dv_out, ds, dg)
        return dq, dk, dv, df, None, None, None, None, None


def nha_layer_prologue(q, k, v, f, inv_freq, *, feature_map: Optional[str], gate_logit_normalizer: float,
                       seqlen_offset: int = 0, cu_seqlens: Optional[torch.Tensor] = None):
    """One launch for the elementwise chain of nha_fla/layers/nha.py:214-237 on the raw projections
    q [B,T,HQ,K], k [B,T,H,K], v [B,T,H,V], f [B,T,H,M] (B = 1 with cu_seqlens, an int32 device
    tensor).  Returns (q_swa, k_swa, q_gsa, k_gsa, v, s, g); without a feature map q_gsa / k_gsa
    are q / k themselves.  Differentiable with respect to q, k, v, f (one launch backward too)."""
    _need_cuda(q, k, v, f, inv_freq, cu_seqlens)
    if feature_map not in _FMAP:
        raise NotImplementedError(f"Feature map `{feature_map}` has no fused prologue.")
    _dtype_code(q)
    q, k, v, f = (x.contiguous() for x in (q, k, v, f))
    inv_freq = inv_freq.detach().to(torch.float32).contiguous()
    fm = _FMAP[feature_map]
    cu = None if cu_seqlens is None else cu_seqlens.to(device=q.device, dtype=torch.int32).contiguous()
    args = (q, k, v, f, inv_freq, fm, float(gate_logit_normalizer), int(seqlen_offset), cu)
    if torch.is_grad_enabled() and any(x.requires_grad for x in (q, k, v, f)):
        outs = _LayerPrologueFunction.apply(*args)
        if fm:
            return outs
        return outs[0], outs[1], q, k, outs[2], outs[3], outs[4]
    q_swa, k_swa, q_gsa, k_gsa, v_out, s, g = _prologue_fwd(*args)
    return q_swa, k_swa, (q_gsa if fm else q), (k_gsa if fm else k), v_out, s, g


def _epilogue_fwd(o, w, b, eps: float):
    lib = _lib.load()
    dim = o.shape[-1]
    y = torch.empty_like(o)
    a = _lib.NhaLayerEpilogueArgs(o=_ptr(o), y=_ptr(y), weight=_ptr(w), bias=_ptr(b), rows=o.numel() // dim, dim=dim,
                                  dtype=_dtype_code(o), eps=float(eps), stream=_stream(o.device))
    _lib.check(lib.nha_layer_epilogue(C.byref(a)))
    return y


class _LayerEpilogueFunction(torch.autograd.Function):
    """Autograd node of the fused epilogue; the weight / bias gradients are reduced from the
    kernel's per-workgroup partial sums in a fixed order."""

    @staticmethod
    def forward(ctx, o, weight, bias, eps):
        w = None if weight is None else weight.detach().to(torch.float32).contiguous()
        b = None if bias is None else bias.detach().to(torch.float32).contiguous()
        ctx.save_for_backward(o, w)
        ctx.eps = eps
        ctx.wb = (None if weight is None else weight.dtype, None if bias is None else bias.dtype)
        return _epilogue_fwd(o, w, b, eps)

    @staticmethod
    def backward(ctx, dy):
        lib = _lib.load()
        o, w = ctx.saved_tensors
        dy = dy.contiguous()
        dim = o.shape[-1]
        rows = o.numel() // dim
        parts = lib.nha_layer_epilogue_bwd_parts(rows)
        wdt, bdt = ctx.wb
        need_w = wdt is not None and ctx.needs_input_grad[1]
        need_b = bdt is not None and ctx.needs_input_grad[2]
        dwp = torch.empty(parts, dim, dtype=torch.float32, device=o.device) if need_w else None
        dbp = torch.empty(parts, dim, dtype=torch.float32, device=o.device) if need_b else None
        do = torch.empty_like(o)
        a = _lib.NhaLayerEpilogueBwdArgs(o=_ptr(o), dy=_ptr(dy), dout=_ptr(do), weight=_ptr(w), dweight_partial=_ptr(dwp),
                                         dbias_partial=_ptr(dbp), rows=rows, dim=dim, dtype=_dtype_code(o),
                                         eps=float(ctx.eps), stream=_stream(o.device))
        _lib.check(lib.nha_layer_epilogue_bwd(C.byref(a)))
        return (do, dwp.sum(0).to(wdt) if need_w else None, dbp.sum(0).to(bdt) if need_b else None, None)


def nha_layer_epilogue(o, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float):
    """rms_norm(silu(o)) * weight (+ bias) over the last dimension in one launch: the normalisation
    half of nha_fla/layers/nha.py:278.  Differentiable with respect to o, weight and bias (last
    dimension a multiple of 8 and at most 8192 for the backward)."""
    _need_cuda(o, weight, bias)
    _dtype_code(o)
    o = o.contiguous()
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (o, weight, bias)):
        dim = o.shape[-1]
        if dim % 8 or dim > 8192:
            raise NotImplementedError(f"nha_layer_epilogue backward needs a last dimension % 8 == 0 and <= 8192, got {dim}")
        return _LayerEpilogueFunction.apply(o, weight, bias, float(eps))
    w = None if weight is None else weight.detach().to(torch.float32).contiguous()
    b = None if bias is None else bias.detach().to(torch.float32).contiguous()
    return _epilogue_fwd(o, w, b, float(eps))


def _short_conv_args(x, cu):
    T_tot = x.shape[0] * x.shape[1]
    N = (cu.numel() - 1) if cu is not None else x.shape[0]
    return T_tot, N


class _ShortConvFunction(torch.autograd.Function):
    """Autograd node of the short convolution: one launch per direction; the weight / bias gradients are
    reduced from the kernel's per-run partial sums in a fixed order."""

    @staticmethod
    def forward(ctx, x, weight, bias, cu, act):
        lib = _lib.load()
        Cn, KS = weight.shape[0], weight.shape[-1]
        w = weight.detach().to(x.dtype).reshape(Cn, KS).contiguous()
        b = None if bias is None else bias.detach().to(x.dtype).contiguous()
        T_tot, N = _short_conv_args(x, cu)
        y = torch.empty_like(x)
        a = _lib.NhaShortConvArgs(x=_ptr(x), weight=_ptr(w), bias=_ptr(b), y=_ptr(y), cu_seqlens=_ptr(cu), T_tot=T_tot, N=N,
                                  C=Cn, KS=KS, activation=int(act), dtype=_dtype_code(x), stream=_stream(x.device))
        _lib.check(lib.nha_short_conv(C.byref(a)))
        ctx.save_for_backward(x, w, b, cu)
        ctx.act = int(act)
        ctx.wb = (weight.dtype, weight.shape, None if bias is None else bias.dtype)
        return y

    @staticmethod
    def backward(ctx, dy):
        lib = _lib.load()
        x, w, b, cu = ctx.saved_tensors
        dy = dy.contiguous()
        Cn, KS = w.shape
        T_tot, N = _short_conv_args(x, cu)
        parts = lib.nha_short_conv_bwd_parts(T_tot)
        wdt, wshape, bdt = ctx.wb
        need_w = ctx.needs_input_grad[1]
        need_b = bdt is not None and ctx.needs_input_grad[2]
        dwp = torch.empty(parts, Cn, KS, dtype=torch.float32, device=x.device) if need_w else None
        dbp = torch.empty(parts, Cn, dtype=torch.float32, device=x.device) if need_b else None
        dx = torch.empty_like(x)
        a = _lib.NhaShortConvBwdArgs(x=_ptr(x), weight=_ptr(w), bias=_ptr(b), dy=_ptr(dy), dx=_ptr(dx), dweight_partial=_ptr(dwp),
                                     dbias_partial=_ptr(dbp), cu_seqlens=_ptr(cu), T_tot=T_tot, N=N, C=Cn, KS=KS,
                                     activation=ctx.act, dtype=_dtype_code(x), stream=_stream(x.device))
        _lib.check(lib.nha_short_conv_bwd(C.byref(a)))
        return (dx, dwp.sum(0).to(wdt).reshape(wshape) if need_w else None, dbp.sum(0).to(bdt) if need_b else None, None, None)


def short_conv_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether nha_short_conv serves this call: GPU tensors in bf16 / fp32, 2 to 4 taps, channels a multiple of 8."""
    return (x.is_cuda and x.dtype in (torch.bfloat16, torch.float32) and 2 <= weight.shape[-1] <= 4
            and weight.shape[0] % 8 == 0)


def nha_short_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], *,
                   cu_seqlens: Optional[torch.Tensor] = None, activation: Optional[str] = "silu") -> torch.Tensor:
    """Depthwise causal convolution over ``x [B, T, C]`` with ``weight [C, 1, KS]`` (+ ``bias [C]``) and optional
    SiLU in one launch, restarting at ``cu_seqlens`` boundaries (then ``B == 1``): what the layer's
    ``ShortConvolution`` modules compute on a fresh sequence (nha_fla/layers/nha.py:186-206).  Differentiable with
    respect to x, weight and bias."""
    _need_cuda(x, weight, bias)
    if activation not in (None, "silu", "swish"):
        raise ValueError(f"activation must be None, 'silu' or 'swish', got {activation!r}")
    if x.dim() != 3:
        raise ValueError(f"x must be [batch, tokens, channels], got {tuple(x.shape)}")
    Cn = x.shape[-1]
    if weight.shape[0] != Cn or weight.numel() != Cn * weight.shape[-1]:
        raise ValueError(f"weight must be [{Cn}, 1, taps] for x with {Cn} channels, got {tuple(weight.shape)}")
    if bias is not None and bias.numel() != Cn:
        raise ValueError(f"bias must have {Cn} entries, got {tuple(bias.shape)}")
    if cu_seqlens is not None and x.shape[0] != 1:
        raise ValueError("cu_seqlens needs the packed layout [1, T_tot, C]")
    if cu_seqlens is not None:
        # the kernels walk the boundaries: they must start at 0, not decrease and end at the token count
        cu_host = _cu_to_host(cu_seqlens)
        if cu_host.ndim != 1 or cu_host.size < 2 or cu_host[0] != 0 or cu_host[-1] != x.shape[1] \
                or (np.diff(cu_host) < 0).any():
            raise ValueError(f"cu_seqlens must rise from 0 to the token count {x.shape[1]}, got {cu_host.tolist()[:8]}"
                             f"{'...' if cu_host.size > 8 else ''}")
    cu = None if cu_seqlens is None else cu_seqlens.to(device=x.device, dtype=torch.int32).contiguous()
    return _ShortConvFunction.apply(x.contiguous(), weight, bias, cu, 0 if activation is None else 1)


def hybrid_prologue_supported(q: torch.Tensor, D: int, M: int) -> bool:
    """Whether nha_hybrid_prologue serves these tensors: GPU, bf16 / fp32, head size 64 / 128 / 256, M a multiple of 8."""
    return q.is_cuda and q.dtype in (torch.bfloat16, torch.float32) and D in (64, 128, 256) and M % 8 == 0


def _row_view(x: torch.Tensor, width: int, what: str):
    """(tensor, elements between the rows of two tokens) of a `[B, T, width]` view whose rows are contiguous and
    whose tokens are evenly spaced (a column slice of a fused projection output, or a contiguous tensor)."""
    B, T = x.shape[0], x.shape[1]
    if x.dim() != 3 or x.shape[2] != width:
        raise ValueError(f"{what} must be [batch, tokens, {width}], got {tuple(x.shape)}")
    if (width > 1 and x.stride(2) != 1) or (B > 1 and T > 1 and x.stride(0) != T * x.stride(1)):
        x = x.contiguous()
    stride = x.stride(1) if T > 1 else (x.stride(0) if B > 1 else width)
    esz = x.element_size()
    if (stride * esz) % 16 or x.data_ptr() % 16:
        x = x.contiguous()
        stride = width
    return x, stride


@torch.no_grad()
def nha_hybrid_prologue(q, k, v, f, cos, sin, *, num_heads: int, num_kv_heads: int, head_dim: int, num_slots: int,
                        q_weight=None, k_weight=None, eps: float = 1e-6, mask=None, gate_logit_normalizer: float = 8.0,
                        want_s: bool = True, positions=None, inv_freq=None):
    """One launch for the glue of a hybrid decoder attention block (inference): per-head RMSNorm of q and k (when
    weights are given), rotary embedding, the gates and the padding mask
    (nha_fla/models/qwen3_moe_nha/qwennha.py:103-144, :240-247).  q / k / v / f are `[B, T, heads * dim]` views
    (column slices of one fused projection output are read in place); cos / sin `[B or 1, T, D]`, or None with
    `positions [B, T]` (int64) and `inv_freq [D/2]` (fp32), from which the kernel forms the table rows itself; mask
    `[B, T]` or None; f None writes g = s = 0.  Returns contiguous q, sq `[B,T,HQ,D]`, k, sk, v `[B,T,H,D]`, g, s `[B,T,H,M]`
    (s None unless `want_s`)."""
    _need_cuda(q, k, v, cos, sin, positions, inv_freq)
    B, T = q.shape[0], q.shape[1]
    HQ, H, D, M = num_heads, num_kv_heads, head_dim, num_slots
    dt, dev = q.dtype, q.device
    if (cos is None) == (positions is None):
        raise ValueError("pass either cos and sin or positions and inv_freq")
    q, qs = _row_view(q, HQ * D, "q")
    k, ks = _row_view(k, H * D, "k")
    v, vs = _row_view(v, H * D, "v")
    fs = 0
    if f is not None:
        f, fs = _row_view(f, H * M, "f")
    cs_stride = 0
    if cos is not None:
        if cos.shape[-1] != D or cos.shape[-2] != T or cos.shape[0] not in (1, B) or sin.shape != cos.shape:
            raise ValueError(f"cos / sin must be [{B} or 1, {T}, {D}], got {tuple(cos.shape)} / {tuple(sin.shape)}")
        cos, sin = cos.to(dt).contiguous(), sin.to(dt).contiguous()
        cs_stride = T * D if cos.shape[0] == B and B > 1 else 0
    else:
        if tuple(positions.shape) != (B, T) or inv_freq.numel() != D // 2:
            raise ValueError(f"positions must be [{B}, {T}] and inv_freq [{D // 2}], got {tuple(positions.shape)} / "
                             f"{tuple(inv_freq.shape)}")
        positions = positions.to(torch.int64).contiguous()
        inv_freq = inv_freq.to(torch.float32).contiguous()
    for x in (k, v, f, q_weight, k_weight):
        if x is not None and x.dtype != dt:
            raise ValueError(f"every tensor must have the dtype of q ({dt}), got {x.dtype}")
    if mask is not None:
        mask = mask.reshape(B * T).to(dt).contiguous()
    new = lambda h, d: torch.empty(B, T, h, d, dtype=dt, device=dev)
    qo, sqo, ko, sko, vo, go = new(HQ, D), new(HQ, D), new(H, D), new(H, D), new(H, D), new(H, M)
    so = new(H, M) if want_s else None
    a = _lib.NhaHybridPrologueArgs(
        q=_ptr(q), k=_ptr(k), v=_ptr(v), f=_ptr(f), q_stride=qs, k_stride=ks, v_stride=vs, f_stride=fs,
        q_weight=_ptr(None if q_weight is None else q_weight.contiguous()),
        k_weight=_ptr(None if k_weight is None else k_weight.contiguous()), cos=_ptr(cos), sin=_ptr(sin),
        cs_batch_stride=cs_stride, positions=_ptr(positions), inv_freq=_ptr(inv_freq), mask=_ptr(mask), q_out=_ptr(qo), sq_out=_ptr(sqo),
        k_out=_ptr(ko), sk_out=_ptr(sko), v_out=_ptr(vo), g_out=_ptr(go), s_out=_ptr(so), B=B, T=T, HQ=HQ, H=H, D=D, M=M,
        dtype=_dtype_code(q), eps=float(eps), gate_logit_normalizer=float(gate_logit_normalizer), stream=_stream(dev))
    _lib.check(_lib.load().nha_hybrid_prologue(C.byref(a)))
    return qo, sqo, ko, sko, vo, go, so


def zero_sink_attention_supported(q: torch.Tensor, k: torch.Tensor) -> bool:
    """Whether nha_sink_window_fwd serves these tensors: GPU, bf16, head size 64 or 128, a multiple of four query heads
    per kv-head, tensors of one call below 4 GiB."""
    HQ, H, D = q.shape[-2], k.shape[-2], q.shape[-1]
    tokens = q.numel() // (HQ * D)
    return (q.is_cuda and q.dtype == torch.bfloat16 and D in (64, 128) and HQ % H == 0 and (HQ // H) % 4 == 0
            and tokens * H * D * 2 < (1 << 32) and tokens <= 65535 * CHUNK)


@torch.no_grad()
def zero_sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int, num_sinks: int,
                        scale: Optional[float] = None, cu_seqlens: Optional[torch.Tensor] = None,
                        output_lse: bool = False):
    """Sliding-window softmax attention preceded by `num_sinks` all-zero key / value rows per sequence: the "full
    attention" layers of the hybrid decoder models (nha_fla/models/qwen3_moe_nha/qwennha.py:323-336, :400-413).  q
    `[B,T,HQ,D]` and k, v `[B,T,H,D]` (rotated q / k; `[1,T_tot,...]` with cu_seqlens); query t of a sequence sees keys
    t - window < j <= t and clamp(window - 1 - t, 0, num_sinks) sinks of logit 0 and value 0.  One launch of the
    prefill's window loop.  Returns o `[B,T,HQ,D]` (and the log of the softmax denominator `[B,T,HQ]`)."""
    _need_cuda(q, k, v)
    if not zero_sink_attention_supported(q, k):
        raise _lib.NhaError(_lib.NHA_ERR_UNSUPPORTED, "zero_sink_attention: bf16, head size 64 / 128 and a multiple of four "
                                                       "query heads per kv-head are served")
    B, T, HQ, D = q.shape
    H = k.shape[2]
    if cu_seqlens is not None:
        if B != 1:
            raise ValueError("cu_seqlens needs the packed layout [1, T_tot, ...]")
        cu_host = _cu_to_host(cu_seqlens)
    else:
        cu_host = np.arange(0, (B + 1) * T, T, dtype=np.int32)
    if scale is None:
        scale = D ** -0.5
    dev = q.device
    q_, k_, v_ = (_flat(x) for x in (q, k, v))
    cu_d, idx_d, off_d, NT = prefill_tables(cu_host, dev)
    o = torch.empty(B * T, HQ, D, dtype=q.dtype, device=dev)
    lse = torch.empty(B * T, HQ, dtype=torch.float32, device=dev) if output_lse else None
    a = _lib.NhaSinkWindowArgs(q=_ptr(q_), k=_ptr(k_), v=_ptr(v_), o=_ptr(o), lse=_ptr(lse), cu_seqlens=_ptr(cu_d),
                               chunk_indices=_ptr(idx_d), chunk_offsets=_ptr(off_d), T_tot=B * T, N=cu_host.size - 1, NT=NT,
                               HQ=HQ, H=H, D=D, window=int(window), sinks=int(num_sinks), dtype=_dtype_code(q),
                               scale=float(scale), stream=_stream(dev))
    lib = _lib.load()
    nbytes = lib.nha_sink_window_scratch_bytes(C.byref(a))
    scratch = _workspace(nbytes, dev, a.stream or 0)
    a.scratch, a.scratch_bytes = _ptr(scratch), nbytes
    _lib.check(lib.nha_sink_window_fwd(C.byref(a)))
    o = o.view(B, T, HQ, D)
    return (o, lse.view(B, T, HQ)) if output_lse else o


@torch.no_grad()
def nha_zero_sink_rescale_(o: torch.Tensor, lse_swa: torch.Tensor, window: int, num_sinks: int) -> torch.Tensor:
    """In place: row (b, t, head) of ``o [B,T,HQ,D]`` times (e^lse + num_sinks) / (e^lse + clamp(window - 1 - t, 0,
    num_sinks)) -- takes the zero-logit sinks that the NHA kernel's zero slot states put into every softmax back out
    where the reference's window no longer covers them (nha_fla/models/qwen3_moe_nha/qwennha.py:323-336)."""
    _need_cuda(o, lse_swa)
    B, T, HQ, D = o.shape
    if not o.is_contiguous() or lse_swa.dtype != torch.float32 or not lse_swa.is_contiguous() or tuple(lse_swa.shape) != (B, T, HQ):
        raise ValueError("o must be contiguous [B,T,HQ,D] and lse_swa contiguous fp32 [B,T,HQ]")
    lib = _lib.load()
    _lib.check(lib.nha_zero_sink_rescale(_ptr(o), _ptr(lse_swa), B, T, HQ, D, int(window), int(num_sinks), _dtype_code(o),
                                         _stream(o.device)))
    return o


class _ChunkNHAFunction(torch.autograd.Function):
    """Autograd node of chunk_nha on packed tensors: same outputs and gradient set as
    ChunkNativeHybridAttentionFunction (nha_fla/ops/nha/chunk.py:364-564)."""

    @staticmethod
    def forward(ctx, q_swa, k_swa, q_gsa, k_gsa, v, s, g, h0k, h0v, cu_host, wl, shift, scale, want_state, impl):
        h0 = None if h0k is None else (h0k, h0v)
        o, lse_swa, lse_gsa, hkt, hvt = nha_prefill(q_swa, k_swa, q_gsa, k_gsa, v, s, g, cu_host, wl=wl, shift=shift,
                                                    scale=scale, h0=h0, want_state=want_state, impl=impl)
        ctx.save_for_backward(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, h0k, h0v)
        ctx.cu_host, ctx.wl, ctx.shift, ctx.scale = cu_host, wl, shift, scale
        ctx.set_materialize_grads(False)
        if not want_state:
            return o, lse_swa, lse_gsa, None, None
        return o, lse_swa, lse_gsa, hkt, hvt

    @staticmethod
    def backward(ctx, do, dlse_swa, dlse_gsa, dhkt, dhvt):
        q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, h0k, h0v = ctx.saved_tensors
        if do is None:
            do = torch.zeros_like(o)
        want_dh0 = h0k is not None and (ctx.needs_input_grad[7] or ctx.needs_input_grad[8])
        dht = None if dhkt is None and dhvt is None else (dhkt, dhvt)
        grads = nha_prefill_bwd(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, do, ctx.cu_host,
                                wl=ctx.wl, shift=ctx.shift, scale=ctx.scale,
                                h0=None if h0k is None else (h0k, h0v), dlse_swa=dlse_swa, dlse_gsa=dlse_gsa,
                                dht=dht, want_dh0=want_dh0)
        dh0k, dh0v = grads[7], grads[8]
        if dh0k is not None:
            dh0k, dh0v = dh0k.to(h0k.dtype), dh0v.to(h0v.dtype)
        return (*grads[:7], dh0k, dh0v, None, None, None, None, None, None)


def _flat(x):
    return x.reshape(x.shape[0] * x.shape[1], *x.shape[2:]).contiguous()


@torch.compiler.disable
def chunk_nha(
    q_swa: torch.Tensor,
    k_swa: torch.Tensor,
    q_gsa: torch.Tensor,
    k_gsa: torch.Tensor,
    v: torch.Tensor,
    s: torch.Tensor,
    g: torch.Tensor,
    cu_seqlens: Optional[torch.Tensor] = None,
    max_seqlen: Optional[int] = None,
    scale: Optional[float] = None,
    window_size_left: int = -1,
    window_size_right: int = -1,
    head_first: Optional[bool] = False,
    gsa_kv_shift: int = 0,
    initial_state: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    output_final_state: bool = False,
    impl: Optional[str] = None,
):
    r"""Chunk-level Native Hybrid Attention forward (nha_fla/ops/nha/chunk.py:568-690).

    q_swa/q_gsa ``[B,T,HQ,D]``; k_swa/k_gsa ``[B,T,H,D]``, v ``[B,T,H,V]``, s/g ``[B,T,H,M]`` with
    ``HQ % H == 0`` (the reference takes ``H == HQ``).  ``cu_seqlens`` ``[N+1]`` selects varlen
    packing (then ``B == 1``).  The SWA branch is causal: ``window_size_right`` is accepted and
    has no effect, as in the reference's ``causal=True`` flash-attn call (chunk.py:423-431).
    Returns ``(o [B,T,HQ,V], lse_swa [B,T,HQ], lse_gsa [B,T,HQ])`` plus ``(hkt [N,H,K,M],
    hvt [N,H,M,V])`` fp32 when ``output_final_state`` (chunk.py:688-690).
    """
    if head_first:
        raise DeprecationWarning(
            "head_first is deprecated and will be removed in a future version. "
            "Please use head_first=False for now instead.",
        )
    assert q_swa.dim() == 4, "Expected [B, T, H, D] for input"
    _need_cuda(q_swa, k_swa, q_gsa, k_gsa, v, s, g)
    if q_swa.dtype == torch.float16:
        # float16 tensors: computed in float32 (every float16 value is one) by the generic kernels, o returned in float16
        out = chunk_nha(*(x.float() for x in (q_swa, k_swa, q_gsa, k_gsa, v, s, g)), cu_seqlens=cu_seqlens, max_seqlen=max_seqlen,
                        scale=scale, window_size_left=window_size_left, window_size_right=window_size_right, head_first=head_first,
                        gsa_kv_shift=gsa_kv_shift, initial_state=initial_state, output_final_state=output_final_state, impl=impl)
        return (out[0].to(torch.float16), *out[1:])
    B, T, HQ, D = q_swa.shape
    H = k_swa.shape[2]
    if scale is None:
        scale = D ** -0.5
    if HQ % H:
        raise ValueError(f"query heads ({HQ}) must be a multiple of kv heads ({H})")
    for name, x, hh in (("q_gsa", q_gsa, HQ), ("k_gsa", k_gsa, H), ("v", v, H), ("s", s, H), ("g", g, H)):
        if x.shape[0] != B or x.shape[1] != T or x.shape[2] != hh:
            raise ValueError(f"{name} has shape {tuple(x.shape)}, expected [{B},{T},{hh},*]")
    if cu_seqlens is not None:
        if B != 1:
            raise ValueError("varlen (cu_seqlens) inputs must be packed with batch size 1")
        cu_host = _cu_to_host(cu_seqlens)
        if int(cu_host[-1]) != T:
            raise ValueError(f"cu_seqlens[-1] = {int(cu_host[-1])} does not match the packed length {T}")
    else:
        cu_host = np.arange(0, (B + 1) * T, T, dtype=np.int32)          # chunk.py:660
    dt = q_swa.dtype
    args = [_flat(x.to(dt)) for x in (q_swa, k_swa, q_gsa, k_gsa, v, s, g)]
    h0 = (None, None) if initial_state is None or initial_state[0] is None else tuple(initial_state)
    # empty sequences (a fully padded batch row after unpadding yields a repeated cu_seqlens entry): the
    # kernels see the packing without them; their final state is their initial state
    lens = np.diff(cu_host)
    if (lens < 0).any():
        raise ValueError("cu_seqlens must be non-decreasing")
    keep = None
    if (lens == 0).any():
        keep = torch.from_numpy(np.nonzero(lens > 0)[0]).to(q_swa.device)
        n_all = lens.size
        cu_host = np.concatenate([[0], np.cumsum(lens[lens > 0])]).astype(np.int32)
        h0_all = h0
        if h0[0] is not None:
            h0 = (h0[0][keep], h0[1][keep])
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (*args, *h0)):
        if impl is None:
            # the registered operator (nha_amd/custom_ops.py): schema, fake-tensor shapes and autograd formula
            o, lse_swa, lse_gsa, hkt, hvt = torch.ops.nha_amd.prefill_fwd(
                *args, torch.from_numpy(np.ascontiguousarray(cu_host, dtype=np.int32)), int(window_size_left),
                int(gsa_kv_shift), float(scale), h0[0], h0[1], bool(output_final_state))
        else:
            o, lse_swa, lse_gsa, hkt, hvt = _ChunkNHAFunction.apply(
                *args, h0[0], h0[1], cu_host, window_size_left, gsa_kv_shift, scale, output_final_state, impl)
    else:
        o, lse_swa, lse_gsa, hkt, hvt = nha_prefill(
            *args, cu_host, wl=window_size_left, shift=gsa_kv_shift, scale=scale,
            h0=None if h0[0] is None else h0, want_state=output_final_state, impl=impl)
    if keep is not None and output_final_state:
        def spread(part, init):
            full = torch.zeros(n_all, *part.shape[1:], dtype=part.dtype, device=part.device) if init is None \
                else init.to(part.dtype).clone()
            return full.index_copy(0, keep, part)
        hkt, hvt = spread(hkt, h0_all[0]), spread(hvt, h0_all[1])
    o = o.view(B, T, HQ, -1)
    lse_swa = lse_swa.view(B, T, HQ)
    lse_gsa = lse_gsa.view(B, T, HQ)
    if output_final_state:
        return o, lse_swa, lse_gsa, (hkt, hvt)
    return o, lse_swa, lse_gsa


@torch.no_grad()
def fused_chunk_nha_prefill(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    rotary_q: torch.Tensor,
    rotary_k: torch.Tensor,
    s: torch.Tensor,
    g: torch.Tensor,
    window_size: int,
    initial_state: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    output_final_state: bool = False,
    scale: Optional[float] = None,
    impl: Optional[str] = None,
) -> Tuple[torch.Tensor, Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]]:
    r"""Fused NHA prefill, inference only (nha_fla/ops/nha/chunk_fused.py:291-380): window covers
    raw tokens ``[t-W+1, t]``, the slots hold tokens ``<= t-W``.  q/rotary_q ``[B,T,HQ,K]``;
    k/rotary_k/v/s/g ``[B,T,H,*]``.  Returns ``(o [B,T,HQ,V], (hkt, hvt))`` (Nones unless
    ``output_final_state``).  The reference's limits ``W <= 64`` and power-of-two dims <= 128
    (:331-332) do not apply here."""
    B, T, HQ, K = q.shape
    H = k.shape[2]
    W = int(window_size)
    assert k.shape[1] == T and v.shape[1] == T and s.shape[1] == T and g.shape[1] == T
    assert rotary_q.shape == q.shape and rotary_k.shape == k.shape
    assert HQ % H == 0
    assert W >= 1
    _need_cuda(q, k, v, rotary_q, rotary_k, s, g)
    if q.dtype == torch.float16:   # computed in float32, o returned in float16
        o, st = fused_chunk_nha_prefill(*(x.float() for x in (q, k, v, rotary_q, rotary_k, s, g)), window_size=window_size,
                                        initial_state=initial_state, output_final_state=output_final_state, scale=scale, impl=impl)
        return o.to(torch.float16), st
    if initial_state is not None and initial_state[0] is not None:
        hk0, hv0 = initial_state
        assert tuple(hk0.shape) == (B, H, K, s.shape[-1]) and tuple(hv0.shape) == (B, H, s.shape[-1], v.shape[-1]), \
            f"initial_state must be at the kv-head count [B, {H}, ...], got {tuple(hk0.shape)} / {tuple(hv0.shape)}"
    else:
        initial_state = None
    if scale is None:
        scale = K ** -0.5
    cu_host = np.arange(0, (B + 1) * T, T, dtype=np.int32)
    dt = q.dtype
    args = [_flat(x.to(dt)) for x in (rotary_q, rotary_k, q, k, v, s, g)]
    o, _, _, hkt, hvt = nha_prefill(*args, cu_host, wl=W - 1, shift=W, scale=scale, h0=initial_state,
                                    want_state=output_final_state, want_lse=False, impl=impl)
    return o.view(B, T, HQ, -1), (hkt, hvt)


def _decode_state(initial_state, output_final_state, NG, B, H, K, V, M, dev):
    """State plumbing shared by the two T == 1 ops (fused_recurrent.py:169-179, :533-545)."""
    if initial_state is not None and initial_state != (None, None) and initial_state[0] is not None:
        hk0, hv0 = initial_state
        if hk0.dtype != torch.float32 or hv0.dtype != torch.float32:
            raise TypeError("the slot state must be float32")
        hk0, hv0 = hk0.contiguous(), hv0.contiguous()
        assert tuple(hk0.shape) == (B, H, K, M) and tuple(hv0.shape) == (B, H, M, V), \
            f"initial_state must be ([{B},{H},{K},{M}], [{B},{H},{M},{V}]), got {tuple(hk0.shape)} / {tuple(hv0.shape)}"
    else:
        hk0 = hv0 = None
    hkt = hvt = None
    if output_final_state:
        if NG == 1 and hk0 is not None:
            hkt, hvt = hk0, hv0                                          # in place, as the reference
        else:
            hkt = torch.empty(B, H, K, M, dtype=torch.float32, device=dev)
            hvt = torch.empty(B, H, M, V, dtype=torch.float32, device=dev)
    return hk0, hv0, hkt, hvt


def fused_recurrent_nha_decode(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    sw_k: torch.Tensor,
    sw_v: torch.Tensor,
    sq: Optional[torch.Tensor] = None,
    s: Optional[torch.Tensor] = None,
    cos: Optional[torch.Tensor] = None,
    sin: Optional[torch.Tensor] = None,
    initial_state: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    output_final_state: bool = False,
    scale: Optional[float] = None,
) -> Tuple[torch.Tensor, Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]]:
    r"""Single-token fused NHA decode step with GQA (nha_fla/ops/nha/fused_recurrent.py:431-584).

    q ``[B,1,HQ,K]`` raw; popped k/v/g ``[B,1,H,*]``; ``sw_k/sw_v [B,W,H,*]`` ascending in time;
    either ``sq`` (pre-rotated, with pre-rotated ``sw_k``) or ``cos/sin [B|1, W2>=W, K]``
    (in-kernel rotate-half on raw ``q``/``sw_k``; last W rows used, row W-1 = query position).
    Returns ``(o [B,1,HQ,V], (hkt, hvt))``; the state is updated in place when ``HQ == H``."""
    B, T, HQ, K = q.shape
    H = sw_k.shape[2]
    V = v.shape[-1]
    M = g.shape[-1]
    W = sw_k.shape[1]
    assert T == 1 and k.shape[1] == 1 and g.shape[1] == 1
    assert k.shape[2] == H and v.shape[2] == H and g.shape[2] == H, \
        f"popped-entry head count must match the kv-head count ({H}) of the window tensors"
    assert sw_v.shape[1] == W and sw_v.shape[2] == H
    assert HQ % H == 0
    assert K >= 16 and V >= 16
    _need_cuda(q, k, v, g, sw_k, sw_v, sq, s, cos, sin)
    if q.dtype == torch.float16:   # computed in float32, o returned in float16
        f = lambda x: None if x is None else x.float()
        o, st = fused_recurrent_nha_decode(f(q), f(k), f(v), f(g), f(sw_k), f(sw_v), sq=f(sq), s=f(s), cos=f(cos), sin=f(sin),
                                           initial_state=initial_state, output_final_state=output_final_state, scale=scale)
        return o.to(torch.float16), st
    NG = HQ // H
    if scale is None:
        scale = K ** -0.5
    dt = q.dtype
    rotary = cos is not None
    c_sb = c_sw = 0
    if rotary:
        assert sq is None, "pass either sq (pre-rotated) or cos/sin (in-kernel rotary), not both"
        assert sin is not None and cos.shape == sin.shape
        assert cos.shape[0] in (1, B) and cos.shape[1] >= W and cos.shape[2] == K, \
            f"rotary cos/sin must be [1|{B}, W2>={W}, K={K}], got {tuple(cos.shape)}"
        assert K % 2 == 0, "in-kernel rotate-half requires an even head dim"
        cos = cos[:, -W:].to(dt).contiguous()
        sin = sin[:, -W:].to(dt).contiguous()
        c_sb = cos.stride(0) if cos.shape[0] == B else 0
        c_sw = cos.stride(1)
    else:
        assert sq is not None and sq.shape == q.shape
    if s is not None:
        assert s.shape == g.shape
    dev = q.device
    cont = lambda x: None if x is None else x.to(dt).contiguous()
    q_, sq_, k_, v_, g_, s_, swk_, swv_ = map(cont, (q, sq, k, v, g, s, sw_k, sw_v))
    hk0, hv0, hkt, hvt = _decode_state(initial_state, output_final_state, NG, B, H, K, V, M, dev)
    o = torch.empty(B, 1, HQ, V, dtype=dt, device=dev)
    a = _lib.NhaDecodeArgs()
    a.mode, a.dtype = _lib.NHA_DECODE_WINDOW, _dtype_code(q_)
    a.B, a.HQ, a.H, a.K, a.V, a.M, a.W = B, HQ, H, K, V, M, W
    a.scale = float(scale)
    a.q, a.sq = _ptr(q_), _ptr(sq_)
    a.k_pop, a.v_pop, a.g_pop, a.s_pop = _ptr(k_), _ptr(v_), _ptr(g_), _ptr(s_)
    a.win_k, a.win_v = _ptr(swk_), _ptr(swv_)
    a.cos, a.sin, a.cos_sb, a.cos_sw = _ptr(cos), _ptr(sin), c_sb, c_sw
    a.hk_in, a.hv_in, a.hk_out, a.hv_out = _ptr(hk0), _ptr(hv0), _ptr(hkt), _ptr(hvt)
    a.o, a.stream = _ptr(o), _stream(dev)
    _lib.check(_lib.load().nha_decode_step(C.byref(a)))
    return o, (hkt, hvt)


@torch.compiler.disable
def fused_recurrent_nha(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    sliding_window: torch.Tensor,
    s: torch.Tensor,
    g: torch.Tensor,
    scale: Optional[float] = None,
    initial_state: Optional[Tuple[torch.Tensor]] = None,
    output_final_state: Optional[bool] = False,
) -> Tuple[torch.Tensor, torch.Tensor, list]:
    r"""Single-token NHA inference step with caller-supplied window logits
    (nha_fla/ops/nha/fused_recurrent.py:588-682).  q ``[B,1,HQ,K]``; k/v/s/g ``[B,1,H,*]``;
    ``sliding_window [B,1,HQ,W]`` logits.  Returns ``(o [B,1,HQ,V]`` slot part only,
    ``swa_score [B,1,HQ,W]`` fp32 window probabilities of the mixing softmax, ``[hkt, hvt])``."""
    T = q.shape[1]
    if T != 1:
        raise ValueError(
            f"fused_recurrent_nha is the single-token inference path and expects T == 1, got T = {T}."
        )
    assert not q.requires_grad, "fused_recurrent_nha is inference-only (no autograd)"
    _need_cuda(q, k, v, sliding_window, s, g)
    if q.dtype == torch.float16:   # computed in float32, o returned in float16
        o, p, st = fused_recurrent_nha(q.float(), k.float(), v.float(), sliding_window.float(), s.float(), g.float(), scale=scale,
                                       initial_state=initial_state, output_final_state=output_final_state)
        return o.to(torch.float16), p, st
    if scale is None:
        scale = k.shape[-1] ** -0.5
    B, _, HQ, K = q.shape
    H, V, M, W = k.shape[2], v.shape[-1], s.shape[-1], sliding_window.shape[-1]
    assert HQ % H == 0
    NG = HQ // H
    dt = q.dtype
    dev = q.device
    cont = lambda x: x.to(dt).contiguous()
    q_, k_, v_, sw_, s_, g_ = map(cont, (q, k, v, sliding_window, s, g))
    hk0, hv0, hkt, hvt = _decode_state(initial_state, output_final_state, NG, B, H, K, V, M, dev)
    o = torch.empty(B, 1, HQ, V, dtype=dt, device=dev)
    probs = torch.empty(B, 1, HQ, W, dtype=torch.float32, device=dev)
    a = _lib.NhaDecodeArgs()
    a.mode, a.dtype = _lib.NHA_DECODE_LOGITS, _dtype_code(q_)
    a.B, a.HQ, a.H, a.K, a.V, a.M, a.W = B, HQ, H, K, V, M, W
    a.scale = float(scale)
    a.q = _ptr(q_)
    a.k_pop, a.v_pop, a.g_pop, a.s_pop = _ptr(k_), _ptr(v_), _ptr(g_), _ptr(s_)
    a.win_logits, a.win_probs = _ptr(sw_), _ptr(probs)
    a.hk_in, a.hv_in, a.hk_out, a.hv_out = _ptr(hk0), _ptr(hv0), _ptr(hkt), _ptr(hvt)
    a.o, a.stream = _ptr(o), _stream(dev)
    _lib.check(_lib.load().nha_decode_step(C.byref(a)))
    return o, probs, [hkt, hvt]
