"""The packed prefill and its backward as registered PyTorch operators (``torch.ops.nha_amd.*``).

``chunk_nha`` is the reference's entry point and keeps its decorator (``@torch.compiler.disable``,
nha_fla/ops/nha/chunk.py:567).  The two operators below give the same HIP calls a schema, a shape function
for fake / meta tensors and an autograd formula, so that code which calls them directly is traced by
``torch.compile`` / ``torch.export`` without a graph break and checked by ``torch.library.opcheck``:

    nha_amd::prefill_fwd(q_swa, k_swa, q_gsa, k_gsa, v, s, g, cu_seqlens, wl, shift, scale, h0k, h0v,
                         want_state) -> (o, lse_swa, lse_gsa, hkt, hvt)
    nha_amd::prefill_bwd(...)          -> (dq_swa, dk_swa, dq_gsa, dk_gsa, dv, ds, dg, dh0k, dh0v)

Tensors are token-major ``[T_tot, heads, dim]`` on the GPU; ``cu_seqlens`` is an int32 tensor ``[N+1]`` on the
CPU (the varlen tables are built on the host, nha_fla/ops/nha/chunk.py:660).  Outputs that are not asked
for (final states, initial-state gradients) come back as empty tensors: an operator returns tensors only.
``chunk_nha_packed`` wraps ``prefill_fwd`` the way ``chunk_nha`` wraps the same call."""
from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor

from . import ops as _ops


def _cu_numpy(cu_seqlens: Tensor):
    if cu_seqlens.device.type != "cpu" or cu_seqlens.dtype != torch.int32:
        raise ValueError("cu_seqlens must be an int32 tensor on the CPU")
    return cu_seqlens.contiguous().numpy()


def _empty(ref: Tensor) -> Tensor:
    return torch.empty(0, dtype=torch.float32, device=ref.device)


@torch.library.custom_op("nha_amd::prefill_fwd", mutates_args=(), device_types="cuda")
def prefill_fwd(q_swa: Tensor, k_swa: Tensor, q_gsa: Tensor, k_gsa: Tensor, v: Tensor, s: Tensor, g: Tensor,
                cu_seqlens: Tensor, wl: int, shift: int, scale: float, h0k: Optional[Tensor], h0v: Optional[Tensor],
                want_state: bool) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    h0 = None if h0k is None else (h0k, h0v)
    o, lse_swa, lse_gsa, hkt, hvt = _ops.nha_prefill(q_swa, k_swa, q_gsa, k_gsa, v, s, g, _cu_numpy(cu_seqlens), wl=wl,
                                                     shift=shift, scale=scale, h0=h0, want_state=want_state)
    if not want_state:
        hkt, hvt = _empty(o), _empty(o)
    return o, lse_swa, lse_gsa, hkt, hvt


@prefill_fwd.register_fake
def _(q_swa, k_swa, q_gsa, k_gsa, v, s, g, cu_seqlens, wl, shift, scale, h0k, h0v, want_state):
    T, HQ, K = q_swa.shape
    H, V, M = k_swa.shape[1], v.shape[2], s.shape[2]
    N = cu_seqlens.shape[0] - 1
    f32 = dict(dtype=torch.float32, device=q_swa.device)
    o = q_swa.new_empty(T, HQ, V)
    lse_swa, lse_gsa = torch.empty(T, HQ, **f32), torch.empty(T, HQ, **f32)
    if want_state:
        return o, lse_swa, lse_gsa, torch.empty(N, H, K, M, **f32), torch.empty(N, H, M, V, **f32)
    return o, lse_swa, lse_gsa, torch.empty(0, **f32), torch.empty(0, **f32)


@torch.library.custom_op("nha_amd::prefill_bwd", mutates_args=(), device_types="cuda")
def prefill_bwd(q_swa: Tensor, k_swa: Tensor, q_gsa: Tensor, k_gsa: Tensor, v: Tensor, s: Tensor, g: Tensor, o: Tensor,
                lse_swa: Tensor, lse_gsa: Tensor, dout: Tensor, cu_seqlens: Tensor, wl: int, shift: int, scale: float,
                h0k: Optional[Tensor], h0v: Optional[Tensor], dlse_swa: Optional[Tensor], dlse_gsa: Optional[Tensor],
                dhkt: Optional[Tensor], dhvt: Optional[Tensor], want_dh0: bool
                ) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    dht = None if dhkt is None and dhvt is None else (dhkt, dhvt)
    grads = _ops.nha_prefill_bwd(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, dout, _cu_numpy(cu_seqlens),
                                 wl=wl, shift=shift, scale=scale, h0=None if h0k is None else (h0k, h0v),
                                 dlse_swa=dlse_swa, dlse_gsa=dlse_gsa, dht=dht, want_dh0=want_dh0)
    dh0k, dh0v = grads[7], grads[8]
    if dh0k is None:
        dh0k, dh0v = _empty(o), _empty(o)
    return (*grads[:7], dh0k, dh0v)


@prefill_bwd.register_fake
def _(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, dout, cu_seqlens, wl, shift, scale, h0k, h0v, dlse_swa,
      dlse_gsa, dhkt, dhvt, want_dh0):
    outs = tuple(torch.empty_like(x) for x in (q_swa, k_swa, q_gsa, k_gsa, v, s, g))
    f32 = dict(dtype=torch.float32, device=q_swa.device)
    if want_dh0:
        N = cu_seqlens.shape[0] - 1
        H, K, V, M = k_swa.shape[1], q_swa.shape[2], v.shape[2], s.shape[2]
        return (*outs, torch.empty(N, H, K, M, **f32), torch.empty(N, H, M, V, **f32))
    return (*outs, torch.empty(0, **f32), torch.empty(0, **f32))


def _setup_context(ctx, inputs, output):
    q_swa, k_swa, q_gsa, k_gsa, v, s, g, cu_seqlens, wl, shift, scale, h0k, h0v, want_state = inputs
    o, lse_swa, lse_gsa, _, _ = output
    ctx.save_for_backward(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, h0k, h0v, cu_seqlens)
    ctx.wl, ctx.shift, ctx.scale, ctx.want_state = wl, shift, scale, want_state
    ctx.set_materialize_grads(False)


def _backward(ctx, do, dlse_swa, dlse_gsa, dhkt, dhvt):
    q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, h0k, h0v, cu_seqlens = ctx.saved_tensors
    if do is None:
        do = torch.zeros_like(o)
    if not ctx.want_state:
        dhkt = dhvt = None            # the empty placeholders carry no cotangent
    want_dh0 = h0k is not None and (ctx.needs_input_grad[11] or ctx.needs_input_grad[12])
    grads = torch.ops.nha_amd.prefill_bwd(q_swa, k_swa, q_gsa, k_gsa, v, s, g, o, lse_swa, lse_gsa, do.to(o.dtype).contiguous(),
                                          cu_seqlens, ctx.wl, ctx.shift, ctx.scale, h0k, h0v, dlse_swa, dlse_gsa, dhkt, dhvt,
                                          want_dh0)
    dh0k = dh0v = None
    if want_dh0:
        dh0k, dh0v = grads[7].to(h0k.dtype), grads[8].to(h0v.dtype)
    return (*grads[:7], None, None, None, None, dh0k, dh0v, None)


torch.library.register_autograd("nha_amd::prefill_fwd", _backward, setup_context=_setup_context)


def chunk_nha_packed(q_swa: Tensor, k_swa: Tensor, q_gsa: Tensor, k_gsa: Tensor, v: Tensor, s: Tensor, g: Tensor,
                     cu_seqlens: Tensor, *, window_size_left: int = -1, gsa_kv_shift: int = 0,
                     scale: Optional[float] = None, initial_state: Optional[Tuple[Tensor, Tensor]] = None,
                     output_final_state: bool = False):
    """``chunk_nha`` on packed token-major tensors ``[T_tot, heads, dim]`` through the registered operator
    (differentiable, traceable).  ``cu_seqlens``: int32 ``[N+1]`` on the CPU.  Returns ``(o, lse_swa, lse_gsa)``
    plus ``(hkt, hvt)`` when ``output_final_state``."""
    if scale is None:
        scale = q_swa.shape[-1] ** -0.5
    h0k, h0v = (None, None) if initial_state is None else initial_state
    o, lse_swa, lse_gsa, hkt, hvt = torch.ops.nha_amd.prefill_fwd(q_swa, k_swa, q_gsa, k_gsa, v, s, g, cu_seqlens,
                                                                  int(window_size_left), int(gsa_kv_shift), float(scale),
                                                                  h0k, h0v, bool(output_final_state))
    if output_final_state:
        return o, lse_swa, lse_gsa, (hkt, hvt)
    return o, lse_swa, lse_gsa
