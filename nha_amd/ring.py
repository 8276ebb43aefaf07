"""Resident decode state: fp32 slot state + W-slot K/V/gate ring buffers, stepped by ONE kernel.

Replaces the cat-shift window cache and the pop/update choreography around the decode op in the
reference (nha_fla/models/nha_cache.py:105-131, :143-154; models/qwen3_moe_nha/qwennha.py:151-176,
:351-365): the kernel pops the oldest ring entry into the slots, stores the new token in its
slot and attends over the valid entries, reading state and window once per kv-head."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib
from .ops import _dtype_code, _need_cuda, _ptr, _stream


@dataclass
class NHARingState:
    """Per-layer decode state for B sequences.  ``ring_k`` holds the window keys as the window
    branch reads them (already rotated), ``ring_kg`` the slot-branch keys (raw), ``ring_g`` the
    log forget gates of the cached tokens; ``count[b]`` tokens have been cached so far."""
    hk: torch.Tensor        # [B,H,K,M] fp32
    hv: torch.Tensor        # [B,H,M,V] fp32
    ring_k: torch.Tensor    # [B,W,H,K]
    ring_kg: torch.Tensor   # [B,W,H,K]
    ring_v: torch.Tensor    # [B,W,H,V]
    ring_g: torch.Tensor    # [B,W,H,M]
    count: torch.Tensor     # [B] int32; the tensor bound to this name changes with every step
    count_alt: Optional[torch.Tensor] = None   # the other counter array (the step writes count + 1 there)
    # the slots never absorb anything (every cached log-gate is 0 and every write strength 0: the zero-sink layers of
    # the hybrid models): hk and hv stay zero, and the step neither reads nor writes them
    zero_state: bool = False

    @classmethod
    def empty(cls, B, H, K, V, M, W, dtype=torch.bfloat16, device="cuda") -> "NHARingState":
        z = lambda *s, dt=dtype: torch.zeros(*s, dtype=dt, device=device)
        return cls(z(B, H, K, M, dt=torch.float32), z(B, H, M, V, dt=torch.float32), z(B, W, H, K), z(B, W, H, K),
                   z(B, W, H, V), z(B, W, H, M), z(B, dt=torch.int32))

    @classmethod
    def from_prefill(cls, k_swa, k_gsa, v, g, final_state, window: int, cu_seqlens=None) -> "NHARingState":
        """The decode state that continues a prefill with ``(window_size_left, gsa_kv_shift) =
        (window - 1, window)``: the slot state is the prefill's final state (it has absorbed the
        tokens that left the window), ring slot ``j % window`` holds token ``j`` for the last
        ``min(L, window)`` tokens of each sequence and ``count = L``.  Takes the prefill's own
        operands: k_swa (rotated), k_gsa, v ``[B,T,H,*]``, g ``[B,T,H,M]`` (``[1,T_tot,...]`` with
        cu_seqlens) and ``final_state = (hk [N,H,K,M], hv [N,H,M,V])``.  The hand-over the reference
        does by slicing the last ``window`` rows into its cache (nha_fla/models/nha_cache.py:87-91)."""
        _need_cuda(k_swa, k_gsa, v, g, final_state[0], final_state[1])
        dev, W = k_swa.device, int(window)
        B, T, H, K = k_swa.shape
        V, M = v.shape[-1], g.shape[-1]
        if cu_seqlens is None:
            starts = torch.arange(B, device=dev, dtype=torch.long) * T
            lens = torch.full((B,), T, device=dev, dtype=torch.long)
        else:
            if B != 1:
                raise ValueError("cu_seqlens needs the packed layout [1, T_tot, ...]")
            cu = cu_seqlens.to(device=dev, dtype=torch.long)
            starts, lens = cu[:-1], cu[1:] - cu[:-1]
        N = starts.numel()
        hk, hv = final_state
        if tuple(hk.shape) != (N, H, K, M) or tuple(hv.shape) != (N, H, M, V):
            raise ValueError(f"final_state must be ([{N},{H},{K},{M}], [{N},{H},{M},{V}]), got {tuple(hk.shape)}, {tuple(hv.shape)}")
        r = torch.arange(W, device=dev, dtype=torch.long)
        last = (lens - 1)[:, None]
        tok = last - torch.remainder(last - r[None, :], W)            # newest token j <= L-1 with j % W == r
        valid = tok >= 0
        src = (starts[:, None] + tok.clamp_min(0)).reshape(-1)

        def gather(x):
            rows = x.reshape(B * T, *x.shape[2:]).index_select(0, src).reshape(N, W, *x.shape[2:])
            return rows * valid[:, :, None, None].to(rows.dtype)

        return cls(hk.to(torch.float32).clone(), hv.to(torch.float32).clone(), gather(k_swa), gather(k_gsa), gather(v),
                   gather(g), lens.to(torch.int32))

    @property
    def window(self) -> int:
        return self.ring_k.shape[1]


def ring_advance(state: NHARingState) -> None:
    """count += 1 for every sequence, in place (one small launch).  For steps taken with ``advance=False``: a
    captured HIP graph replays fixed pointers, so it cannot trade the two counter arrays as the eager step does;
    it runs the step on ``count`` and then this launch."""
    _lib.check(_lib.load().nha_decode_advance(_ptr(state.count), state.count.numel(), _stream(state.count.device)))


def ring_decode_step(state: NHARingState, q: torch.Tensor, sq: torch.Tensor, k_new: torch.Tensor,
                     kg_new: torch.Tensor, v_new: torch.Tensor, g_new: torch.Tensor,
                     scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                     advance: bool = True) -> torch.Tensor:
    """One decode step for every sequence of ``state`` (updated in place).

    q (slot-branch query) and sq (window query, rotated) ``[B,HQ,K]``; the new token's window key
    ``k_new`` (rotated), slot key ``kg_new`` ``[B,H,K]``, value ``[B,H,V]`` and log gate
    ``g_new [B,H,M]``.  Returns ``o [B,HQ,V]``."""
    _need_cuda(q, sq, k_new, kg_new, v_new, g_new, state.hk)
    B, HQ, K = q.shape
    _, W, H, _ = state.ring_k.shape
    V, M = state.ring_v.shape[-1], state.ring_g.shape[-1]
    dt = state.ring_k.dtype
    for name, x, shp in (("q", q, (B, HQ, K)), ("sq", sq, (B, HQ, K)), ("k_new", k_new, (B, H, K)),
                         ("kg_new", kg_new, (B, H, K)), ("v_new", v_new, (B, H, V)), ("g_new", g_new, (B, H, M))):
        if tuple(x.shape) != shp or x.dtype != dt or not x.is_contiguous():
            raise ValueError(f"{name} must be a contiguous {dt} tensor of shape {shp}, got {tuple(x.shape)} {x.dtype}")
    if scale is None:
        scale = K ** -0.5
    o = out if out is not None else torch.empty(B, HQ, V, dtype=dt, device=q.device)
    a = _lib.NhaDecodeArgs()
    a.mode, a.dtype = _lib.NHA_DECODE_RING, _dtype_code(q)
    a.B, a.HQ, a.H, a.K, a.V, a.M, a.W = B, HQ, H, K, V, M, W
    a.scale = float(scale)
    a.q, a.sq = _ptr(q), _ptr(sq)
    a.ring_k, a.ring_kg, a.ring_v, a.ring_g = map(_ptr, (state.ring_k, state.ring_kg, state.ring_v, state.ring_g))
    a.k_new, a.kg_new, a.v_new, a.g_new = _ptr(k_new), _ptr(kg_new), _ptr(v_new), _ptr(g_new)
    a.count = _ptr(state.count)
    if not state.zero_state:      # NULL states: the kernel takes zeros and writes nothing back
        a.hk_in, a.hv_in, a.hk_out, a.hv_out = _ptr(state.hk), _ptr(state.hv), _ptr(state.hk), _ptr(state.hv)
    a.o, a.stream = _ptr(o), _stream(q.device)
    if advance:
        # the kernel writes count + 1 into the second array; the two arrays then trade places
        if state.count_alt is None:
            state.count_alt = torch.empty_like(state.count)
        a.count_next = _ptr(state.count_alt)
    lib = _lib.load()
    _lib.check(lib.nha_decode_step(C.byref(a)))
    if advance:
        state.count, state.count_alt = state.count_alt, state.count
    return o
