"""Per-layer decode cache on resident ring buffers.

The reference keeps, per layer, a time-ordered window (k, v, log-gate) that it shifts with a `cat`
every step, pops the oldest entry from before each step (`get_pop_kvf`) and stores next to the
recurrent slot state (nha_fla/models/nha_cache.py:43-154; call sites
models/llama3_nha/llamanha.py:113-137, models/qwen3_moe_nha/qwennha.py:151-176).  Here the window
lives in W-slot ring buffers that never move and one kernel launch per step pops, stores and
attends (nha_amd/ring.py); this class is the bookkeeping around them with the reference cache's
vocabulary: layers indexed by `layer_idx`, `get_seq_length`, `get_pop_kvf`, `to_legacy_cache`.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .ring import NHARingState, ring_decode_step


class NHARingCache:
    """Decode cache for a stack of NHA layers with window `window_size`."""

    def __init__(self, window_size: int, seen_tokens: int = 0):
        self.window_size = int(window_size)
        self.states: List[Optional[NHARingState]] = []
        self._seen_tokens = seen_tokens

    def __len__(self) -> int:
        return len(self.states)

    def __getitem__(self, layer_idx: int) -> Dict[str, object]:
        """The layer's state in the reference's layout: `recurrent_state` (hk, hv) and `attn_state`
        (k, v, g) time-ordered `[B, n, H*dim]` (a gathered copy, n = min(tokens, window); the
        sequences of a batch must be equally long, as the reference's cat-shift cache needs)."""
        if layer_idx >= len(self.states) or self.states[layer_idx] is None:
            raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")
        st = self.states[layer_idx]
        k, v, g = self.window(layer_idx)
        return dict(recurrent_state=(st.hk, st.hv), attn_state=(k.flatten(-2), v.flatten(-2), g.flatten(-2)),
                    conv_state=None, ffn_state=None)

    def _uniform_count(self, st: NHARingState) -> int:
        c = st.count.tolist()
        if any(x != c[0] for x in c):
            raise ValueError("time-ordered views need sequences of equal length; use the ring buffers directly")
        return c[0]

    def prefill(self, layer_idx: int, k_swa, k_gsa, v, g, final_state, cu_seqlens=None) -> NHARingState:
        """Hand a prompt's prefill (operands and final state of chunk_nha / fused_chunk_nha_prefill
        with (window_size_left, gsa_kv_shift) = (W-1, W)) over to the ring buffers of `layer_idx`."""
        st = NHARingState.from_prefill(k_swa, k_gsa, v, g, final_state, self.window_size, cu_seqlens=cu_seqlens)
        while len(self.states) <= layer_idx:
            self.states.append(None)
        self.states[layer_idx] = st
        if layer_idx == 0:
            self._seen_tokens += int(st.count.max().item())
        return st

    def decode(self, layer_idx: int, q_gsa, q_swa, k_swa, k_gsa, v, g, scale: Optional[float] = None) -> torch.Tensor:
        """One token per sequence through layer `layer_idx`: pops the entry leaving the window into the
        slots, stores the new token, attends (one launch).  Tensors `[B, heads, dim]`; returns o."""
        st = self.states[layer_idx]
        o = ring_decode_step(st, q_gsa, q_swa, k_swa, k_gsa, v, g, scale=scale)
        if layer_idx == 0:
            self._seen_tokens += 1
        return o

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if layer_idx >= len(self.states) or self.states[layer_idx] is None:
            return 0
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        return None

    def get_pop_kvf(self, layer_idx: int, window_size: Optional[int] = None) -> Tuple[Optional[torch.Tensor], ...]:
        """(k_gsa, v, g) `[B, 1, H*dim]` of the entry the next step pops into the slots, or Nones while
        the window is not full (nha_fla/models/nha_cache.py:143-154).  The step itself does not need
        this call: it reads the ring slot in the kernel."""
        if layer_idx >= len(self.states) or self.states[layer_idx] is None:
            return (None, None, None)
        st = self.states[layer_idx]
        W = st.window
        if window_size is not None and window_size != W:
            raise ValueError(f"this cache was built for window {W}, got {window_size}")
        n = self._uniform_count(st)
        if n < W:
            return (None, None, None)
        slot = n % W
        return tuple(x[:, slot:slot + 1].flatten(-2) for x in (st.ring_kg, st.ring_v, st.ring_g))

    def window(self, layer_idx: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Time-ordered copy (oldest first) of the cached window: rotated keys, values, log gates
        `[B, n, H, dim]`."""
        st = self.states[layer_idx]
        W, n = st.window, self._uniform_count(st)
        m = min(n, W)
        idx = (torch.arange(n - m, n, device=st.ring_k.device) % W)
        return st.ring_k[:, idx], st.ring_v[:, idx], st.ring_g[:, idx]

    def to_legacy_cache(self) -> Tuple:
        return tuple(self[i] for i in range(len(self.states)))
