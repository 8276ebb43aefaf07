"""Per-layer decode cache on resident ring buffers.

The reference keeps, per layer, a time-ordered window (k, v, log-gate) that it shifts with a `cat`
every step, pops the oldest entry from before each step (`get_pop_kvf`) and stores next to the
recurrent slot state (nha_fla/models/nha_cache.py:43-154; call sites
models/llama3_nha/llamanha.py:113-137, models/qwen3_moe_nha/qwennha.py:151-176).  Here the window
lives in W-slot ring buffers that never move and one kernel launch per step pops, stores and
attends (nha_amd/ring.py); this class is the bookkeeping around them with the reference cache's
protocol: layers indexed by `layer_idx`, `update(recurrent_state, attn_state, conv_state, ffn_state,
layer_idx, offset, cache_kwargs)`, iteration, `get_seq_length` (the token count BEFORE the latest
update, as the reference reports it), `get_pop_kvf`, `to_legacy_cache` / `from_legacy_cache`.

A layer's entry can hold its window in either form: ring buffers (`prefill` / `decode`, the form the
decode kernel consumes) or, when a caller hands `attn_state` tuples to `update` as it would to the
reference's cache, the reference's time-ordered tensors, kept by the same window rule.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .ring import NHARingState, ring_advance, ring_decode_step


class NHARingCache:
    """Decode cache for a stack of NHA layers with window `window_size`."""

    def __init__(self, window_size: Optional[int] = None, seen_tokens: int = 0):
        self.window_size = None if window_size is None else int(window_size)
        self.states: List[Optional[NHARingState]] = []     # ring-buffer form of a layer's window + slot state
        self.extra: List[Dict[str, object]] = []           # what `update` was given: recurrent / conv / ffn / attn state
        self.former_tokens = seen_tokens
        self._seen_tokens = seen_tokens
        self._layer_tokens: Dict[int, int] = {}            # tokens a layer's ring has taken so far (longest sequence)

    def __len__(self) -> int:
        return max(len(self.states), len(self.extra))

    def __iter__(self):
        for i in range(len(self)):
            yield self[i]

    def _grow(self, layer_idx: int) -> None:
        while len(self.states) <= layer_idx:
            self.states.append(None)
        while len(self.extra) <= layer_idx:
            self.extra.append(dict(recurrent_state=None, attn_state=None, conv_state=None, ffn_state=None))

    def _count_tokens(self, layer_idx: int, offset: int, whole_step: bool = False) -> None:
        """`update` counts as the reference does: `former_tokens` is the count before this update.  The
        reference's attention modules update a layer twice per forward (window entries with the new tokens'
        count, then the recurrent state with offset 0), after which both counters agree; `prefill` and
        `decode` are such whole steps."""
        if layer_idx == 0:
            self.former_tokens = self._seen_tokens
            self._seen_tokens += int(offset)
            if whole_step:
                self.former_tokens = self._seen_tokens

    def update(self, recurrent_state=None, attn_state=None, conv_state=None, ffn_state=None, layer_idx: int = 0,
               offset: Optional[int] = 1, cache_kwargs: Optional[Dict[str, object]] = None) -> Dict[str, object]:
        """The reference cache's update (nha_fla/models/nha_cache.py:43-141): stores whichever states are
        given for `layer_idx`, counts `offset` new tokens on layer 0, returns the layer's entry.  An
        `attn_state` (k, v, g) `[..., n, dim]` follows the reference's window rule: entries are appended
        in time order and, once `cache_kwargs['window_size']` of them are held, the oldest leave; a chunk
        longer than the window stores its freshest `window_size` entries and the returned entry carries
        the whole chunk."""
        self._count_tokens(layer_idx, offset)
        self._grow(layer_idx)
        e = self.extra[layer_idx]
        if recurrent_state is not None:
            e["recurrent_state"] = recurrent_state
        if conv_state is not None:
            e["conv_state"] = conv_state
        if ffn_state is not None:
            e["ffn_state"] = ffn_state
        returned_attn = None
        if attn_state is not None:
            if not isinstance(attn_state, tuple) or len(attn_state) != 3:
                raise ValueError("`attn_state` must be a tuple of three tensors: keys, values, log gates")
            W = (cache_kwargs or {}).get("window_size", None)
            held = e["attn_state"]
            n_new = attn_state[0].shape[-2]
            if held is None:
                joined = attn_state
            else:
                joined = tuple(torch.cat([h, a], -2) for h, a in zip(held, attn_state))
            if W is not None and joined[0].shape[-2] > W:
                if n_new > W:
                    returned_attn = attn_state
                joined = tuple(x[..., -W:, :].contiguous() for x in joined)
            e["attn_state"] = joined
        out = self[layer_idx]
        if returned_attn is not None:
            out = dict(out)
            out["attn_state"] = returned_attn
        return out

    @classmethod
    def from_legacy_cache(cls, past_key_values=None, seen_tokens: int = 0,
                          window_size: Optional[int] = None) -> "NHARingCache":
        """A cache holding the per-layer dicts of `to_legacy_cache()` (nha_fla/models/nha_cache.py:167-182)."""
        cache = cls(window_size=window_size, seen_tokens=seen_tokens)
        if isinstance(past_key_values, (list, tuple)):
            for i, st in enumerate(past_key_values):
                cache._grow(i)
                cache.extra[i].update({k: st.get(k) for k in ("recurrent_state", "attn_state", "conv_state", "ffn_state")})
        return cache

    def __getitem__(self, layer_idx: int) -> Dict[str, object]:
        """The layer's state in the reference's layout: `recurrent_state` (hk, hv) and `attn_state`
        (k, v, g) time-ordered `[B, n, H*dim]` (a gathered copy, n = min(tokens, window); the
        sequences of a batch must be equally long, as the reference's cat-shift cache needs)."""
        if layer_idx >= len(self) or (self._ring(layer_idx) is None and not self._has_extra(layer_idx)):
            raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")
        e = self.extra[layer_idx] if layer_idx < len(self.extra) else {}
        st = self._ring(layer_idx)
        if st is None:
            return dict(recurrent_state=e.get("recurrent_state"), attn_state=e.get("attn_state"),
                        conv_state=e.get("conv_state"), ffn_state=e.get("ffn_state"))
        k, v, g = self.window(layer_idx)
        return dict(recurrent_state=(st.hk, st.hv), attn_state=(k.flatten(-2), v.flatten(-2), g.flatten(-2)),
                    conv_state=e.get("conv_state"), ffn_state=e.get("ffn_state"))

    def _ring(self, layer_idx: int) -> Optional[NHARingState]:
        return self.states[layer_idx] if layer_idx < len(self.states) else None

    def _has_extra(self, layer_idx: int) -> bool:
        return layer_idx < len(self.extra) and any(v is not None for v in self.extra[layer_idx].values())

    def _uniform_count(self, st: NHARingState) -> int:
        c = st.count.tolist()
        if any(x != c[0] for x in c):
            raise ValueError("time-ordered views need sequences of equal length; use the ring buffers directly")
        return c[0]

    def prefill(self, layer_idx: int, k_swa, k_gsa, v, g, final_state, cu_seqlens=None,
                window_size: Optional[int] = None, zero_state: bool = False) -> NHARingState:
        """Hand a prompt's prefill (operands and final state of chunk_nha / fused_chunk_nha_prefill
        with (window_size_left, gsa_kv_shift) = (W-1, W)) over to the ring buffers of `layer_idx`.
        `window_size` overrides the cache's window for this layer (models mix short-window layers with
        2048-token ones)."""
        W = self._window(window_size)
        st = NHARingState.from_prefill(k_swa, k_gsa, v, g, final_state, W, cu_seqlens=cu_seqlens)
        # `zero_state`: a layer whose gates are all 0 and whose write strengths are all 0 (the caller's promise, for
        # this prompt and every later step): its slot state stays zero and the decode step skips it
        st.zero_state = bool(zero_state)
        self._grow(layer_idx)
        self.states[layer_idx] = st
        longest = k_swa.shape[1] if cu_seqlens is None else int(st.count.max().item())
        self._layer_tokens[layer_idx] = longest
        self._count_tokens(layer_idx, longest, whole_step=True)
        return st

    def _window(self, window_size: Optional[int]) -> int:
        """The window of a call: its own `window_size`, else the one the cache was built with."""
        W = self.window_size if window_size is None else int(window_size)
        if W is None:
            raise ValueError("this cache was built without a window size: pass `window_size` with the call "
                             "(the attention modules do) or to the constructor")
        return W

    def has_ring(self, layer_idx: int) -> bool:
        """Whether `layer_idx` holds ring buffers (a prompt was handed over with `prefill`)."""
        return self._ring(layer_idx) is not None

    def layer_tokens(self, layer_idx: int) -> int:
        """Tokens the ring of `layer_idx` has taken (its longest sequence): the next token's position."""
        return self._layer_tokens.get(layer_idx, 0)

    def decode(self, layer_idx: int, q_gsa, q_swa, k_swa, k_gsa, v, g, scale: Optional[float] = None,
               in_place_counters: bool = False) -> torch.Tensor:
        """One token per sequence through layer `layer_idx`: pops the entry leaving the window into the
        slots, stores the new token, attends (one launch).  Tensors `[B, heads, dim]`; returns o.
        `in_place_counters`: advance the ring counters with a second small launch on the same array instead of
        trading the two counter arrays (what a step recorded into a HIP graph needs: a replay uses fixed pointers)."""
        st = self.states[layer_idx]
        o = ring_decode_step(st, q_gsa, q_swa, k_swa, k_gsa, v, g, scale=scale, advance=not in_place_counters)
        if in_place_counters:
            ring_advance(st)
        self.note_step(layer_idx)
        return o

    def note_step(self, layer_idx: int) -> None:
        """Host-side bookkeeping of one decode step of `layer_idx` (token counts; no GPU work): `decode` calls it,
        and so does every replay of a recorded step."""
        self._layer_tokens[layer_idx] = self._layer_tokens.get(layer_idx, 0) + 1
        self._count_tokens(layer_idx, 1, whole_step=True)

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        """Tokens cached before the latest update of layer 0 (`former_tokens`,
        nha_fla/models/nha_cache.py:156-160): during a model's forward, after layer 0 has stored the
        step's tokens, the later layers still read the position the step started from."""
        if layer_idx >= len(self) or (self._ring(layer_idx) is None and not self._has_extra(layer_idx)):
            return 0
        return self.former_tokens

    @property
    def seen_tokens(self) -> int:
        """Tokens cached so far, the latest update included."""
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        return None

    def get_pop_kvf(self, layer_idx: int, window_size: Optional[int] = None) -> Tuple[Optional[torch.Tensor], ...]:
        """(k_gsa, v, g) `[B, 1, H*dim]` of the entry the next step pops into the slots, or Nones while
        the window is not full (nha_fla/models/nha_cache.py:143-154).  The step itself does not need
        this call: it reads the ring slot in the kernel."""
        st = self._ring(layer_idx)
        if st is None:
            held = self.extra[layer_idx]["attn_state"] if layer_idx < len(self.extra) else None
            if held is None:
                return (None, None, None)
            W = self._window(window_size)
            if held[0].shape[-2] >= W:
                return tuple(x[..., 0:1, :] for x in held)
            return (None, None, None)
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
        return tuple(self[i] for i in range(len(self)))


class NHACache(NHARingCache):
    """`NHARingCache` under the reference cache's name and constructor (`NHACache(seen_tokens=0)`,
    nha_fla/models/nha_cache.py:20-29; built without arguments at scripts/verify_opt_parity.py:671): the
    window size is not a property of the reference's cache -- its callers pass it with every `update`
    and `get_pop_kvf`, as the attention modules here pass it to `prefill` -- so it is an optional keyword."""

    def __init__(self, seen_tokens: int = 0, window_size: Optional[int] = None):
        super().__init__(window_size=window_size, seen_tokens=seen_tokens)
