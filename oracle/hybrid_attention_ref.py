"""TEST INFRASTRUCTURE ONLY: CPU restatement of the hybrid decoder models' attention blocks.

Follows the reference's own sequence of operations, cat-shift cache included, in float64 on the CPU
(nha_fla/models/qwen3_moe_nha/qwennha.py:88-398 for the MoE flavour, nha_fla/models/llama3_nha/
llamanha.py:64-262 for the dense one, nha_fla/models/nha_cache.py:43-154 for the cache), on top of
this package's pinned per-token recurrences (`prefill_ref`, `decode_ref`).  Only tests may import it.

Pinned by: tests/test_hybrid_modules.py checks the zero-sink branch against a brute-force softmax over
explicitly materialised zero rows, the window rule of the cache against a list-based model of it, and
the gate-pooling helper against torch's avg_pool1d on random weights; the NHA branches reduce to
`prefill_ref` / `decode_ref`, which tests/test_oracle_pins.py pins.

`round_to` (e.g. torch.bfloat16) rounds every tensor at the points where a model running in that dtype
rounds (projection outputs, norm outputs, gates, rotated q / k), so that a comparison with a bf16 run
measures the attention arithmetic and not the accumulated rounding of the projections.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .nha_ref import decode_ref, prefill_ref

F64 = torch.float64


def _rope_tables(pos: torch.Tensor, D: int, theta: float):
    """cos / sin `[B, T, D]` of the default rotary embedding for integer positions `[B, T]`."""
    inv = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = pos.to(torch.float32)[..., None] * inv
    emb = torch.cat([ang, ang], -1)
    return emb.cos(), emb.sin()


def _rotate_half(x, cos, sin):
    """transformers' apply_rotary_pos_emb with unsqueeze_dim=2 (qwennha.py:247, llamanha.py:150)."""
    h = x.shape[-1] // 2
    rot = torch.cat([-x[..., h:], x[..., :h]], -1)
    return x * cos[:, :, None, :] + rot * sin[:, :, None, :]


def zero_sink_attention_ref(sq, sk, v, window: int, num_sinks: int):
    """The reference's `naive_swa` chain for a layer whose window exceeds 64 (qwennha.py:323-336,
    :400-413; llamanha.py:204-216, :258-270): `num_sinks` zero rows are put in front of q, k and v, the
    band [i-W+1, i] is taken in the shifted coordinates, the scale is 1/sqrt(D), the first `num_sinks`
    output rows are dropped.  sq `[B,T,HQ,D]`, sk / v `[B,T,H,D]` (kv heads are repeated group-major)."""
    B, T, HQ, D = sq.shape
    G = HQ // sk.shape[2]
    sk, v = sk.repeat_interleave(G, 2), v.repeat_interleave(G, 2)
    z = lambda x: torch.zeros(B, num_sinks, *x.shape[2:], dtype=x.dtype)
    q_, k_, v_ = torch.cat([z(sk), sq], 1), torch.cat([z(sk), sk], 1), torch.cat([z(v), v], 1)
    n = T + num_sinks
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    valid = (j >= (i - window + 1).clamp(min=0)) & (j <= i)
    qk = torch.einsum("bthd,bnhd->bhtn", q_, k_) / D ** 0.5
    qk = qk.masked_fill(~valid[None, None], -1e7)
    p = qk.transpose(1, 2).softmax(-1)                          # [B, n, HQ, n]
    return torch.einsum("bthw,bwhd->bthd", p, v_)[:, num_sinks:]


class HybridAttentionRef:
    """One attention block.  `weights`: q_proj / k_proj / v_proj / o_proj / g_proj `.weight` (and
    optional `.bias`), `q_norm.weight` / `k_norm.weight` for the MoE flavour."""

    def __init__(self, weights: Dict[str, torch.Tensor], *, num_heads: int, num_kv_heads: int, head_dim: int,
                 num_slots: int, window_size: int, qk_norm: bool, eps: float = 1e-6, rope_theta: float = 10000.0,
                 round_to: Optional[torch.dtype] = None):
        self.w = {k: v.detach().to("cpu", F64) for k, v in weights.items()}
        self.HQ, self.H, self.D, self.M, self.W = num_heads, num_kv_heads, head_dim, num_slots, window_size
        self.qk_norm, self.eps, self.theta, self.round_to = qk_norm, eps, rope_theta, round_to

    def _r(self, x):
        return x if self.round_to is None else x.to(self.round_to).to(F64)

    def _lin(self, name, x):
        y = x @ self.w[name + ".weight"].T
        if name + ".bias" in self.w:
            y = y + self.w[name + ".bias"]
        return self._r(y)

    def _norm(self, name, x):
        y = self._r(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps))
        return self._r(self.w[name + ".weight"] * y)

    def forward(self, x, position_ids, cache: Optional[dict] = None, attention_mask=None):
        """x `[B,T,hidden]`, position_ids `[B,T]`; `cache` is this layer's dict (empty at first), holding
        the time-ordered window `k`, `v`, `g` `[B,n,H,*]` (un-rotated keys) and the slot state `hk`, `hv`."""
        x = x.detach().to("cpu", F64)
        B, T, _ = x.shape
        HQ, H, D, M, W = self.HQ, self.H, self.D, self.M, self.W
        q = self._lin("q_proj", x).view(B, T, HQ, D)
        k = self._lin("k_proj", x).view(B, T, H, D)
        v = self._lin("v_proj", x).view(B, T, H, D)
        f = self._lin("g_proj", x).view(B, T, H, M)
        if self.qk_norm:                                            # qwennha.py:105-106
            q, k = self._norm("q_norm", q), self._norm("k_norm", k)
        g = self._r(self._r(torch.nn.functional.logsigmoid(f)) / 8)  # qwennha.py:120
        had_content = cache is not None and "k" in cache
        decode = T == 1 and had_content
        s = None if decode else self._r(1 - self._r(torch.exp(g)))  # qwennha.py:126-130
        if attention_mask is not None:                              # qwennha.py:133-144
            if attention_mask.dim() == 4:                           # [B,1,Q,T'] against head-first tensors (:134-136)
                m = attention_mask.to(F64)[:, :, :, -T:].transpose(1, 2)
            else:
                m = attention_mask.to(F64)[:, -T:, None, None]
            v = v * m
            if s is not None:
                s = s * m
        state = (cache["hk"], cache["hv"]) if had_content and cache.get("hk") is not None else None
        nha = W <= 64
        if cache is not None:
            # the entry that leaves the window is read before the window takes the new tokens
            # (qwennha.py:151-176; nha_cache.py:143-154: only once the window is full)
            if had_content and cache["k"].shape[1] >= W:
                pop = tuple(cache[n][:, 0:1] for n in ("k", "v", "g"))
            else:
                pop = (torch.zeros(B, 1, H, D, dtype=F64), torch.zeros(B, 1, H, D, dtype=F64), torch.zeros(B, 1, H, M, dtype=F64))
            if not had_content:                                     # nha_cache.py:84-97
                for n, t in (("k", k), ("v", v), ("g", g)):
                    cache[n] = t[:, -W:].clone()
            else:                                                   # nha_cache.py:104-131, T <= W
                for n, t in (("k", k), ("v", v), ("g", g)):
                    held = cache[n]
                    cache[n] = torch.cat([held[:, T:], t], 1) if held.shape[1] == W else torch.cat([held, t], 1)
        if decode:
            kw, vw = cache["k"], cache["v"]
            n = kw.shape[1]
            swa_pos = position_ids.to("cpu") - torch.arange(n - 1, -1, -1)[None]          # qwennha.py:211
            cos, sin = (self._r(t.to(F64)) for t in _rope_tables(swa_pos, D, self.theta))
            if nha:                                                  # qwennha.py:351-365
                o, hk, hv, _, _ = decode_ref(q, pop[0], pop[1], pop[2], kw, vw, cos=cos, sin=sin,
                                             initial_state=state, dtype=F64)
                cache["hk"], cache["hv"] = hk, hv
            else:                                                    # qwennha.py:377-389, llamanha.py:238-246
                sq = self._r(_rotate_half(q, cos[:, -1:], sin[:, -1:]))
                sk = self._r(_rotate_half(kw, cos, sin))
                G = HQ // H
                sk_, v_ = sk.repeat_interleave(G, 2), vw.repeat_interleave(G, 2)
                zk = torch.zeros(B, M, HQ, D, dtype=F64)
                k_all, v_all = torch.cat([zk, sk_], 1), torch.cat([zk, v_], 1)
                p = (torch.einsum("bthd,bnhd->bthn", sq, k_all) / D ** 0.5).softmax(-1)
                o = torch.einsum("bthw,bwhd->bthd", p, v_all)
        else:
            cos, sin = (self._r(t.to(F64)) for t in _rope_tables(position_ids.to("cpu"), D, self.theta))
            sq, sk = self._r(_rotate_half(q, cos, sin)), self._r(_rotate_half(k, cos, sin))
            if nha:                                                  # qwennha.py:308-321, llamanha.py:186-203
                o, _, _, hk, hv = prefill_ref(sq, sk, q, k, v, s, g, window_size_left=W - 1, gsa_kv_shift=W,
                                              initial_state=state, dtype=F64)
                if cache is not None:
                    cache["hk"], cache["hv"] = hk, hv
            else:
                o = zero_sink_attention_ref(sq, sk, v, W, M)
        o = self._r(o)
        return self._lin("o_proj", o.reshape(B, T, HQ * D))
