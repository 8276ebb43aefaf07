"""Attention modules of the hybrid decoder models, on the GQA-native prefill and the ring-buffer decode.

The reference's converted decoder models (nha_fla/models/qwen3_moe_nha/qwennha.py:43-413, the MoE
flavour with per-head q/k RMSNorm; nha_fla/models/llama3_nha/llamanha.py:30-270, the dense flavour)
replace every softmax-attention block by one of two kinds of layer, chosen per layer index
(qwennha.py:64-68, llamanha.py:58-62):

* an NHA layer (window <= 64): M gated slots + a short sliding window under one softmax.  Prefill is
  one `fused_chunk_nha_prefill` call on the kv-head layout (qwennha.py:308-321; the dense flavour's
  repeat-to-query-heads chain, llamanha.py:186-203, computes the same numbers).  Decode is one
  `ring_decode_step` launch on the layer's resident ring buffers instead of the reference's
  pop / cat-shift / re-rotate / decode-op sequence (qwennha.py:151-176, :200-226, :351-365): keys are
  rotated once, at their own position, when they enter the ring.
* a "full attention" layer (window 2048): plain sliding-window softmax attention preceded by
  `num_slots` all-zero key/value rows (qwennha.py:323-336, llamanha.py:204-216).  Query t therefore
  sees `clamp(W-1-t, 0, M)` zero-logit sinks next to its window.  Here that is the same NHA kernel with
  slot states that stay zero (s = 0, g = 0: M zero logits with zero values at every t), rescaled per
  query by (e^lse_swa + M) / (e^lse_swa + sinks(t)) from the window log-sum-exp the kernel returns.
  Decode keeps all M sinks at every step, as the reference's torch path does (llamanha.py:238-246,
  qwennha.py:377-389; its optional flash-attn call, qwennha.py:371-375, has none, and that package is
  no part of this build).

The cache is `NHARingCache`; a layer hands its prompt over with `cache.prefill` and steps with
`cache.decode`.  Everything heavy runs in libnha_hip.so; the projections are torch GEMMs.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .cache import NHARingCache
from .ops import (chunk_nha, fused_chunk_nha_prefill, hybrid_prologue_supported, nha_hybrid_prologue,
                  nha_zero_sink_rescale_, zero_sink_attention, zero_sink_attention_supported)

GATE_LOGIT_NORMALIZER = 8          # qwennha.py:62, llamanha.py:96
FULL_ATTENTION_WINDOW = 2048       # qwennha.py:66, llamanha.py:60
NHA_MAX_WINDOW = 64                # layers with a longer window are the zero-sink kind (qwennha.py:307, llamanha.py:187)


@dataclass
class HybridNHAConfig:
    """The fields of the reference's model configurations that the attention modules read
    (configuration_qwen3_moe_nha.py:36-109, configuration_llama3_nha.py:13-73); any object with
    these attributes (a transformers config among them) works in its place."""
    hidden_size: int = 2048
    num_attention_heads: int = 32
    num_key_value_heads: int = 4
    head_dim: Optional[int] = None
    num_slots: int = 64
    window_size: int = 32
    block_size: Optional[int] = None
    transformer_idx: Optional[int] = None
    attention_bias: bool = False
    attention_dropout: float = 0.0
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    max_position_embeddings: int = 32768


class HeadRMSNorm(nn.Module):
    """RMSNorm over the last (head) dimension, statistics in fp32, as the q/k norms of the MoE flavour
    (qwennha.py:83-84)."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.variance_epsilon = eps

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        dt = x.dtype
        x = x.to(torch.float32)
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * x.to(dt)


class RotaryTables(nn.Module):
    """cos / sin of the default rotary embedding, `[B, T, head_dim]` for integer positions `[B, T]`
    (two copies of the head_dim/2 angles side by side: the rotate-half convention)."""

    def __init__(self, head_dim: int, base: float = 10000.0):
        super().__init__()
        self.head_dim, self.base = head_dim, base
        self._inv_freq = {}          # per device; not a buffer: `module.to(torch.bfloat16)` would round a buffer, and
                                     # frequencies rounded to 8 bits put position 100 off by a quarter of a radian

    def inv_freq(self, device) -> torch.Tensor:
        f = self._inv_freq.get(device)
        if f is None:
            f = 1.0 / (self.base ** (torch.arange(0, self.head_dim, 2, dtype=torch.float32) / self.head_dim))
            f = self._inv_freq[device] = f.to(device)
        return f

    @torch.no_grad()
    def forward(self, x: torch.Tensor, position_ids: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        ang = position_ids.to(x.device, torch.float32)[..., None] * self.inv_freq(x.device)
        emb = torch.cat([ang, ang], -1)
        return emb.cos().to(x.dtype), emb.sin().to(x.dtype)


def rotate_half_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x `[B, T, heads, D]`, cos / sin `[B, T, D]`: x cos + rotate_half(x) sin, evaluated in fp32 and
    rounded to x's dtype once (as the decode kernel's in-kernel rotary does)."""
    half = x.shape[-1] // 2
    xf = x.to(torch.float32)
    rot = torch.cat([-xf[..., half:], xf[..., :half]], -1)
    return (xf * cos[:, :, None, :].to(torch.float32) + rot * sin[:, :, None, :].to(torch.float32)).to(x.dtype)


def zero_sink_count(T: int, window: int, num_sinks: int, device) -> torch.Tensor:
    """How many of the `num_sinks` zero rows in front of the sequence the W-wide window of query t still
    covers: positions are shifted by num_sinks, the window spans [t + num_sinks - W + 1, t + num_sinks]."""
    t = torch.arange(T, device=device)
    return (window - 1 - t).clamp(0, num_sinks)


def zero_sink_rescale(lse_swa: torch.Tensor, num_sinks: int, sinks_seen: torch.Tensor) -> torch.Tensor:
    """(e^lse + num_sinks) / (e^lse + sinks_seen), formed in log space so that a window whose scores are all
    strongly negative (lse < -88, where e^-lse leaves fp32) still gives the finite ratio num_sinks / sinks_seen
    (with no sink seen the ratio is 1 + num_sinks e^-lse, capped at the largest fp32 so that a row whose
    output has underflowed to zero stays zero instead of becoming 0 * inf)."""
    lse = lse_swa.to(torch.float32)
    log_seen = torch.log(sinks_seen.to(torch.float32))          # -inf where the window covers no sink
    return torch.exp(torch.logaddexp(lse, torch.full_like(lse, math.log(num_sinks)))
                     - torch.logaddexp(lse, log_seen.expand_as(lse))).clamp(max=torch.finfo(torch.float32).max)


def pool_k_to_g(k_weight: torch.Tensor, target_rows: int) -> torch.Tensor:
    """Gate-projection initialisation from a key projection (training/convert_weight.py:7-22): the
    `[rows, hidden]` key weight is averaged over groups of rows/target_rows consecutive rows."""
    rows, hidden = k_weight.shape
    if rows % target_rows != 0:
        raise ValueError(f"The source dimension {rows} must be divisible by the target dimension {target_rows}.")
    return k_weight.reshape(target_rows, rows // target_rows, hidden).mean(1)


@torch.no_grad()
def init_gates_from_keys(model: nn.Module) -> int:
    """For every `...g_proj.weight` of `model` with a sibling `...k_proj.weight`, copy the pooled key
    weight into it (training/convert_weight.py:36-48).  Returns the number of gate projections set."""
    params = dict(model.named_parameters())
    done = 0
    for name, p in params.items():
        if "g_proj" in name and "weight" in name:
            kp = params.get(name.replace("g_proj", "k_proj"))
            if kp is None:
                continue
            p.copy_(pool_k_to_g(kp.detach().to(torch.float32), p.shape[0]).to(p.dtype))
            done += 1
    return done


class HybridNHAAttention(nn.Module):
    """One attention block of a hybrid decoder: projections, gates, rotary, the NHA kernels, o_proj.
    `forward` has the reference modules' signature and returns `(output, None)`."""

    qk_norm = False
    fuse_glue = True      # inference: fused projection GEMM + one glue launch (False keeps the tensor-op chain)
    _recording = False    # set while a decode step is recorded into a HIP graph (record_decode_step)

    def __init__(self, config, layer_idx: int = 0):
        super().__init__()
        self._fused_key, self._fused_wb = None, None
        self.config = config
        self.layer_idx = layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.num_key_value_heads = config.num_key_value_heads or config.num_attention_heads
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.head_dim = getattr(config, "head_dim", None) or self.hidden_size // self.num_heads
        self.scaling = self.head_dim ** -0.5
        self.num_slots = config.num_slots
        self.gate_logit_normalizer = GATE_LOGIT_NORMALIZER
        self.window_size = config.window_size
        block, which = getattr(config, "block_size", None), getattr(config, "transformer_idx", None)
        if block is not None and which is not None and layer_idx % block == which:
            self.window_size = FULL_ATTENTION_WINDOW
        bias = bool(getattr(config, "attention_bias", False)) and self.qk_norm
        HQ, H, D = self.num_heads, self.num_key_value_heads, self.head_dim
        self.q_proj = nn.Linear(self.hidden_size, HQ * D, bias=bias)
        self.k_proj = nn.Linear(self.hidden_size, H * D, bias=bias)
        self.v_proj = nn.Linear(self.hidden_size, H * D, bias=bias)
        self.o_proj = nn.Linear(HQ * D, self.hidden_size, bias=bias)
        self.g_proj = nn.Linear(self.hidden_size, H * self.num_slots, bias=False)
        if self.qk_norm:
            eps = getattr(config, "rms_norm_eps", 1e-6)
            self.q_norm = HeadRMSNorm(D, eps)
            self.k_norm = HeadRMSNorm(D, eps)
        self.rotary_emb = RotaryTables(D, getattr(config, "rope_theta", 10000.0))

    def _fused_projection(self, x: torch.Tensor, with_gates: bool) -> torch.Tensor:
        """q | k | v | (gate logits) of `x` from ONE GEMM on the concatenated projection weights.  The concatenation is
        a copy held by the module (rebuilt when a weight's storage or version changes): inference memory for the
        attention projections doubles, four launches become one."""
        mods = [self.q_proj, self.k_proj, self.v_proj] + ([self.g_proj] if with_gates else [])
        key = tuple((m.weight.data_ptr(), m.weight._version, m.weight.dtype, m.weight.device,
                     None if m.bias is None else (m.bias.data_ptr(), m.bias._version)) for m in mods)
        if self._fused_key != key:
            w = torch.cat([m.weight.detach() for m in mods], 0)
            b = None
            if any(m.bias is not None for m in mods):
                b = torch.cat([m.bias.detach() if m.bias is not None else
                               torch.zeros(m.weight.shape[0], dtype=w.dtype, device=w.device) for m in mods], 0)
            self._fused_key, self._fused_wb = key, (w, b)
        w, b = self._fused_wb
        return F.linear(x, w, b)

    def record_decode_step(self, cache: NHARingCache, batch: int) -> "RecordedDecodeStep":
        """Record this block's single-token step on `cache` (which holds the prompt) into a HIP graph."""
        return RecordedDecodeStep(self, cache, batch)

    @property
    def is_nha_layer(self) -> bool:
        return self.window_size <= NHA_MAX_WINDOW

    def _tables(self, x, position_ids, position_embeddings, past, T):
        if position_embeddings is not None:
            cos, sin = position_embeddings
            return cos[:, -T:], sin[:, -T:]
        if position_ids is None:
            start = past.layer_tokens(self.layer_idx) if past is not None else 0
            position_ids = torch.arange(start, start + T, device=x.device)[None].expand(x.shape[0], T)
        return self.rotary_emb(x, position_ids)

    def forward(
        self,
        hidden_states: torch.Tensor,
        attention_mask: Optional[torch.Tensor] = None,
        position_ids: Optional[torch.LongTensor] = None,
        past_key_value: Optional[NHARingCache] = None,
        use_cache: bool = False,
        cache_position: Optional[torch.LongTensor] = None,
        position_embeddings: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
        **kwargs,
    ) -> Tuple[torch.Tensor, None]:
        if past_key_value is None:
            past_key_value = kwargs.get("past_key_values")
        if past_key_value is not None and not isinstance(past_key_value, NHARingCache):
            raise TypeError("the hybrid attention modules keep their decode state in an nha_amd.NHARingCache "
                            f"(NHARingCache.from_legacy_cache converts), got {type(past_key_value).__name__}")
        B, T, _ = hidden_states.shape
        HQ, H, D, M, W = self.num_heads, self.num_key_value_heads, self.head_dim, self.num_slots, self.window_size
        nha = self.is_nha_layer
        has_state = past_key_value is not None and past_key_value.has_ring(self.layer_idx)
        decode_step = (not self.training) and T == 1 and has_state
        mask2d = None
        if attention_mask is not None and attention_mask.dim() == 2:
            mask2d = attention_mask[:, -T:]
        # inference on the GPU: one GEMM for the q / k / v / gate projections and one launch for everything between
        # them and the attention op (q / k norm, gates, padding mask, rotary, contiguous operands)
        fused = (self.fuse_glue and not torch.is_grad_enabled() and hybrid_prologue_supported(hidden_states, D, M)
                 and (attention_mask is None or mask2d is not None)
                 and not (hidden_states.dtype == torch.float32 and torch.is_autocast_enabled()))
        if fused:
            y = self._fused_projection(hidden_states, with_gates=nha)
            o0, o1, o2 = HQ * D, HQ * D + H * D, HQ * D + 2 * H * D
            cos = sin = pos = inv = None
            if position_embeddings is not None:
                cos, sin = self._tables(hidden_states, position_ids, position_embeddings, past_key_value, T)
            else:                                  # the rows of the rotary tables are formed inside the glue launch
                pos, inv = position_ids, self.rotary_emb.inv_freq(hidden_states.device)
                if pos is None:
                    start = past_key_value.layer_tokens(self.layer_idx) if past_key_value is not None else 0
                    pos = torch.arange(start, start + T, device=hidden_states.device)[None].expand(B, T)
            q, sq, k, sk, v, g, s = nha_hybrid_prologue(
                y[..., :o0], y[..., o0:o1], y[..., o1:o2], y[..., o2:] if nha else None, cos, sin, positions=pos, inv_freq=inv,
                num_heads=HQ,
                num_kv_heads=H, head_dim=D, num_slots=M, q_weight=self.q_norm.weight if self.qk_norm else None,
                k_weight=self.k_norm.weight if self.qk_norm else None,
                eps=self.q_norm.variance_epsilon if self.qk_norm else 0.0, mask=mask2d,
                gate_logit_normalizer=self.gate_logit_normalizer, want_s=not decode_step)
        else:
            q = self.q_proj(hidden_states).view(B, T, HQ, D)
            k = self.k_proj(hidden_states).view(B, T, H, D)
            v = self.v_proj(hidden_states).view(B, T, H, D)
            if self.qk_norm:
                q, k = self.q_norm(q), self.k_norm(k)
            if nha:
                g = F.logsigmoid(self.g_proj(hidden_states).view(B, T, H, M)) / self.gate_logit_normalizer
            else:                                  # the slots of a full-attention layer never absorb anything
                g = torch.zeros(B, T, H, M, dtype=v.dtype, device=v.device)
            mask_t = None
            if attention_mask is not None:         # left padding: a padded token writes nothing into the slots
                if mask2d is not None:             # [batch, tokens]
                    mask_t = mask2d.to(v.dtype)[:, :, None, None]
                elif attention_mask.dim() == 4:
                    # [batch, 1, queries, tokens]: the reference multiplies its head-first [B, heads, T, dim] tensors by
                    # mask[:, :, :, -T:] (qwennha.py:133-136), so the last T columns broadcast over (token, dim);
                    # the same product on the token-major layout here
                    mask_t = attention_mask[:, :, :, -T:].to(v.dtype).transpose(1, 2)
                else:
                    raise ValueError("attention_mask must be [batch, tokens] or [batch, 1, queries, tokens], got "
                                     f"{tuple(attention_mask.shape)}")
                v = v * mask_t
            cos, sin = self._tables(v, position_ids, position_embeddings, past_key_value, T)
            sq, sk = rotate_half_apply(q, cos, sin), rotate_half_apply(k, cos, sin)
            dt = q.dtype
            if dt == torch.float32 and torch.is_autocast_enabled():
                dt = torch.get_autocast_gpu_dtype()
            q, k, v, g, sq, sk = (x.to(dt).contiguous() for x in (q, k, v, g, sq, sk))
            s = None
            if not decode_step:
                if nha:
                    s = 1 - torch.exp(g).to(g.dtype)
                    if mask_t is not None:
                        s = s * mask_t
                else:
                    s = torch.zeros_like(g)

        if decode_step:
            o = past_key_value.decode(self.layer_idx, q[:, 0], sq[:, 0], sk[:, 0], k[:, 0], v[:, 0], g[:, 0],
                                      scale=self.scaling, in_place_counters=self._recording)[:, None]
        else:
            if has_state:
                raise NotImplementedError("a multi-token step on top of a cached prompt is not supported "
                                          "(the reference's modules do not support it either)")
            want_state = use_cache or past_key_value is not None
            if not nha and not torch.is_grad_enabled() and zero_sink_attention_supported(sq, sk):
                # a full-attention layer at inference: the window loop alone, the sinks in its denominator (no state
                # pass, no slot branch, nothing to rescale); its slot states are zero by construction
                o = zero_sink_attention(sq, sk, v, W, M, scale=self.scaling)
                state = (None, None)
                if want_state:
                    state = (torch.zeros(B, H, D, M, dtype=torch.float32, device=o.device),
                             torch.zeros(B, H, M, D, dtype=torch.float32, device=o.device))
            elif nha and not torch.is_grad_enabled():
                o, state = fused_chunk_nha_prefill(q=q, k=k, v=v, rotary_q=sq, rotary_k=sk, s=s, g=g, window_size=W,
                                                   output_final_state=want_state, scale=self.scaling)
            else:
                out = chunk_nha(sq, sk, q, k, v, s, g, window_size_left=W - 1, window_size_right=0, gsa_kv_shift=W,
                                output_final_state=want_state, scale=self.scaling)
                o, lse_swa = out[0], out[1]
                state = out[3] if want_state else (None, None)
                if not nha:
                    # M zero-logit sinks were in the softmax at every t; the reference's window covers
                    # zero_sink_count(t) of them
                    if not torch.is_grad_enabled() and D in (64, 128, 256) and o.is_contiguous():
                        o = nha_zero_sink_rescale_(o, lse_swa.contiguous(), W, M)        # one launch, in place
                    else:
                        n0 = zero_sink_count(T, W, M, lse_swa.device)[None, :, None]
                        o = (o.to(torch.float32) * zero_sink_rescale(lse_swa, M, n0)[..., None]).to(o.dtype)
            if past_key_value is not None:
                past_key_value.prefill(self.layer_idx, sk, k, v, g, state, window_size=W, zero_state=not nha)
        o = self.o_proj(o.reshape(B, T, HQ * D))
        return o, None


class RecordedDecodeStep:
    """One decode step of an attention block as a HIP graph: `step(hidden [B,1,hidden], position_ids [B,1])` copies
    its arguments into the graph's input buffers `x` and `pos` (not when they are those buffers), replays the recorded launches (fused projection, glue, ring decode
    step, counter advance, output projection) and returns the graph's output buffer `[B,1,hidden]` (overwritten by
    the next step).  The host does no per-launch work, which is what a step of a few tens of microseconds of GPU
    time needs: the eager block spends more time issuing its launches than the GPU spends on them."""

    def __init__(self, block: "HybridNHAAttention", cache: NHARingCache, batch: int, mask_len: Optional[int] = None):
        if not cache.has_ring(block.layer_idx):
            raise ValueError("record a decode step after the prompt has been handed to the cache")
        p = block.q_proj.weight
        self.block, self.cache = block, cache
        self.x = torch.zeros(batch, 1, block.hidden_size, dtype=p.dtype, device=p.device)
        self.pos = torch.zeros(batch, 1, dtype=torch.long, device=p.device)
        st = cache.states[block.layer_idx]
        count0 = st.count.clone()
        snap = [t.clone() for t in (st.hk, st.hv, st.ring_k, st.ring_kg, st.ring_v, st.ring_g)]
        tokens = (cache._layer_tokens.get(block.layer_idx, 0), cache.former_tokens, cache._seen_tokens)
        # the launches are issued once eagerly on a side stream (lazy kernel set-up happens outside the recording),
        # then recorded; both runs are steps on the real cache, so its contents are put back afterwards
        side = torch.cuda.Stream(device=p.device)
        side.wait_stream(torch.cuda.current_stream(p.device))
        with torch.cuda.stream(side), torch.no_grad():
            self._run()
        torch.cuda.current_stream(p.device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.out = self._run()
        for t, s in zip((st.hk, st.hv, st.ring_k, st.ring_kg, st.ring_v, st.ring_g), snap):
            t.copy_(s)
        st.count.copy_(count0)
        cache._layer_tokens[block.layer_idx], cache.former_tokens, cache._seen_tokens = tokens
        self._count_ptr = st.count.data_ptr()

    def _run(self):
        self.block._recording = True
        try:
            return self.block(self.x, position_ids=self.pos, past_key_value=self.cache, use_cache=True)[0]
        finally:
            self.block._recording = False

    @torch.no_grad()
    def step(self, hidden_states: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
        if self.cache.states[self.block.layer_idx].count.data_ptr() != self._count_ptr:
            raise RuntimeError("the cache took an eager decode step since this step was recorded (the eager step trades "
                               "the ring's two counter arrays, the recording holds the address of one): record again")
        # a caller that fills the graph's own input buffers (`self.x`, `self.pos`) passes them back and saves the copies
        if hidden_states is not self.x:
            self.x.copy_(hidden_states)
        if position_ids is not self.pos:
            self.pos.copy_(position_ids)
        self.graph.replay()
        self.cache.note_step(self.block.layer_idx)
        return self.out


class Qwen3MoeNativeHybridAttention(HybridNHAAttention):
    """The MoE flavour's block: RMSNorm on every q and k head before rotary, optional projection biases
    (nha_fla/models/qwen3_moe_nha/qwennha.py:43-86)."""
    qk_norm = True


class LlamaNativeHybridAttention(HybridNHAAttention):
    """The dense flavour's block: bias-free projections, no q/k norm (nha_fla/models/llama3_nha/llamanha.py:30-62)."""
    qk_norm = False
