"""NativeHybridAttention layer: the API shell of nha_fla/layers/nha.py:25-343 around chunk_nha.

Constructor arguments, parameter names (q_proj, k_proj, v_proj, f_proj, g_norm, o_proj, optional
q/k/v_conv1d), forward signature, return tuple and error behaviour follow the reference layer, so a
checkpoint of the reference loads here.  The op underneath is the HIP chunk_nha; k/v/s/g are handed
to it at the kv-head count (the reference repeats them to the q-head count first, :229-230).

The reference takes RMSNorm, RotaryEmbedding, ShortConvolution, the feature maps, rms_norm_linear
and the unpad helpers from flash-linear-attention, which is not vendored; they are restated here in
plain PyTorch from their published behaviour (elementwise / projection glue around the hot path).
The layer is trainable: chunk_nha carries its own backward, the glue around it is plain autograd.
The elementwise glue on either side of the op runs as two fused HIP launches, each with a fused
backward (nha_layer_prologue / nha_layer_epilogue); `fuse_glue = False` keeps the tensor-op chain.
"""
from __future__ import annotations

import warnings
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops as _ops
from .ops import chunk_nha, nha_layer_epilogue, nha_layer_prologue


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype)) if elementwise_affine else None
        self.register_parameter("bias", None)

    def forward(self, x):
        y = x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + self.eps)
        if self.weight is not None:
            y = y * self.weight.float()
        return y.to(x.dtype)


def rms_norm_linear(x, norm_weight, norm_bias, linear_weight, linear_bias, eps: float = 1e-5):
    """linear(rms_norm(x)) -- the fused epilogue of nha_fla/layers/nha.py:278."""
    y = x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + eps)
    if norm_weight is not None:
        y = y * norm_weight.float()
    if norm_bias is not None:
        y = y + norm_bias.float()
    return F.linear(y.to(linear_weight.dtype), linear_weight, linear_bias)


class SwishFeatureMap(nn.Module):
    def forward(self, x):
        return F.silu(x)


class ReLUFeatureMap(nn.Module):
    def forward(self, x):
        return F.relu(x)


class T2RFeatureMap(nn.Module):
    def __init__(self, head_dim: int, dot_dim: Optional[int] = None, bias: bool = False):
        super().__init__()
        self.layer = nn.Linear(head_dim, head_dim if dot_dim is None else dot_dim, bias=bias)

    def forward(self, x):
        return F.relu(self.layer(x))


class RotaryEmbedding(nn.Module):
    """Rotate-half RoPE over the whole head dim; positions restart at every cu_seqlens boundary."""

    def __init__(self, dim: int, base: float = 10000.0):
        super().__init__()
        self.dim, self.base = dim, base

    def inv_freq(self, device) -> torch.Tensor:
        return 1.0 / (self.base ** (torch.arange(0, self.dim, 2, device=device, dtype=torch.float32) / self.dim))

    def _tables(self, pos: torch.Tensor, dtype):
        inv = self.inv_freq(pos.device)
        fr = pos.float()[:, None] * inv[None, :]
        return fr.cos().to(dtype), fr.sin().to(dtype)

    def forward(self, q, k, seqlen_offset=0, cu_seqlens=None, max_seqlen=None):
        B, T = q.shape[0], q.shape[1]
        pos = torch.arange(T, device=q.device)
        if cu_seqlens is not None:
            cu = cu_seqlens.to(q.device).long()
            seq = torch.bucketize(pos, cu[1:], right=True)
            pos = pos - cu[seq]
        pos = pos + seqlen_offset
        cos, sin = self._tables(pos, q.dtype)                     # [T, dim/2]

        def rot(x):
            x1, x2 = x[..., : self.dim // 2], x[..., self.dim // 2: self.dim]
            c, s = cos[None, :, None, :], sin[None, :, None, :]
            out = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)
            return out if self.dim == x.shape[-1] else torch.cat([out, x[..., self.dim:]], dim=-1)

        return rot(q), rot(k)


class ShortConvolution(nn.Module):
    """Depthwise causal conv1d (kernel_size taps) + optional SiLU, restarting at cu_seqlens boundaries."""

    def __init__(self, hidden_size: int, kernel_size: int, bias: bool = False, activation: Optional[str] = "silu"):
        super().__init__()
        self.hidden_size, self.kernel_size, self.activation = hidden_size, kernel_size, activation
        self.weight = nn.Parameter(torch.empty(hidden_size, 1, kernel_size).uniform_(-kernel_size ** -0.5, kernel_size ** -0.5))
        self.bias = nn.Parameter(torch.zeros(hidden_size)) if bias else None

    def _final_state(self, x, cu_seqlens):
        return _short_conv_final_state(x, cu_seqlens, self.kernel_size)

    def forward(self, x, cache=None, output_final_state=False, cu_seqlens=None):
        B, T, Dm = x.shape
        if cache is None and _ops.short_conv_supported(x, self.weight):
            # a fresh sequence on the GPU: one HIP launch (taps, sequence restarts and SiLU fused)
            y = _ops.nha_short_conv(x, self.weight, self.bias, cu_seqlens=cu_seqlens,
                                    activation=self.activation if self.activation in ("silu", "swish") else None)
            return y, (self._final_state(x, cu_seqlens) if output_final_state else None)
        xs = x.transpose(1, 2)
        if cache is not None:
            xs = torch.cat([cache.to(xs.dtype), xs], dim=-1)
        else:
            xs = F.pad(xs, (self.kernel_size - 1, 0))
        if cu_seqlens is not None and cache is None:
            # zero the taps that would reach into the previous packed sequence
            pos = torch.arange(T, device=x.device)
            cu = cu_seqlens.to(x.device).long()
            local = pos - cu[torch.bucketize(pos, cu[1:], right=True)]
            y = torch.zeros_like(x.transpose(1, 2))
            xin = x.transpose(1, 2)
            for tap in range(self.kernel_size):
                back = self.kernel_size - 1 - tap
                shifted = F.pad(xin, (back, 0))[..., :T]
                y = y + shifted * (local >= back).to(x.dtype)[None, None, :] * self.weight[:, 0, tap][None, :, None]
            if self.bias is not None:
                y = y + self.bias[None, :, None]
        else:
            y = F.conv1d(xs, self.weight, self.bias, groups=Dm)
        final = None
        if output_final_state:
            if cu_seqlens is not None and cache is None:
                # one state per packed sequence: its last kernel_size - 1 inputs, zeros where it is shorter
                cu = cu_seqlens.to(x.device).long()
                ends = cu[1:]
                back = torch.arange(self.kernel_size - 1, 0, -1, device=x.device)              # W-1 .. 1
                idx = ends[:, None] - back[None, :]                                            # [N, W-1]
                ok = idx >= cu[:-1, None]
                gathered = x[0][idx.clamp(min=0)]                                              # [N, W-1, Dm]
                final = (gathered * ok[..., None].to(x.dtype)).transpose(1, 2).contiguous()     # [N, Dm, W-1]
            else:
                final = xs[..., -(self.kernel_size - 1):].contiguous()
        if self.activation in ("silu", "swish"):
            y = F.silu(y)
        return y.transpose(1, 2), final


def _short_conv_final_state(x, cu_seqlens, kernel_size):
    """The last kernel_size - 1 inputs of every sequence as [N, C, kernel_size - 1], zeros where it is shorter."""
    B, T, Dm = x.shape
    if cu_seqlens is None:
        xs = F.pad(x.transpose(1, 2), (kernel_size - 1, 0))
        return xs[..., -(kernel_size - 1):].contiguous()
    cu = cu_seqlens.to(x.device).long()
    back = torch.arange(kernel_size - 1, 0, -1, device=x.device)
    idx = cu[1:, None] - back[None, :]
    ok = idx >= cu[:-1, None]
    gathered = x[0][idx.clamp(min=0)]
    return (gathered * ok[..., None].to(x.dtype)).transpose(1, 2).contiguous()


def get_unpad_data(attention_mask: torch.Tensor):
    """Positions of the kept tokens in the flattened `[batch * seqlen]` order, the packed sequences'
    boundaries (int32, leading zero) and the longest sequence, from a `[batch, seqlen]` 0/1 mask."""
    kept = attention_mask.reshape(-1).nonzero().squeeze(-1)
    lengths = attention_mask.to(torch.int32).sum(dim=-1)
    bounds = torch.zeros(lengths.numel() + 1, dtype=torch.int32, device=attention_mask.device)
    bounds[1:] = lengths.cumsum(0)
    return kept, bounds, int(lengths.max())


def pad_input(x: torch.Tensor, indices: torch.Tensor, batch: int, seqlen: int):
    """Inverse of the unpadding: rows of the packed `x` go back to their `[batch, seqlen]` places, zeros elsewhere."""
    full = torch.zeros(batch * seqlen, *x.shape[1:], dtype=x.dtype, device=x.device)
    full.index_copy_(0, indices, x)
    return full.view(batch, seqlen, *x.shape[1:])


class NativeHybridAttention(nn.Module):
    """Drop-in for nha_fla.layers.nha.NativeHybridAttention (forward path)."""

    def __init__(
        self,
        mode: str = 'chunk',
        hidden_size: int = 1024,
        expand_k: float = 1.,
        expand_v: float = 1.,
        num_heads: int = 4,
        num_kv_heads: Optional[int] = None,
        use_short_conv: bool = False,
        conv_size: int = 4,
        conv_bias: bool = False,
        num_slots: Optional[int] = None,
        elementwise_affine: Optional[bool] = True,
        norm_eps: float = 1e-5,
        gate_logit_normalizer: int = 8,
        feature_map: str = 'swish',
        use_output_gate: bool = False,
        use_norm: bool = True,
        fuse_norm: bool = True,
        layer_idx: Optional[int] = None,
        scale: Optional[float] = 1.,
        window_size: int = 2048,
        rope_theta: float = 10000.,
        max_position_embeddings: Optional[int] = None,
        gsa_aux_loss_enable: bool = False,
        gsa_aux_loss_coeff: Optional[float] = None,
        gsa_aux_loss_target_ratio: float = 1.0,
        gsa_kv_shift: int = 0,
        **kwargs,
    ):
        super().__init__()
        if feature_map not in ('swish', 'relu', 't2r'):
            raise NotImplementedError(f"Feature map `{feature_map}` is not supported now.")
        if layer_idx is None:
            warnings.warn(f"{type(self).__name__} was built without `layer_idx`: a forward call that uses a cache "
                          "needs it to find this layer's states and will fail.")
        kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        groups = num_heads // kv_heads
        key_dim, value_dim = int(hidden_size * expand_k), int(hidden_size * expand_v)
        # the attributes the reference layer exposes (nha_fla/layers/nha.py:59-98), under the same names
        for name, value in dict(
                mode=mode, hidden_size=hidden_size, expand_k=expand_k, expand_v=expand_v, num_heads=num_heads,
                num_kv_heads=kv_heads, num_kv_groups=groups, key_dim=key_dim, value_dim=value_dim,
                key_dim_per_group=key_dim // groups, value_dim_per_group=value_dim // groups,
                head_k_dim=key_dim // num_heads, head_v_dim=value_dim // num_heads,
                use_short_conv=use_short_conv, conv_size=conv_size, conv_bias=conv_bias,
                gate_logit_normalizer=gate_logit_normalizer, use_output_gate=use_output_gate, use_norm=use_norm,
                fuse_norm=fuse_norm, scale=scale, window_size=window_size, rope_theta=rope_theta,
                max_position_embeddings=max_position_embeddings, gsa_aux_loss_enable=gsa_aux_loss_enable,
                gsa_aux_loss_coeff=gsa_aux_loss_coeff, gsa_aux_loss_target_ratio=gsa_aux_loss_target_ratio,
                gsa_kv_shift=gsa_kv_shift, layer_idx=layer_idx, norm_eps=norm_eps).items():
            setattr(self, name, value)
        self.num_slots = self.head_k_dim if num_slots is None else num_slots
        maps = {'swish': SwishFeatureMap, 'relu': ReLUFeatureMap, 't2r': lambda: T2RFeatureMap(self.head_k_dim, self.head_k_dim)}
        self.feature_map = maps[feature_map]()
        # projections: queries at the q-head count, keys / values / gate logits at the kv-head count
        widths = dict(q_proj=key_dim, k_proj=self.key_dim_per_group, v_proj=self.value_dim_per_group,
                      f_proj=kv_heads * self.num_slots)
        for name, width in widths.items():
            setattr(self, name, nn.Linear(hidden_size, width, bias=False))
        if use_short_conv:
            for name in ('q', 'k', 'v'):
                setattr(self, name + '_conv1d',
                        ShortConvolution(widths[name + '_proj'], conv_size, bias=conv_bias, activation='silu'))
        self.g_norm = RMSNorm(hidden_size, elementwise_affine, eps=norm_eps, dtype=torch.float32)
        self.o_proj = nn.Linear(value_dim, hidden_size, bias=False)
        self.rotary = RotaryEmbedding(dim=self.head_k_dim, base=rope_theta)
        self.fuse_glue = True
        self._inv_freq = None

    def _fused_glue(self, x: torch.Tensor) -> bool:
        """The fused prologue/epilogue kernels (differentiable) cover the swish, relu and identity
        feature maps in bf16 / fp32 on the GPU, with a value dimension the epilogue's backward takes."""
        return (self.fuse_glue and x.is_cuda and x.dtype in (torch.bfloat16, torch.float32)
                and isinstance(self.feature_map, (SwishFeatureMap, ReLUFeatureMap, type(None)))
                and self.o_proj.weight.dtype == x.dtype and self.head_k_dim % 2 == 0
                and self.value_dim % 8 == 0 and self.value_dim <= 8192)

    def forward(
        self,
        hidden_states: torch.Tensor,
        attention_mask: Optional[torch.Tensor] = None,
        past_key_values=None,
        use_cache: Optional[bool] = False,
        output_attentions: Optional[bool] = False,
        **kwargs,
    ) -> Tuple[torch.Tensor, None, object]:
        if attention_mask is not None:
            assert attention_mask.dim() == 2, (
                f"attention_mask must be the [batch, tokens] padding mask (1 = token, 0 = padding); got shape "
                f"{tuple(attention_mask.shape)}.  Per-query masks [batch, tokens, tokens] are not supported.")
        batch_size, q_len, _ = hidden_states.shape
        last_state = None
        if past_key_values is not None and len(past_key_values) > self.layer_idx:
            last_state = past_key_values[self.layer_idx]
        recurrent_state = last_state['recurrent_state'] if last_state is not None else None
        if q_len == 1 and last_state is not None:
            raise NotImplementedError(
                "this layer has no single-token step on top of a cached state (the reference layer raises here "
                "too); call it on the whole chunk, or decode with nha_amd.NHARingCache / the hybrid attention blocks")
        mode = self.mode
        cu_seqlens = kwargs.get('cu_seqlens')
        max_seqlen = kwargs.get('max_seqlen')
        indices = None
        if attention_mask is not None:
            indices, cu_seqlens, max_seqlen = get_unpad_data(attention_mask[:, -q_len:])
            hidden_states = hidden_states.reshape(batch_size * q_len, -1)[indices].unsqueeze(0)
        conv_state_q = conv_state_k = conv_state_v = None
        if self.use_short_conv:
            if last_state is not None:
                conv_state_q, conv_state_k, conv_state_v = last_state['conv_state']
            q, conv_state_q = self.q_conv1d(self.q_proj(hidden_states), conv_state_q, use_cache, cu_seqlens)
            k, conv_state_k = self.k_conv1d(self.k_proj(hidden_states), conv_state_k, use_cache, cu_seqlens)
            v, conv_state_v = self.v_conv1d(self.v_proj(hidden_states), conv_state_v, use_cache, cu_seqlens)
        else:
            q, k, v = self.q_proj(hidden_states), self.k_proj(hidden_states), self.v_proj(hidden_states)
        f = self.f_proj(hidden_states)
        q = q.unflatten(-1, (-1, self.head_k_dim))
        k = k.unflatten(-1, (-1, self.head_k_dim))
        v = v.unflatten(-1, (-1, self.head_v_dim))
        f = f.unflatten(-1, (-1, self.num_slots))
        seqlen_offset = 0
        if last_state is not None and 'seqlen_offset' in last_state:
            seqlen_offset = last_state['seqlen_offset']
        fused = self._fused_glue(q) and f.dtype == q.dtype
        if fused:
            if self._inv_freq is None or self._inv_freq.device != q.device:
                self._inv_freq = self.rotary.inv_freq(q.device)
            fm = None if self.feature_map is None else ('swish' if isinstance(self.feature_map, SwishFeatureMap) else 'relu')
            q_swa, k_swa, q_gsa, k_gsa, v, s, g = nha_layer_prologue(
                q, k, v, f, self._inv_freq, feature_map=fm, gate_logit_normalizer=self.gate_logit_normalizer,
                seqlen_offset=seqlen_offset, cu_seqlens=cu_seqlens)
        else:
            if self.feature_map is not None:
                q_gsa, k_gsa = self.feature_map(q), self.feature_map(k)
            else:
                q_gsa, k_gsa = q, k
            v = F.silu(v)
            f = F.logsigmoid(f) / self.gate_logit_normalizer
            s = (1 - f.exp()).to(f.dtype)
            g = f
            # rotary on the kv-head keys: identical across the heads of a group, so rotating before the
            # (implicit, in-kernel) group expansion equals the reference's repeat-then-rotate
            q_swa, k_swa = self.rotary(q, k, seqlen_offset=seqlen_offset, cu_seqlens=cu_seqlens)
        if mode == 'chunk':
            output, lse_swa, lse_gsa = chunk_nha(
                q_swa=q_swa, k_swa=k_swa, q_gsa=q_gsa, k_gsa=k_gsa, v=v, s=s, g=g,
                scale=self.scale,
                window_size_left=self.window_size,
                window_size_right=0,
                head_first=False,
                gsa_kv_shift=self.gsa_kv_shift,
                cu_seqlens=cu_seqlens,
                max_seqlen=max_seqlen,
            )
            if self.training:
                lse_max = torch.maximum(lse_swa, lse_gsa)
                w_swa, w_gsa = torch.exp(lse_swa - lse_max), torch.exp(lse_gsa - lse_max)
                self._store_compression_stats(w_swa, w_gsa)
                if self.gsa_aux_loss_enable:
                    output, gsa_aux_loss = self._apply_gsa_aux_loss(output, lse_swa, lse_gsa)
                    self._store_gsa_aux_loss(gsa_aux_loss)
        else:
            raise NotImplementedError(f"Not supported mode `{mode}`.")
        if past_key_values is not None:
            past_key_values.update(
                recurrent_state=recurrent_state,
                conv_state=(conv_state_q, conv_state_k, conv_state_v) if self.use_short_conv else None,
                layer_idx=self.layer_idx,
                offset=q_len,
            )
        o = output[:, :, :, :self.head_v_dim].flatten(-2)
        if fused:
            o = F.linear(nha_layer_epilogue(o, self.g_norm.weight, self.g_norm.bias, self.norm_eps),
                         self.o_proj.weight, self.o_proj.bias)
        else:
            o = rms_norm_linear(F.silu(o), self.g_norm.weight, self.g_norm.bias, self.o_proj.weight, self.o_proj.bias,
                                eps=self.norm_eps)
        if attention_mask is not None:
            o = pad_input(o.squeeze(0), indices, batch_size, q_len)
        return o, None, past_key_values

    def _apply_gsa_aux_loss(self, output: torch.Tensor, lse_swa: torch.Tensor, lse_gsa: torch.Tensor):
        """One-sided auxiliary loss on the slot branch's share of the softmax mass
        (nha_fla/layers/nha.py:300-317): binary cross-entropy of lse_gsa - stopgrad(lse_swa) against
        the target ratio; its gradient, scaled by the coefficient, rides on `output`."""
        delta = lse_gsa.float() - lse_swa.detach().float()
        target = torch.full_like(delta, self.gsa_aux_loss_target_ratio)
        loss = F.binary_cross_entropy_with_logits(delta, target, reduction='mean')
        return _AttachLossGrad.apply(output, loss, self.gsa_aux_loss_coeff), loss

    @torch.no_grad()
    def _store_gsa_aux_loss(self, gsa_aux_loss: torch.Tensor):
        if not hasattr(self, '_gsa_aux_losses'):
            self._gsa_aux_losses = []
        self._gsa_aux_losses.append(gsa_aux_loss.item())

    @torch.no_grad()
    def _store_compression_stats(self, w_swa: torch.Tensor, w_gsa: torch.Tensor):
        """GSA vs SWA share of the softmax mass (nha_fla/layers/nha.py:288-298)."""
        gsa_ratio = (w_gsa / (w_swa + w_gsa)).mean().item()
        if not hasattr(self, '_compression_stats'):
            self._compression_stats = []
        self._compression_stats.append({'gsa_ratio': gsa_ratio, 'swa_ratio': 1.0 - gsa_ratio})


class _AttachLossGrad(torch.autograd.Function):
    """Identity on `hidden` whose backward also sends `coeff` into `loss`, so that backpropagating
    the model's own objective trains the auxiliary loss with weight coeff
    (nha_fla/layers/nha.py:327-345)."""

    @staticmethod
    def forward(ctx, hidden, loss, coeff):
        ctx.coeff, ctx.like = coeff, loss
        return hidden.view_as(hidden)

    @staticmethod
    def backward(ctx, dhidden):
        if not ctx.coeff:
            return dhidden, None, None
        return dhidden, torch.full_like(ctx.like, ctx.coeff), None
