"""nha_amd: MI355X-native implementation of NHA's fused hybrid-attention hot path.

Public surface mirrors the reference's op API (see nha_amd/ops.py) plus the resident ring-buffer
decode state (nha_amd/ring.py) and the per-layer cache around it (nha_amd/cache.py).  Everything computes through libnha_hip.so (nha_amd/csrc)."""
from ._lib import NhaError
from .ops import (chunk_nha, fused_chunk_nha_prefill, fused_recurrent_nha, fused_recurrent_nha_decode, release_workspaces,
                  zero_sink_attention)
from .custom_ops import chunk_nha_packed      # also registers torch.ops.nha_amd.prefill_fwd / prefill_bwd
from .ring import NHARingState, ring_decode_step
from .cache import NHACache, NHARingCache
from .hybrid import (HybridNHAConfig, LlamaNativeHybridAttention, Qwen3MoeNativeHybridAttention, init_gates_from_keys,
                     pool_k_to_g)

__all__ = ["chunk_nha", "chunk_nha_packed", "fused_chunk_nha_prefill", "fused_recurrent_nha", "fused_recurrent_nha_decode",
           "NHARingState", "ring_decode_step", "NHARingCache", "NHACache", "NhaError", "HybridNHAConfig",
           "LlamaNativeHybridAttention", "Qwen3MoeNativeHybridAttention", "init_gates_from_keys", "pool_k_to_g", "release_workspaces", "zero_sink_attention"]
