"""Import-path aliases for the hybrid decoder models' attention blocks and their cache."""
from nha_amd.cache import NHACache
from nha_amd.hybrid import LlamaNativeHybridAttention, Qwen3MoeNativeHybridAttention

__all__ = ["NHACache", "LlamaNativeHybridAttention", "Qwen3MoeNativeHybridAttention"]
