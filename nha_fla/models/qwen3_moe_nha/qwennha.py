from nha_amd.hybrid import Qwen3MoeNativeHybridAttention

__all__ = ["Qwen3MoeNativeHybridAttention"]
