from nha_amd.hybrid import LlamaNativeHybridAttention

__all__ = ["LlamaNativeHybridAttention"]
