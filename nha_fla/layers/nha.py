from nha_amd.layer import NativeHybridAttention

__all__ = ["NativeHybridAttention"]
