from .qwennha import Qwen3MoeNativeHybridAttention  # noqa: F401
