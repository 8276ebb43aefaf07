from .llamanha import LlamaNativeHybridAttention  # noqa: F401
