from nha_amd.ops import fused_chunk_nha_prefill

__all__ = ["fused_chunk_nha_prefill"]
