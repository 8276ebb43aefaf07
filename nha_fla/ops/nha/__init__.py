from nha_amd.ops import chunk_nha, fused_chunk_nha_prefill, fused_recurrent_nha, fused_recurrent_nha_decode

__all__ = ["chunk_nha", "fused_chunk_nha_prefill", "fused_recurrent_nha", "fused_recurrent_nha_decode"]
