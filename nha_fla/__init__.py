"""Import-path alias: `nha_fla.ops` / `nha_fla.layers.nha` resolve to the MI355X implementation in
`nha_amd`, so code written against the reference package imports unchanged."""
from nha_amd.ops import chunk_nha, fused_chunk_nha_prefill, fused_recurrent_nha, fused_recurrent_nha_decode

__all__ = ["chunk_nha", "fused_chunk_nha_prefill", "fused_recurrent_nha", "fused_recurrent_nha_decode"]
