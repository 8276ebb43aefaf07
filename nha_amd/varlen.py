"""Host-side varlen chunk tables (bit-exact integer math, done by the C ABI's
nha_varlen_indices; replaces fla's prepare_chunk_indices as consumed at
nha_fla/ops/nha_naive/chunk.py:59-64, :557-558)."""
from __future__ import annotations

import numpy as np

from . import _lib

CHUNK = 64   # the kernels' chunk size (nha_fla/ops/nha/chunk.py:155 gives 64 whenever T_tot > 32)


def chunk_tables(cu_seqlens_host, chunk_size: int = CHUNK):
    """cu_seqlens (host int sequence / numpy, length N+1) -> (chunk_indices int32 [NT,2],
    chunk_offsets int32 [N+1]) as numpy arrays."""
    lib = _lib.load()
    cu = np.ascontiguousarray(np.asarray(cu_seqlens_host, dtype=np.int32))
    if cu.ndim != 1 or cu.size < 2:
        raise ValueError("cu_seqlens must be a 1-D sequence of length N+1 >= 2")
    n = cu.size - 1
    nt = lib.nha_varlen_num_chunks(cu.ctypes.data, n, chunk_size)
    if nt < 0:
        _lib.check(nt)
    idx = np.empty((nt, 2), dtype=np.int32)
    off = np.empty(n + 1, dtype=np.int32)
    _lib.check(lib.nha_varlen_indices(cu.ctypes.data, n, chunk_size, idx.ctypes.data, off.ctypes.data))
    return idx, off
