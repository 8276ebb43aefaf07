"""Integer oracle for the varlen (cu_seqlens) index math of the NHA prefill path.

TEST INFRASTRUCTURE ONLY (used by tests/ and smoke()); the shipped package never imports it.

The reference derives these tables with flash-linear-attention's ``prepare_chunk_indices``
(un-vendored, unpinned dependency; setup.py:35) and consumes them as
``i_n, i_t = chunk_indices[2*i], chunk_indices[2*i+1]; bos, eos = cu_seqlens[i_n], cu_seqlens[i_n+1]``
(nha_fla/ops/nha_naive/chunk.py:59-64, :131-134, :644-649) with ``NT = len(chunk_indices)`` (:558).
The slot-branch shift is nha_fla/ops/nha/chunk.py:53-78 and the window is flash-attn's causal
``window_size_left`` (key j visible to query i iff i - wl <= j <= i, same sequence).

Two independent statements are given: closed forms (``*_closed``) and a brute-force search over
tokens (``*_brute``); tests/test_varlen_index.py checks one against the other on exhaustive
small cases and on the reference's own stress lists (tests/test_varlen.py:60-73).
"""
from __future__ import annotations

import numpy as np


def chunk_size_for(total_tokens: int) -> int:
    """``min(64, max(16, next_pow2(T)))`` -- nha_fla/ops/nha/chunk.py:155."""
    p = 1
    while p < total_tokens:
        p *= 2
    return min(64, max(16, p))


def chunk_tables_closed(cu_seqlens, bt: int):
    """(chunk_indices int32 [NT,2], chunk_offsets int32 [N+1]) in sequence-major order."""
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    lens = cu[1:] - cu[:-1]
    nchunks = (lens + bt - 1) // bt
    offs = np.concatenate([[0], np.cumsum(nchunks)]).astype(np.int32)
    seq = np.repeat(np.arange(len(lens)), nchunks)
    it = np.arange(int(offs[-1])) - np.repeat(offs[:-1].astype(np.int64), nchunks)
    idx = np.stack([seq, it], axis=1).astype(np.int32).reshape(-1, 2)
    return idx, offs


def chunk_tables_brute(cu_seqlens, bt: int):
    """Same tables by walking every token."""
    cu = [int(c) for c in cu_seqlens]
    rows, offs = [], [0]
    for n in range(len(cu) - 1):
        seen = set()
        for t in range(cu[n], cu[n + 1]):
            c = (t - cu[n]) // bt
            if c not in seen:
                seen.add(c)
                rows.append((n, c))
        offs.append(len(rows))
    return np.asarray(rows, dtype=np.int32).reshape(-1, 2), np.asarray(offs, dtype=np.int32)


def token_tables_closed(cu_seqlens, wl: int, shift: int):
    """Per global token t: (seq, bos, lo, hi, gsa_src).  lo/hi = first/last visible window key
    (global index); gsa_src = global index of the token written to the slots at step t, or -1
    for a zero row (nha_fla/ops/nha/chunk.py:72-77: a sequence no longer than ``shift`` stays
    all-zero)."""
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    lens = cu[1:] - cu[:-1]
    T = int(cu[-1])
    seq = np.repeat(np.arange(len(lens)), lens)
    bos = cu[:-1][seq]
    t = np.arange(T)
    lo = bos.copy() if wl < 0 else np.maximum(bos, t - wl)
    hi = t.copy()
    src = np.where((t - shift >= bos) & (lens[seq] > shift), t - shift, -1) if shift > 0 else t.copy()
    return (seq.astype(np.int32), bos.astype(np.int32), lo.astype(np.int32),
            hi.astype(np.int32), src.astype(np.int32))


def token_tables_brute(cu_seqlens, wl: int, shift: int):
    cu = [int(c) for c in cu_seqlens]
    seq, bos, lo, hi, src = [], [], [], [], []
    for n in range(len(cu) - 1):
        st, en = cu[n], cu[n + 1]
        # the shifted copy of nha_fla/ops/nha/chunk.py:70-77, tracked by source index
        y = [-1] * (en - st)
        if shift <= 0:
            y = list(range(st, en))
        elif en - st > shift:
            y[shift:] = list(range(st, en - shift))
        for t in range(st, en):
            vis = [j for j in range(st, en) if j <= t and (wl < 0 or j >= t - wl)]
            seq.append(n); bos.append(st); lo.append(min(vis)); hi.append(max(vis)); src.append(y[t - st])
    f = lambda a: np.asarray(a, dtype=np.int32)
    return f(seq), f(bos), f(lo), f(hi), f(src)
