"""nha_prefill_fwd_noalloc (the entry point that allocates nothing: its workspace is an array inside
the library) against nha_prefill_fwd on the same inputs, through the C ABI: two calls in a row, the
second with a smaller input, so the second finds the first's leftovers in the shared array."""
import ctypes as C

import numpy as np
import pytest
import torch

from nha_amd import _lib
from nha_amd.ops import _ptr, prefill_tables
from tests.util import prefill_inputs

pytestmark = pytest.mark.gpu
KEYS = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")


def _args(d, lens, HQ, H, D, wl, shift, dtype, outs):
    dev = torch.device("cuda:0")
    T = sum(lens)
    xs = [d[k].reshape(T, *d[k].shape[2:]).contiguous().to(dev) for k in KEYS]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cu_d, idx_d, off_d, NT = prefill_tables(cu, dev)
    N = len(lens)
    o = torch.zeros(T, HQ, D, dtype=dtype, device=dev)
    ls = torch.zeros(T, HQ, dtype=torch.float32, device=dev)
    lg = torch.zeros_like(ls)
    hkt = torch.zeros(N, H, D, 64, dtype=torch.float32, device=dev)
    hvt = torch.zeros(N, H, 64, D, dtype=torch.float32, device=dev)
    h0k, h0v = (t.to(dev).float().contiguous() for t in d["h0"])
    a = _lib.NhaPrefillArgs()
    a.q_swa, a.k_swa, a.q_gsa, a.k_gsa, a.v, a.s, a.g = (_ptr(x) for x in xs)
    a.o, a.lse_swa, a.lse_gsa, a.hkt, a.hvt, a.h0k, a.h0v = _ptr(o), _ptr(ls), _ptr(lg), _ptr(hkt), _ptr(hvt), _ptr(h0k), _ptr(h0v)
    a.cu_seqlens, a.chunk_indices, a.chunk_offsets = _ptr(cu_d), _ptr(idx_d), _ptr(off_d)
    a.T_tot, a.N, a.NT, a.HQ, a.H, a.K, a.V, a.M = T, N, NT, HQ, H, D, D, 64
    a.wl, a.shift, a.scale = wl, shift, D ** -0.5
    a.dtype = _lib.NHA_DTYPE_BF16 if dtype == torch.bfloat16 else _lib.NHA_DTYPE_F32
    a.impl = _lib.NHA_IMPL_AUTO
    a.stream = torch.cuda.current_stream(dev).cuda_stream
    outs.append((xs, cu_d, idx_d, off_d, h0k, h0v))   # keep the operands alive
    return a, (o, ls, lg, hkt, hvt)


@pytest.mark.parametrize("dtype,HQ,H,D", [(torch.bfloat16, 8, 2, 128), (torch.bfloat16, 4, 4, 256), (torch.float32, 4, 2, 64)])
def test_noalloc_matches_the_allocating_entry_point(dtype, HQ, H, D):
    lib = _lib.load()
    keep = []
    for seed, lens in ((11, [700, 130, 64, 1]), (12, [200, 65])):   # the second call is the smaller one
        T = sum(lens)
        d = prefill_inputs(seed, 1, T, HQ, H, D, D, 64, dtype=dtype, with_state=True, N=len(lens))
        a, ref = _args(d, lens, HQ, H, D, 63, 64, dtype, keep)
        nbytes = lib.nha_prefill_scratch_bytes(C.byref(a))
        assert 0 < nbytes <= _lib.NHA_NOALLOC_SCRATCH_BYTES
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0")
        a.scratch, a.scratch_bytes = _ptr(ws), nbytes
        _lib.check(lib.nha_prefill_fwd(C.byref(a)))
        b, got = _args(d, lens, HQ, H, D, 63, 64, dtype, keep)
        b.scratch, b.scratch_bytes = None, 0
        _lib.check(lib.nha_prefill_fwd_noalloc(C.byref(b)))
        torch.cuda.synchronize()
        for name, x, y in zip(("o", "lse_swa", "lse_gsa", "hkt", "hvt"), got, ref):
            assert torch.equal(x, y), f"{name} differs between the two entry points (seed {seed}, {dtype}, D={D})"
            assert torch.isfinite(x.float()).all()


def test_noalloc_rejects_what_does_not_fit():
    lib = _lib.load()
    keep = []
    lens = [4096] * 4
    d = prefill_inputs(13, 1, sum(lens), 8, 8, 128, 128, 64, dtype=torch.bfloat16, with_state=True, N=len(lens))
    a, _ = _args(d, lens, 8, 8, 128, 63, 64, torch.bfloat16, keep)
    assert lib.nha_prefill_scratch_bytes(C.byref(a)) > _lib.NHA_NOALLOC_SCRATCH_BYTES
    rc = lib.nha_prefill_fwd_noalloc(C.byref(a))
    assert rc == _lib.NHA_ERR_SCRATCH
    assert b"nha_prefill_fwd_noalloc" in lib.nha_last_error()
