"""GPU parity of the prefill kernels (through the C ABI via nha_amd.ops) against the fp64 oracle."""
import itertools
import random

import numpy as np
import pytest
import torch

from oracle import nha_ref as R
from tests.util import assert_close, prefill_inputs

pytestmark = pytest.mark.gpu

KEYS = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")


def run_case(tag, d, *, wl, shift, dtype, impl, cu=None, scale=None, check_lse=True):
    from nha_amd import chunk_nha
    print("case", tag, dtype, impl, flush=True)
    c = {k: v.cuda() for k, v in d.items() if k in KEYS}
    h0 = d.get("h0")
    out = chunk_nha(*[c[k] for k in KEYS], cu_seqlens=None if cu is None else torch.tensor(cu, dtype=torch.int32).cuda(),
                    scale=scale, window_size_left=wl, window_size_right=0, gsa_kv_shift=shift,
                    initial_state=None if h0 is None else (h0[0].cuda(), h0[1].cuda()), output_final_state=True,
                    impl=impl)
    o, lse_swa, lse_gsa, (hkt, hvt) = out
    ro, rls, rlg, rhk, rhv = R.prefill_ref(*[d[k] for k in KEYS], window_size_left=wl, gsa_kv_shift=shift,
                                           cu_seqlens=cu, initial_state=h0, scale=scale)
    assert o.dtype == dtype and hkt.dtype == torch.float32
    assert_close(tag + " o", o, ro, dtype)
    assert_close(tag + " hk", hkt, rhk, dtype)
    assert_close(tag + " hv", hvt, rhv, dtype)
    if check_lse:
        assert_close(tag + " lse_swa", lse_swa, rls, dtype)
        assert_close(tag + " lse_gsa", lse_gsa, rlg, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_simple_reference_grid(dtype):
    """The reference's prefill grid (scripts/verify_opt_parity.py:437-444), both call conventions."""
    seed = 3000
    for T, B, W, M in itertools.product((63, 128, 257, 1000), (1, 4), (32, 64), (16, 64)):
        if T == 1000 and B == 4 and M == 16:
            continue
        K = V = 64
        H, NG = 2, 4
        d = prefill_inputs(seed, B, T, H * NG, H, K, V, M, dtype=dtype, with_state=(T == 128))
        seed += 1
        run_case(f"pf_t{T}_b{B}_w{W}_m{M} shifted", d, wl=W - 1, shift=W, dtype=dtype, impl="simple")
        if B == 1:
            run_case(f"pf_t{T}_b{B}_w{W}_m{M} layer", d, wl=W, shift=0, dtype=dtype, impl="simple")


def test_simple_fp32_config1():
    """B=1, T=512, H=4, D=64, M=64, W=64, fp32, q,k,v ~ N(0,1)/sqrt(D), gates logsigmoid(N(0,1))."""
    d = prefill_inputs(0, 1, 512, 4, 4, 64, 64, 64, dtype=torch.float32, gate_div=1.0, qk_scale=64 ** -0.5)
    run_case("cfg1 shifted", d, wl=63, shift=64, dtype=torch.float32, impl="simple")
    run_case("cfg1 layer", d, wl=64, shift=0, dtype=torch.float32, impl="simple")


def test_simple_odd_shapes_and_unbounded_window():
    d = prefill_inputs(5, 2, 150, 6, 3, 24, 40, 10, dtype=torch.float32, with_state=True)
    run_case("odd", d, wl=-1, shift=3, dtype=torch.float32, impl="simple", scale=0.3)
    d = prefill_inputs(6, 1, 70, 2, 2, 16, 16, 5, dtype=torch.float32, gate_div=1.0, gate_mean=-6.0)
    d["g"] = d["g"] * 0 - 10.0
    d["s"] = 1 - d["g"].exp()
    run_case("strong gates", d, wl=9, shift=0, dtype=torch.float32, impl="simple")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_simple_varlen(dtype):
    """Varlen lists of the reference's stress test (tests/test_varlen.py:60-73), scaled to what
    the CPU recurrence finishes in seconds, incl. sequences of length 1 and 2 and shorter than the shift."""
    random.seed(0)
    for li, lens in enumerate([[128, 64, 200, 10], [300, 1, 129, 2, 64], [random.randint(1, 100) for _ in range(40)],
                               [1, 200, 3, 50, 4, 130, 2, 7]]):
        cu = [0] + list(np.cumsum(lens))
        T, H, NG, K, V, M = cu[-1], 2, 2, 64, 64, 16
        d = prefill_inputs(40 + li, 1, T, H * NG, H, K, V, M, dtype=dtype, with_state=True, N=len(lens))
        run_case(f"varlen{li} shifted", d, wl=31, shift=32, dtype=dtype, impl="simple", cu=cu)
        run_case(f"varlen{li} layer", d, wl=32, shift=0, dtype=dtype, impl="simple", cu=cu)


def test_fused_chunk_prefill_api():
    from nha_amd import fused_chunk_nha_prefill
    d = prefill_inputs(11, 2, 200, 8, 2, 64, 64, 64, dtype=torch.bfloat16, with_state=True)
    c = {k: v.cuda() for k, v in d.items() if k in KEYS}
    W = 64
    o, (hkt, hvt) = fused_chunk_nha_prefill(q=c["q_gsa"], k=c["k_gsa"], v=c["v"], rotary_q=c["q_swa"], rotary_k=c["k_swa"],
                                            window_size=W, s=c["s"], g=c["g"],
                                            initial_state=(d["h0"][0].cuda(), d["h0"][1].cuda()), output_final_state=True)
    ro, _, _, rhk, rhv = R.prefill_ref(*[d[k] for k in KEYS], window_size_left=W - 1, gsa_kv_shift=W, initial_state=d["h0"])
    assert_close("fused o", o, ro, torch.bfloat16)
    assert_close("fused hk", hkt, rhk, torch.bfloat16)
    o2, st = fused_chunk_nha_prefill(q=c["q_gsa"], k=c["k_gsa"], v=c["v"], rotary_q=c["q_swa"], rotary_k=c["k_swa"],
                                     window_size=W, s=c["s"], g=c["g"])
    assert st == (None, None)


def test_api_errors():
    from nha_amd import chunk_nha
    d = prefill_inputs(1, 1, 32, 2, 2, 16, 16, 8)
    c = [d[k].cuda() for k in KEYS]
    with pytest.raises(DeprecationWarning):
        chunk_nha(*c, head_first=True)
    with pytest.raises(AssertionError):
        chunk_nha(c[0][0], *c[1:])
    with pytest.raises(RuntimeError):
        chunk_nha(*[d[k] for k in KEYS])                     # CPU tensors: no fallback
    with pytest.raises(ValueError):
        chunk_nha(*[x.expand(2, -1, -1, -1) for x in c], cu_seqlens=torch.tensor([0, 32], dtype=torch.int32).cuda())


@pytest.mark.gpu
def test_varlen_tables_on_the_device_bit_exact_vs_oracle():
    """The chunk tables the kernels consume (built by the host-side C entry points, copied to the GPU by
    prefill_tables) equal the integer oracle bit for bit: the reference test's length lists
    (tests/test_varlen.py:60-73 of the reference) and the benchmark's 32768-token varlen draw."""
    import random
    import numpy as np
    import bench
    from nha_amd.ops import prefill_tables
    from oracle import varlen_index as VI
    random.seed(0)
    cases = [[128] * 4, [128, 64, 200, 10], [4096, 2048, 1, 1024, 2], [random.randint(1, 100) for _ in range(256)],
             [1, 2000, 3, 50, 4, 3000, 2, 7], bench.workload_lengths(torch, bench.WORKLOADS["cfg3"])]
    for lens in cases:
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        cu_d, idx_d, off_d, NT = prefill_tables(cu, torch.device("cuda:0"))
        ridx, roff = VI.chunk_tables_brute(cu.tolist(), 64)
        assert cu_d.dtype == idx_d.dtype == off_d.dtype == torch.int32
        assert torch.equal(cu_d.cpu(), torch.from_numpy(cu))
        assert torch.equal(idx_d.cpu(), torch.from_numpy(ridx))
        assert torch.equal(off_d.cpu(), torch.from_numpy(roff))
        assert NT == ridx.shape[0]
