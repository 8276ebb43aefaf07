"""The registered operators torch.ops.nha_amd.prefill_fwd / prefill_bwd: schema and shape functions on the CPU
(meta tensors), and on the GPU torch.library.opcheck, equality with chunk_nha and a full-graph trace."""
import pytest
import torch

import nha_amd  # noqa: F401  (registers the operators)
from tests.util import randn


def _meta(*shape, dtype=torch.bfloat16):
    return torch.empty(*shape, dtype=dtype, device="meta")


def test_operator_schemas():
    fwd = str(torch.ops.nha_amd.prefill_fwd.default._schema)
    bwd = str(torch.ops.nha_amd.prefill_bwd.default._schema)
    assert fwd.startswith("nha_amd::prefill_fwd(Tensor q_swa, Tensor k_swa, Tensor q_gsa, Tensor k_gsa, Tensor v, Tensor s, Tensor g, Tensor cu_seqlens")
    assert "Tensor? h0k, Tensor? h0v, bool want_state) -> (Tensor, Tensor, Tensor, Tensor, Tensor)" in fwd
    assert bwd.count("Tensor?") == 6 and bwd.endswith("-> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)")


@pytest.mark.parametrize("want_state", [False, True])
def test_shape_functions_on_meta_tensors(want_state):
    T, HQ, H, K, V, M = 300, 8, 2, 64, 64, 64
    cu = torch.tensor([0, 100, 300], dtype=torch.int32)
    xs = (_meta(T, HQ, K), _meta(T, H, K), _meta(T, HQ, K), _meta(T, H, K), _meta(T, H, V), _meta(T, H, M), _meta(T, H, M))
    o, ls, lg, hkt, hvt = torch.ops.nha_amd.prefill_fwd(*xs, cu, 63, 64, 0.125, None, None, want_state)
    assert o.shape == (T, HQ, V) and o.dtype == torch.bfloat16
    assert ls.shape == lg.shape == (T, HQ) and ls.dtype == torch.float32
    assert (hkt.shape, hvt.shape) == (((2, H, K, M), (2, H, M, V)) if want_state else ((0,), (0,)))
    grads = torch.ops.nha_amd.prefill_bwd(*xs, o, ls, lg, _meta(T, HQ, V), cu, 63, 64, 0.125, None, None, None, None, None,
                                          None, want_state)
    assert [g.shape for g in grads[:7]] == [x.shape for x in xs]
    assert grads[7].shape == ((2, H, K, M) if want_state else (0,))


def _inputs(seed, T, HQ, H, D, M, dev):
    gen = torch.Generator().manual_seed(seed)
    dt = torch.bfloat16
    xs = [randn(gen, T, HQ, D, dtype=dt), randn(gen, T, H, D, dtype=dt), randn(gen, T, HQ, D, dtype=dt), randn(gen, T, H, D, dtype=dt),
          randn(gen, T, H, D, dtype=dt), randn(gen, T, H, M, dtype=dt, scale=0.5),
          torch.nn.functional.logsigmoid(torch.randn(T, H, M, generator=gen)).to(dt)]
    return [x.to(dev).requires_grad_(True) for x in xs]


@pytest.mark.gpu
def test_opcheck_and_equality_with_chunk_nha():
    from nha_amd import chunk_nha, chunk_nha_packed
    T, HQ, H, D, M = 200, 4, 2, 64, 64
    cu = torch.tensor([0, 70, 200], dtype=torch.int32)
    xs = _inputs(11, T, HQ, H, D, M, "cuda")
    torch.library.opcheck(torch.ops.nha_amd.prefill_fwd, (*xs, cu, 31, 32, D ** -0.5, None, None, True))
    o, ls, lg, (hk, hv) = chunk_nha_packed(*xs, cu, window_size_left=31, gsa_kv_shift=32, output_final_state=True)
    do = torch.randn_like(o)
    (o.float() * do.float()).sum().backward()
    g1 = [x.grad.clone() for x in xs]
    for x in xs:
        x.grad = None
    o2, ls2, lg2, (hk2, hv2) = chunk_nha(*[x[None] for x in xs], cu_seqlens=cu.cuda(), window_size_left=31, gsa_kv_shift=32,
                                         output_final_state=True)
    (o2[0].float() * do.float()).sum().backward()
    assert torch.equal(o, o2[0]) and torch.equal(ls, ls2[0]) and torch.equal(hk, hk2) and torch.equal(hv, hv2)
    for a, x in zip(g1, xs):
        assert torch.equal(a, x.grad)


@pytest.mark.gpu
def test_full_graph_trace():
    """A function around the operator is captured as one graph (no graph break) and runs to the eager result."""
    from nha_amd import chunk_nha_packed
    T, HQ, H, D, M = 128, 4, 2, 64, 64
    cu = torch.tensor([0, 128], dtype=torch.int32)
    xs = _inputs(12, T, HQ, H, D, M, "cuda")

    def f(*a):
        o, ls, lg = chunk_nha_packed(*a, cu, window_size_left=15, gsa_kv_shift=16)
        return o.float().square().sum() + ls.sum()

    ref = f(*xs)
    ref.backward()
    gref = [x.grad.clone() for x in xs]
    for x in xs:
        x.grad = None
    out = torch.compile(f, backend="aot_eager", fullgraph=True)(*xs)
    out.backward()
    assert torch.allclose(out, ref)
    for a, x in zip(gref, xs):
        assert torch.equal(a, x.grad)


@pytest.mark.gpu
def test_operator_carries_initial_and_final_states():
    """Initial states in, final states out, cotangents on both: the operator's autograd formula against chunk_nha's."""
    from nha_amd import chunk_nha, chunk_nha_packed
    T, HQ, H, D, M = 260, 4, 2, 64, 64
    cu = torch.tensor([0, 100, 260], dtype=torch.int32)
    xs = _inputs(13, T, HQ, H, D, M, "cuda")
    gen = torch.Generator().manual_seed(14)
    h0k = (torch.randn(2, H, D, M, generator=gen) * 0.1).cuda().requires_grad_(True)
    h0v = (torch.randn(2, H, M, D, generator=gen) * 0.1).cuda().requires_grad_(True)
    do = torch.randn(T, HQ, D, generator=gen).cuda().to(torch.bfloat16)
    dk, dv = torch.randn(2, H, D, M, generator=gen).cuda(), torch.randn(2, H, M, D, generator=gen).cuda()

    def run(fn, packed):
        for x in (*xs, h0k, h0v):
            x.grad = None
        if packed:
            o, ls, lg, (hk, hv) = fn(*xs, cu, window_size_left=40, gsa_kv_shift=0, initial_state=(h0k, h0v), output_final_state=True)
        else:
            o, ls, lg, (hk, hv) = fn(*[x[None] for x in xs], cu_seqlens=cu.cuda(), window_size_left=40, gsa_kv_shift=0,
                                     initial_state=(h0k, h0v), output_final_state=True)
            o, ls, lg = o[0], ls[0], lg[0]
        ((o.float() * do.float()).sum() + (hk * dk).sum() + (hv * dv).sum() + 0.3 * ls.sum() - 0.2 * lg.sum()).backward()
        return [o, ls, lg, hk, hv] + [x.grad.clone() for x in (*xs, h0k, h0v)]

    a, b = run(chunk_nha_packed, True), run(chunk_nha, False)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
