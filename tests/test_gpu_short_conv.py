"""GPU parity of nha_short_conv (forward and backward, through the C ABI) against an fp64 restatement of the
depthwise causal convolution the layer applies to its projections (nha_fla/layers/nha.py:186-206):
y[t][c] = act(b[c] + sum_j w[c][j] x[t - (KS-1) + j][c]), taps before the start of t's sequence zero.
The restatement is pinned by torch's own grouped conv1d on a single sequence."""
import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu


def conv_ref(x, w, b, cu, act):
    """x [T, C] fp64, w [C, KS], b [C] or None, cu: list of boundaries."""
    T, Cn = x.shape
    KS = w.shape[1]
    y = torch.zeros_like(x)
    for s0, s1 in zip(cu[:-1], cu[1:]):
        for j in range(KS):
            back = KS - 1 - j
            if s1 - s0 > back:
                y[s0 + back:s1] += x[s0:s1 - back] * w[:, j]
    if b is not None:
        y = y + b
    return F.silu(y) if act else y


def test_restatement_matches_grouped_conv1d():
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(37, 16, generator=gen, dtype=torch.float64)
    w = torch.randn(16, 4, generator=gen, dtype=torch.float64)
    b = torch.randn(16, generator=gen, dtype=torch.float64)
    ref = F.conv1d(F.pad(x.t()[None], (3, 0)), w[:, None, :], b, groups=16)[0].t()
    assert torch.allclose(conv_ref(x, w, b, [0, 37], False), ref, atol=1e-12)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("KS,Cn,lens,act,bias", [(4, 64, (300,), True, False), (4, 256, (5, 1, 130, 2, 260), True, True),
                                                 (3, 72, (129, 127), False, True), (2, 8, (3, 200), True, False)])
def test_short_conv_forward_backward(dtype, KS, Cn, lens, act, bias):
    from nha_amd.ops import nha_short_conv
    gen = torch.Generator().manual_seed(100 + KS + Cn)
    T = sum(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    x = randn(gen, 1, T, Cn, dtype=dtype)
    w = randn(gen, Cn, 1, KS, dtype=dtype, scale=0.5)
    b = randn(gen, Cn, dtype=dtype, scale=0.5) if bias else None
    dy = randn(gen, 1, T, Cn, dtype=dtype)
    xd, wd = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    bd = None if b is None else b.cuda().requires_grad_(True)
    cu_d = torch.tensor(cu, dtype=torch.int32, device="cuda") if len(lens) > 1 else None
    y = nha_short_conv(xd, wd, bd, cu_seqlens=cu_d, activation="silu" if act else None)
    y.backward(dy.cuda())
    xr, wr = x[0].double().requires_grad_(True), w[:, 0].double().requires_grad_(True)
    br = None if b is None else b.double().requires_grad_(True)
    yr = conv_ref(xr, wr, br, cu, act)
    yr.backward(dy[0].double())
    assert_close("short conv y", y[0], yr.detach(), dtype)
    assert_close("short conv dx", xd.grad[0], xr.grad, dtype)
    assert_close("short conv dw", wd.grad[:, 0], wr.grad, dtype)
    if b is not None:
        assert_close("short conv db", bd.grad, br.grad, dtype)


def test_short_conv_fixed_length_batch():
    """[B, T, C] without cu_seqlens: every batch row is its own sequence."""
    from nha_amd.ops import nha_short_conv
    gen = torch.Generator().manual_seed(7)
    B, T, Cn, KS = 3, 150, 128, 4
    x = randn(gen, B, T, Cn, dtype=torch.bfloat16)
    w = randn(gen, Cn, 1, KS, dtype=torch.bfloat16, scale=0.5)
    xd = x.cuda().requires_grad_(True)
    y = nha_short_conv(xd, w.cuda(), None)
    y.float().sum().backward()
    cu = [i * T for i in range(B + 1)]
    xr = x.reshape(B * T, Cn).double().requires_grad_(True)
    yr = conv_ref(xr, w[:, 0].double(), None, cu, True)
    yr.sum().backward()
    assert_close("batch y", y.reshape(B * T, Cn), yr.detach(), torch.bfloat16)
    assert_close("batch dx", xd.grad.reshape(B * T, Cn), xr.grad, torch.bfloat16)


def test_short_conv_rejects_operands_the_kernel_would_misread():
    """Boundaries that do not end at the token count, a weight or bias of another channel count: refused on the host,
    before any launch (the kernels index weight and bias by x's channels and walk cu_seqlens up to its last entry)."""
    from nha_amd.ops import nha_short_conv
    x = torch.zeros(1, 64, 32, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(32, 1, 4, dtype=torch.bfloat16, device="cuda")
    good = torch.tensor([0, 20, 64], dtype=torch.int32, device="cuda")
    assert nha_short_conv(x, w, None, cu_seqlens=good).shape == x.shape
    for bad in ([0, 20, 60], [0, 20, 70], [4, 20, 64], [0, 40, 30, 64], [64]):
        with pytest.raises(ValueError, match="cu_seqlens must rise"):
            nha_short_conv(x, w, None, cu_seqlens=torch.tensor(bad, dtype=torch.int32, device="cuda"))
    with pytest.raises(ValueError, match="weight must be"):
        nha_short_conv(x, torch.zeros(16, 1, 4, dtype=torch.bfloat16, device="cuda"), None)
    with pytest.raises(ValueError, match="bias must have"):
        nha_short_conv(x, w, torch.zeros(16, dtype=torch.bfloat16, device="cuda"))
