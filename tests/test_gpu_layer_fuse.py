"""The fused layer glue (nha_layer_prologue / nha_layer_epilogue through the C ABI) against the fp64
restatement of nha_fla/layers/nha.py:214-237, :278 in the oracle, and the layer with the fused glue
against the same layer on the tensor-op chain."""
import pytest
import torch

pytestmark = pytest.mark.gpu

NAMES = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")


def _close(name, got, ref, dtype):
    got, ref = got.double().cpu(), ref.double().cpu()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    # bf16: one rounding of the result (2^-8 relative) plus the rounding points of the reference's
    # chain of bf16 tensor ops (logsigmoid -> /n -> exp -> 1-x); fp32: float32 arithmetic error
    atol, rtol = (1e-2, 1e-2) if dtype == torch.bfloat16 else (2e-6, 2e-6)
    bad = (got - ref).abs() > atol + rtol * ref.abs()
    assert not bad.any(), f"{name}: {int(bad.sum())} out of tolerance, max err {(got - ref).abs().max():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,T,HQ,H,K,V,M,fmap,offset,varlen", [
    (2, 300, 4, 2, 128, 128, 64, "swish", 0, False),
    (1, 517, 8, 2, 64, 64, 64, "relu", 1000, False),
    (1, 333, 4, 4, 256, 256, 64, "swish", 0, True),
    (2, 65, 4, 1, 32, 16, 8, None, 5, False),
    (1, 50, 2, 1, 6, 5, 3, "swish", 0, True),              # no 16-byte rows: the element-wise variant
])
def test_prologue_matches_oracle(dtype, B, T, HQ, H, K, V, M, fmap, offset, varlen):
    from nha_amd.ops import nha_layer_prologue
    from oracle import nha_ref as R
    gen = torch.Generator().manual_seed(T + K)
    r = lambda *s: torch.randn(*s, generator=gen).to(dtype)
    q, k, v, f = r(B, T, HQ, K), r(B, T, H, K), r(B, T, H, V), 3 * r(B, T, H, M)
    cu = None
    pos = torch.arange(T) + offset
    if varlen:
        cu = torch.tensor([0, T // 3, T // 3 + 1, T], dtype=torch.int32)
        pos = torch.cat([torch.arange(int(b - a)) for a, b in zip(cu[:-1], cu[1:])]) + offset
    inv = 1.0 / (10000.0 ** (torch.arange(0, K, 2, dtype=torch.float32) / K))
    out = nha_layer_prologue(q.cuda(), k.cuda(), v.cuda(), f.cuda(), inv.cuda(), feature_map=fmap,
                             gate_logit_normalizer=8, seqlen_offset=offset,
                             cu_seqlens=None if cu is None else cu.cuda())
    ref = R.layer_prologue_ref(q.double(), k.double(), v.double(), f.double(), feature_map=fmap,
                               gate_logit_normalizer=8, positions=pos)
    for name, a, b in zip(NAMES, out, ref):
        assert a.dtype == dtype
        _close(name, a, b, dtype)
    if dtype == torch.float32:
        # s + exp(g) = 1 holds for the kernel's own outputs too
        assert ((out[5] + out[6].exp()).cpu() - 1).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,dim,affine", [(300, 1024, "wb"), (77, 4096, "w"), (5, 30, "none"), (2000, 256, "w")])
def test_epilogue_matches_oracle(dtype, rows, dim, affine):
    from nha_amd.ops import nha_layer_epilogue
    from oracle import nha_ref as R
    gen = torch.Generator().manual_seed(rows + dim)
    o = (2 * torch.randn(rows, dim, generator=gen)).to(dtype)
    w = torch.randn(dim, generator=gen) if "w" in affine else None
    b = torch.randn(dim, generator=gen) if "b" in affine else None
    y = nha_layer_epilogue(o.cuda(), None if w is None else w.cuda(), None if b is None else b.cuda(), 1e-5)
    ref = R.layer_epilogue_ref(o.double(), None if w is None else w.double(), None if b is None else b.double(), 1e-5)
    assert y.dtype == dtype and y.shape == o.shape
    _close("y", y, ref, dtype)


def _grad_close(name, got, ref, dtype):
    """Gradients: relative L2 error (bf16 5e-3: one rounding of the result plus the rounded
    intermediates of the forward chain; fp32 1e-5) and max error against the tensor's scale."""
    got, ref = got.double().cpu(), ref.double().cpu()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), name
    l2, mx = (5e-3, 2e-2) if dtype == torch.bfloat16 else (1e-5, 1e-4)
    scale = max(ref.abs().max().item(), 1e-30)
    rel = ((got - ref).norm() / max(ref.norm().item(), 1e-30)).item()
    assert rel <= l2, f"{name}: relative L2 error {rel:.3e}"
    assert (got - ref).abs().max().item() <= mx * scale, f"{name}: max err {(got - ref).abs().max():.3e} vs scale {scale:.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B,T,HQ,H,K,V,M,fmap,offset,varlen", [
    (2, 130, 4, 2, 128, 128, 64, "swish", 0, False),
    (1, 211, 8, 2, 64, 64, 64, "relu", 77, True),
    (2, 40, 4, 1, 32, 16, 8, None, 3, False),
    (1, 30, 2, 1, 6, 5, 3, "swish", 0, True),
])
def test_prologue_backward_matches_oracle_autograd(dtype, B, T, HQ, H, K, V, M, fmap, offset, varlen):
    from nha_amd.ops import nha_layer_prologue
    from oracle import nha_ref as R
    gen = torch.Generator().manual_seed(7 * T + K)
    r = lambda *s: torch.randn(*s, generator=gen).to(dtype)
    x = [r(B, T, HQ, K), r(B, T, H, K), r(B, T, H, V), 3 * r(B, T, H, M)]
    cot = [r(B, T, HQ, K), r(B, T, H, K), r(B, T, HQ, K), r(B, T, H, K), r(B, T, H, V), r(B, T, H, M), r(B, T, H, M)]
    cu, pos = None, torch.arange(T) + offset
    if varlen:
        cu = torch.tensor([0, T // 3, T // 3 + 1, T], dtype=torch.int32)
        pos = torch.cat([torch.arange(int(b - a)) for a, b in zip(cu[:-1], cu[1:])]) + offset
    inv = 1.0 / (10000.0 ** (torch.arange(0, K, 2, dtype=torch.float32) / K))
    xg = [t.cuda().requires_grad_(True) for t in x]
    out = nha_layer_prologue(*xg, inv.cuda(), feature_map=fmap, gate_logit_normalizer=8, seqlen_offset=offset,
                             cu_seqlens=None if cu is None else cu.cuda())
    sum((o.float() * c.cuda().float()).sum() for o, c in zip(out, cot)).backward()
    xr = [t.double().requires_grad_(True) for t in x]
    ref = R.layer_prologue_ref(*xr, feature_map=fmap, gate_logit_normalizer=8, positions=pos)
    sum((o * c.double()).sum() for o, c in zip(ref, cot)).backward()
    for name, a, b in zip(("dq", "dk", "dv", "df"), xg, xr):
        assert a.grad.dtype == dtype
        _grad_close(name, a.grad, b.grad, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,dim,affine", [(300, 1024, "wb"), (77, 4096, "w"), (45, 8192, "w"), (33, 24, "none"), (2000, 256, "w")])
def test_epilogue_backward_matches_oracle_autograd(dtype, rows, dim, affine):
    from nha_amd.ops import nha_layer_epilogue
    from oracle import nha_ref as R
    gen = torch.Generator().manual_seed(rows + dim)
    o = (2 * torch.randn(rows, dim, generator=gen)).to(dtype)
    dy = torch.randn(rows, dim, generator=gen).to(dtype)
    w = (1 + 0.3 * torch.randn(dim, generator=gen)) if "w" in affine else None
    b = torch.randn(dim, generator=gen) if "b" in affine else None
    og = o.cuda().requires_grad_(True)
    wg = None if w is None else w.cuda().requires_grad_(True)
    bg = None if b is None else b.cuda().requires_grad_(True)
    y = nha_layer_epilogue(og, wg, bg, 1e-5)
    y.backward(dy.cuda())
    orf = o.double().requires_grad_(True)
    wr = None if w is None else w.double().requires_grad_(True)
    br = None if b is None else b.double().requires_grad_(True)
    R.layer_epilogue_ref(orf, wr, br, 1e-5).backward(dy.double())
    _grad_close("do", og.grad, orf.grad, dtype)
    if w is not None:
        _grad_close("dw", wg.grad, wr.grad, dtype)
    if b is not None:
        _grad_close("db", bg.grad, br.grad, dtype)
    y2 = nha_layer_epilogue(og, wg, bg, 1e-5)
    g1 = og.grad.clone()
    og.grad = None
    y2.backward(dy.cuda())
    assert torch.equal(og.grad, g1)                          # fixed reduction order: identical on a second run


@pytest.mark.parametrize("kv_heads,varlen", [(2, False), (4, True)])
def test_layer_fused_glue_matches_tensor_op_chain(kv_heads, varlen):
    from nha_amd.layer import NativeHybridAttention
    torch.manual_seed(3)
    layer = NativeHybridAttention(hidden_size=512, num_heads=4, num_kv_heads=kv_heads, num_slots=64, layer_idx=0,
                                  window_size=64).cuda().to(torch.bfloat16).eval()
    with torch.no_grad():
        layer.g_norm.weight.copy_(1 + 0.1 * torch.randn(512))
    x = (torch.randn(2, 200, 512) * 0.5).to(torch.bfloat16).cuda()
    mask = None
    if varlen:
        mask = torch.ones(2, 200, dtype=torch.bool).cuda()
        mask[1, :37] = False                                # left padding, as the reference's generation path pads
    calls = []
    import nha_amd.layer as L
    orig = L.nha_layer_prologue
    L.nha_layer_prologue = lambda *a, **k: (calls.append(1), orig(*a, **k))[1]
    try:
        with torch.no_grad():
            y_fused = layer(x, attention_mask=mask)[0]
            layer.fuse_glue = False
            y_chain = layer(x, attention_mask=mask)[0]
        assert len(calls) == 1                              # the fused kernels ran exactly in the first call
        layer.fuse_glue = True
        xg = x.clone().requires_grad_(True)
        y_grad = layer(xg, attention_mask=mask)[0]          # autograd on: the fused kernels with their backward
        assert len(calls) == 2 and y_grad.requires_grad
        y_grad.float().square().sum().backward()
        g_fused = {n: p.grad.clone() for n, p in layer.named_parameters()}
        gx_fused = xg.grad.clone()
        layer.zero_grad()
        layer.fuse_glue = False
        xc = x.clone().requires_grad_(True)
        layer(xc, attention_mask=mask)[0].float().square().sum().backward()
    finally:
        L.nha_layer_prologue = orig
    scale = max(1.0, y_chain.float().abs().max().item())
    assert (y_fused.float() - y_chain.float()).abs().max().item() <= 2e-2 * scale
    assert torch.equal(y_grad, y_fused)
    rel = lambda a, b: ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-30)).item()
    assert rel(gx_fused, xc.grad) <= 2e-2, rel(gx_fused, xc.grad)
    for n, p in layer.named_parameters():
        assert rel(g_fused[n], p.grad) <= 2e-2, (n, rel(g_fused[n], p.grad))
