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
        y_grad = layer(x, attention_mask=mask)[0]           # autograd on: tensor-op chain
        assert len(calls) == 1 and y_grad.requires_grad
    finally:
        L.nha_layer_prologue = orig
    scale = max(1.0, y_chain.float().abs().max().item())
    assert (y_fused.float() - y_chain.float()).abs().max().item() <= 2e-2 * scale
    assert torch.equal(y_grad, y_chain)
