"""The layer shell and the nha_fla import alias: construction and parameter names on CPU,
forward against a plain-PyTorch restatement of the same layer built on the oracle on GPU."""
import pytest
import torch
import torch.nn.functional as F


def test_import_alias_and_parameter_names():
    from nha_fla.layers.nha import NativeHybridAttention
    from nha_fla.ops import chunk_nha, fused_chunk_nha_prefill, fused_recurrent_nha, fused_recurrent_nha_decode  # noqa: F401
    from nha_fla.ops.nha import chunk_nha as c2
    assert c2 is chunk_nha
    layer = NativeHybridAttention(hidden_size=256, num_heads=4, num_kv_heads=2, num_slots=64, layer_idx=0, window_size=32)
    names = {n for n, _ in layer.named_parameters()}
    assert {"q_proj.weight", "k_proj.weight", "v_proj.weight", "f_proj.weight", "g_norm.weight", "o_proj.weight"} <= names
    assert layer.k_proj.weight.shape == (128, 256) and layer.f_proj.weight.shape == (2 * 64, 256)
    with pytest.raises(NotImplementedError):
        NativeHybridAttention(feature_map="nope", layer_idx=0)
    with pytest.raises(RuntimeError):
        layer(torch.randn(1, 8, 256))                       # CPU tensors: the op has no fallback


@pytest.mark.gpu
def test_layer_forward_matches_oracle_layer():
    from nha_amd.layer import NativeHybridAttention
    from oracle import nha_ref as R
    torch.manual_seed(0)
    hid, H, HKV, M, W = 256, 4, 2, 64, 32
    layer = NativeHybridAttention(hidden_size=hid, num_heads=H, num_kv_heads=HKV, num_slots=M, layer_idx=0,
                                  window_size=W, scale=1.0).cuda().to(torch.bfloat16).eval()
    x = (torch.randn(2, 150, hid) * 0.5).to(torch.bfloat16).cuda()
    o, _, _ = layer(x)
    # plain restatement of nha_fla/layers/nha.py:209-278 on CPU in fp64 with the same (bf16) weights
    D = hid // H
    w = {k: v.detach().cpu().double() for k, v in layer.state_dict().items()}
    xc = x.cpu().double()
    q = (xc @ w["q_proj.weight"].T).unflatten(-1, (H, D))
    k = (xc @ w["k_proj.weight"].T).unflatten(-1, (HKV, D))
    v = F.silu((xc @ w["v_proj.weight"].T).unflatten(-1, (HKV, D)))
    f = F.logsigmoid((xc @ w["f_proj.weight"].T).unflatten(-1, (HKV, M))) / 8
    s, g = 1 - f.exp(), f
    pos = torch.arange(150, dtype=torch.float64)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    fr = torch.outer(pos, inv)
    cos, sin = torch.cat([fr.cos(), fr.cos()], -1)[None], torch.cat([fr.sin(), fr.sin()], -1)[None]
    q_swa, k_swa = R.rope_rotate_half(q, cos, sin), R.rope_rotate_half(k, cos, sin)
    out, _, _, _, _ = R.prefill_ref(q_swa, k_swa, F.silu(q), F.silu(k), v, s, g, window_size_left=W, gsa_kv_shift=0, scale=1.0)
    y = F.silu(out.flatten(-2))
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + 1e-5) * w["g_norm.weight"]
    ref = y @ w["o_proj.weight"].T
    err = (o.cpu().double() - ref).abs().max().item()
    assert err <= 3e-2 * max(1.0, ref.abs().max().item()), err


def _oracle_layer(w, xc, H, HKV, M, W, D, aux_target=None):
    """fp64 restatement of nha_fla/layers/nha.py:209-278 (differentiable: built on the oracle's
    per-token recurrence without detaching)."""
    from oracle import nha_ref as R
    T = xc.shape[1]
    q = (xc @ w["q_proj.weight"].T).unflatten(-1, (H, D))
    k = (xc @ w["k_proj.weight"].T).unflatten(-1, (HKV, D))
    v = F.silu((xc @ w["v_proj.weight"].T).unflatten(-1, (HKV, D)))
    f = F.logsigmoid((xc @ w["f_proj.weight"].T).unflatten(-1, (HKV, M))) / 8
    s, g = 1 - f.exp(), f
    pos = torch.arange(T, dtype=torch.float64)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    fr = torch.outer(pos, inv)
    cos, sin = torch.cat([fr.cos(), fr.cos()], -1)[None], torch.cat([fr.sin(), fr.sin()], -1)[None]
    q_swa, k_swa = R.rope_rotate_half(q, cos, sin), R.rope_rotate_half(k, cos, sin)
    B = xc.shape[0]
    hk = torch.zeros(B, HKV, D, M, dtype=torch.float64)
    hv = torch.zeros(B, HKV, M, D, dtype=torch.float64)
    out, lse_swa, lse_gsa = R._prefill_equal_len(q_swa, k_swa, F.silu(q), F.silu(k), v, s, g, W, 0, 1.0, hk, hv)[:3]
    y = F.silu(out.flatten(-2))
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + 1e-5) * w["g_norm.weight"]
    y = y @ w["o_proj.weight"].T
    if aux_target is None:
        return y
    # nha_fla/layers/nha.py:300-317: BCE of lse_gsa - stopgrad(lse_swa) against the target ratio
    delta = lse_gsa - lse_swa.detach()
    return y, F.binary_cross_entropy_with_logits(delta, torch.full_like(delta, aux_target))


@pytest.mark.gpu
@pytest.mark.parametrize("aux", [False, True])
def test_layer_training_step_matches_oracle_layer(aux):
    """One forward + backward through the layer in fp32: the gradient of every parameter and of the
    input against autograd through the fp64 restatement (1e-3 of each gradient's scale: fp32
    projections and normalisation around the op).  With the auxiliary loss on, its gradient reaches
    the parameters through lse_gsa (the op's dlse_gsa cotangent) with weight coeff."""
    from nha_amd.layer import NativeHybridAttention
    torch.manual_seed(1)
    hid, H, HKV, M, W = 128, 4, 2, 32, 16
    D = hid // H
    coeff, ratio = 3.0, 0.7
    layer = NativeHybridAttention(hidden_size=hid, num_heads=H, num_kv_heads=HKV, num_slots=M, layer_idx=0,
                                  window_size=W, scale=1.0, gsa_aux_loss_enable=aux, gsa_aux_loss_coeff=coeff,
                                  gsa_aux_loss_target_ratio=ratio).cuda().float().train()
    x = (torch.randn(2, 100, hid) * 0.5).cuda().requires_grad_(True)
    tgt = torch.randn(2, 100, hid)
    o, _, _ = layer(x)
    (o * tgt.cuda()).sum().backward()
    w = {k: v.detach().cpu().double().requires_grad_(True) for k, v in layer.state_dict().items()}
    xc = x.detach().cpu().double().requires_grad_(True)
    if aux:
        ref, aux_loss = _oracle_layer(w, xc, H, HKV, M, W, D, aux_target=ratio)
        ((ref * tgt.double()).sum() + coeff * aux_loss).backward()
        assert abs(layer._gsa_aux_losses[-1] - aux_loss.item()) <= 1e-4 * abs(aux_loss.item())
    else:
        ref = _oracle_layer(w, xc, H, HKV, M, W, D)
        (ref * tgt.double()).sum().backward()
    assert (o.detach().cpu().double() - ref.detach()).abs().max() <= 1e-3 * max(1.0, ref.abs().max().item())
    named = dict(layer.named_parameters())
    for name, p in list(named.items()) + [("input", x)]:
        rg = xc.grad if name == "input" else w[name].grad
        assert p.grad is not None, name
        err = (p.grad.cpu().double() - rg).abs().max().item()
        assert err <= 1e-3 * max(rg.abs().max().item(), 1e-6), (name, err, rg.abs().max().item())
