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


def _oracle_layer_general(w, xc, *, H, HKV, M, W, D, cu=None, feature_map="swish", conv=None, conv_cache=None):
    """fp64 restatement of nha_fla/layers/nha.py:186-278 for a packed stream xc [1, T, hid] (cu: sequence
    starts) or a batch [B, T, hid]: optional depthwise causal short convolutions with SiLU (restarting at
    every sequence, or continuing from conv_cache [B, C, k-1] per projection), feature map, gates, RoPE
    with positions inside each sequence, the oracle's prefill, SiLU + RMS norm + output projection.
    Returns (y, conv_states)."""
    from oracle import nha_ref as R
    Bq, T = xc.shape[0], xc.shape[1]
    starts = [0, T] if cu is None else [int(c) for c in cu]

    def short_conv(x, name, cache):
        wt = w[f"{name}.weight"][:, 0, :]                              # [C, k]
        k = wt.shape[1]
        y = torch.zeros_like(x)
        states = []
        for b in range(Bq):
            for n in range(len(starts) - 1):
                lo, hi = starts[n], starts[n + 1]
                seg = x[b, lo:hi]                                       # [L, C]
                hist = torch.zeros(k - 1, x.shape[-1], dtype=x.dtype) if cache is None else cache[b].T
                ext = torch.cat([hist, seg], 0)                         # [k-1+L, C]
                for t in range(hi - lo):
                    y[b, lo + t] = (ext[t:t + k] * wt.T).sum(0)
                states.append(ext[-(k - 1):].T if ext.shape[0] >= k - 1 else None)
        return F.silu(y), states

    q, k_, v = xc @ w["q_proj.weight"].T, xc @ w["k_proj.weight"].T, xc @ w["v_proj.weight"].T
    conv_states = None
    if conv:
        cc = (None, None, None) if conv_cache is None else conv_cache
        q, sq = short_conv(q, "q_conv1d", cc[0])
        k_, sk = short_conv(k_, "k_conv1d", cc[1])
        v, sv = short_conv(v, "v_conv1d", cc[2])
        conv_states = (sq, sk, sv)
    q, k_, v = q.unflatten(-1, (H, D)), k_.unflatten(-1, (HKV, D)), F.silu(v.unflatten(-1, (HKV, D)))
    f = F.logsigmoid((xc @ w["f_proj.weight"].T).unflatten(-1, (HKV, M))) / 8
    s, g = 1 - f.exp(), f
    if feature_map == "swish":
        q_gsa, k_gsa = F.silu(q), F.silu(k_)
    elif feature_map == "relu":
        q_gsa, k_gsa = F.relu(q), F.relu(k_)
    elif feature_map == "t2r":
        tw = w["feature_map.layer.weight"]
        q_gsa, k_gsa = F.relu(q @ tw.T), F.relu(k_ @ tw.T)
    else:
        q_gsa, k_gsa = q, k_
    pos = torch.cat([torch.arange(starts[n + 1] - starts[n], dtype=torch.float64) for n in range(len(starts) - 1)])
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    fr = torch.outer(pos, inv)
    cos, sin = torch.cat([fr.cos(), fr.cos()], -1)[None], torch.cat([fr.sin(), fr.sin()], -1)[None]
    q_swa, k_swa = R.rope_rotate_half(q, cos, sin), R.rope_rotate_half(k_, cos, sin)
    out = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=W, gsa_kv_shift=0, scale=1.0,
                        cu_seqlens=None if cu is None else torch.tensor(starts))[0]
    y = F.silu(out.flatten(-2))
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + 1e-5) * w["g_norm.weight"]
    return y @ w["o_proj.weight"].T, conv_states


def _close(got, ref, tol=3e-2):
    err = (got.detach().cpu().double() - ref).abs().max().item()
    assert err <= tol * max(1.0, ref.abs().max().item()), err


@pytest.mark.gpu
@pytest.mark.parametrize("fuse", [True, False])
def test_layer_attention_mask_unpads_and_repads(fuse):
    """attention_mask [B, T] (nha_fla/layers/nha.py:180-184, :279-280): right padding, left padding, a row
    of one token and a fully padded row.  Valid positions equal the oracle layer run on the packed
    valid tokens; padded positions come back as zeros."""
    from nha_amd.layer import NativeHybridAttention
    torch.manual_seed(3)
    hid, H, HKV, M, W, T = 256, 4, 2, 64, 16, 70
    D = hid // H
    layer = NativeHybridAttention(hidden_size=hid, num_heads=H, num_kv_heads=HKV, num_slots=M, layer_idx=0,
                                  window_size=W, scale=1.0).cuda().to(torch.bfloat16).eval()
    layer.fuse_glue = fuse
    mask = torch.ones(5, T, dtype=torch.int64)
    mask[1, 40:] = 0          # right padding
    mask[2, :25] = 0          # left padding
    mask[3, 1:] = 0           # a single token
    mask[4, :] = 0            # nothing at all
    x = (torch.randn(5, T, hid) * 0.5).to(torch.bfloat16)
    o, _, _ = layer(x.cuda(), attention_mask=mask.cuda())
    assert o.shape == (5, T, hid)
    w = {k: v.detach().cpu().double() for k, v in layer.state_dict().items()}
    flat = mask.flatten().nonzero().flatten()
    lens = mask.sum(-1).tolist()
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    packed = x.double().reshape(5 * T, hid)[flat][None]
    ref, _ = _oracle_layer_general(w, packed, H=H, HKV=HKV, M=M, W=W, D=D, cu=cu)
    got = o.cpu().double().reshape(5 * T, hid)
    _close(got[flat], ref[0])
    pad = (mask.flatten() == 0).nonzero().flatten()
    assert (got[pad] == 0).all()


@pytest.mark.gpu
def test_layer_t2r_feature_map():
    from nha_amd.layer import NativeHybridAttention
    torch.manual_seed(4)
    hid, H, HKV, M, W = 256, 4, 4, 64, 16
    D = hid // H
    layer = NativeHybridAttention(hidden_size=hid, num_heads=H, num_kv_heads=HKV, num_slots=M, layer_idx=0,
                                  window_size=W, scale=1.0, feature_map="t2r").cuda().to(torch.bfloat16).eval()
    x = (torch.randn(2, 90, hid) * 0.5).to(torch.bfloat16)
    o, _, _ = layer(x.cuda())
    w = {k: v.detach().cpu().double() for k, v in layer.state_dict().items()}
    ref, _ = _oracle_layer_general(w, x.double(), H=H, HKV=HKV, M=M, W=W, D=D, feature_map="t2r")
    _close(o, ref)


@pytest.mark.gpu
def test_layer_short_conv_with_the_ring_cache():
    """use_short_conv with use_cache and an NHARingCache as past_key_values: the first chunk stores its
    convolution states through the cache's update(), the second chunk continues the convolutions from
    them (nha_fla/layers/nha.py:186-206, :268-274) and the counters follow the reference cache; a packed
    call returns one convolution state per sequence."""
    from nha_amd import NHARingCache
    from nha_amd.layer import NativeHybridAttention
    torch.manual_seed(5)
    hid, H, HKV, M, W, T1, T2 = 128, 2, 2, 64, 16, 40, 33
    D = hid // H
    layer = NativeHybridAttention(hidden_size=hid, num_heads=H, num_kv_heads=HKV, num_slots=M, layer_idx=0,
                                  window_size=W, scale=1.0, use_short_conv=True, conv_size=4).cuda().float().eval()
    w = {k: v.detach().cpu().double() for k, v in layer.state_dict().items()}
    x = torch.randn(2, T1 + T2, hid) * 0.5
    cache = NHARingCache(W)
    assert len(cache) == 0
    o1, _, pk = layer(x[:, :T1].cuda(), past_key_values=cache, use_cache=True)
    assert pk is cache and len(cache) == 1 and cache.seen_tokens == T1 and cache.get_seq_length(0) == 0
    r1, st1 = _oracle_layer_general(w, x[:, :T1].double(), H=H, HKV=HKV, M=M, W=W, D=D, conv=True)
    _close(o1, r1, 1e-3)
    got_states = cache[0]["conv_state"]
    for gs, rs in zip(got_states, st1):
        assert gs.shape == (2, gs.shape[1], 3)
        _close(gs, torch.stack(rs), 1e-5)
    assert [e["conv_state"] is not None for e in cache] == [True]
    o2, _, _ = layer(x[:, T1:].cuda(), past_key_values=cache, use_cache=True)
    assert cache.seen_tokens == T1 + T2 and cache.get_seq_length(0) == T1
    conv_cache = tuple(torch.stack(s) for s in st1)
    r2, _ = _oracle_layer_general(w, x[:, T1:].double(), H=H, HKV=HKV, M=M, W=W, D=D, conv=True, conv_cache=conv_cache)
    _close(o2, r2, 1e-3)
    legacy = cache.to_legacy_cache()
    again = NHARingCache.from_legacy_cache(legacy, seen_tokens=cache.seen_tokens, window_size=W)
    assert len(again) == 1 and again[0]["conv_state"][0] is legacy[0]["conv_state"][0]
    # packed sequences: the convolutions restart at every boundary, one final state per sequence
    lens = [5, 2, 30]
    cu = torch.tensor([0, 5, 7, 37], dtype=torch.int32)
    xp = torch.randn(1, 37, hid) * 0.5
    c2 = NHARingCache(W)
    op, _, _ = layer(xp.cuda(), past_key_values=c2, use_cache=True, cu_seqlens=cu.cuda())
    rp, stp = _oracle_layer_general(w, xp.double(), H=H, HKV=HKV, M=M, W=W, D=D, conv=True, cu=cu.tolist())
    _close(op, rp, 1e-3)
    for gs, rs in zip(c2[0]["conv_state"], stp):
        assert gs.shape[0] == len(lens)
        _close(gs, torch.stack(rs), 1e-5)
