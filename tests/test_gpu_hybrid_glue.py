"""nha_hybrid_prologue (one launch for the glue of the hybrid decoder blocks, through the C ABI) against the chain of
tensor ops it replaces, evaluated on the CPU in the same dtype with the same rounding points
(nha_fla/models/qwen3_moe_nha/qwennha.py:103-144, :240-247): per-head RMSNorm with fp32 statistics, logsigmoid / 8,
1 - exp, padding mask, rotate-half rotary embedding in fp32 rounded once.

Tolerances: the plain outputs (normed q / k, v, g, s) follow the chain's rounding sequence, so they may differ from
it by one rounding of the last step (bf16: one unit in the last place where hardware exp / rsqrt land on the other
side of a tie); rotated outputs likewise.  bf16: 1e-2 abs + 1e-2 rel; fp32: 2e-6 abs + 2e-6 rel."""
import pytest
import torch
import torch.nn.functional as F

from oracle.hybrid_attention_ref import zero_sink_attention_ref

pytestmark = pytest.mark.gpu


def chain(q, k, v, f, cos, sin, qw, kw, eps, mask, HQ, H, D, M):
    dt = q.dtype
    B, T = q.shape[:2]
    q, k, v = q.reshape(B, T, HQ, D), k.reshape(B, T, H, D), v.reshape(B, T, H, D)

    def norm(x, w):
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        return w * xf.to(dt)

    if qw is not None:
        q, k = norm(q, qw), norm(k, kw)

    def rot(x):
        h = D // 2
        xf = x.float()
        r = torch.cat([-xf[..., h:], xf[..., :h]], -1)
        return (xf * cos[:, :, None].float() + r * sin[:, :, None].float()).to(dt)

    if f is None:
        g = torch.zeros(B, T, H, M, dtype=dt)
        s = torch.zeros_like(g)
    else:
        g = F.logsigmoid(f.reshape(B, T, H, M)) / 8
        s = 1 - torch.exp(g).to(dt)
    if mask is not None:
        m = mask.to(dt)[:, :, None, None]
        v, s = v * m, s * m
    return q, rot(q), k, rot(k), v, g, s


def close(name, got, ref, dt):
    got, ref = got.detach().float().cpu(), ref.detach().float()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    tol = (1e-2, 1e-2) if dt == torch.bfloat16 else (2e-6, 2e-6)
    bad = (got - ref).abs() > tol[0] + tol[1] * ref.abs()
    assert not bad.any(), f"{name}: {int(bad.sum())} elements off, max {float((got - ref).abs().max()):.3e}"


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("HQ,H,D,M,norm,gates,masked,fused_in", [
    (32, 4, 128, 64, True, True, False, True),      # the MoE hybrid's heads, inputs are slices of one projection output
    (8, 2, 128, 64, False, True, True, False),      # the dense flavour (no norm), left padding
    (4, 4, 256, 64, True, False, True, True),       # a layer without slot writes
    (6, 3, 64, 16, True, True, False, False),
])
def test_hybrid_prologue_matches_the_tensor_op_chain(dt, HQ, H, D, M, norm, gates, masked, fused_in):
    from nha_amd.ops import nha_hybrid_prologue
    gen = torch.Generator().manual_seed(HQ * 1000 + D)
    for B, T in ((2, 37), (5, 1)):
        width = HQ * D + 2 * H * D + H * M
        y = (torch.randn(B, T, width, generator=gen) * 1.5).to(dt)
        o0, o1, o2 = HQ * D, HQ * D + H * D, HQ * D + 2 * H * D
        parts = [y[..., :o0], y[..., o0:o1], y[..., o1:o2], y[..., o2:]]
        pos = torch.arange(T)[None] + torch.tensor([[3], [100]] if B == 2 else [[7 * i] for i in range(B)])
        inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
        ang = pos.float()[..., None] * inv
        cos, sin = torch.cat([ang, ang], -1).cos().to(dt), torch.cat([ang, ang], -1).sin().to(dt)
        qw = (1 + 0.1 * torch.randn(D, generator=gen)).to(dt) if norm else None
        kw = (1 + 0.1 * torch.randn(D, generator=gen)).to(dt) if norm else None
        mask = None
        if masked:
            mask = torch.ones(B, T, dtype=torch.long)
            mask[-1, : T // 3] = 0
        ref = chain(parts[0], parts[1], parts[2], parts[3] if gates else None, cos, sin, qw, kw, 1e-6, mask, HQ, H, D, M)
        yd = y.cuda()
        dev_parts = [yd[..., :o0], yd[..., o0:o1], yd[..., o1:o2], yd[..., o2:]]
        if not fused_in:
            dev_parts = [p.contiguous() for p in dev_parts]
        got = nha_hybrid_prologue(dev_parts[0], dev_parts[1], dev_parts[2], dev_parts[3] if gates else None, cos.cuda(),
                                  sin.cuda(), num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=M,
                                  q_weight=None if qw is None else qw.cuda(), k_weight=None if kw is None else kw.cuda(),
                                  eps=1e-6, mask=None if mask is None else mask.cuda())
        for name, a, b in zip(("q", "sq", "k", "sk", "v", "g", "s"), got, ref):
            close(f"{name} B{B} T{T}", a, b, dt)
        # the same with the table rows formed inside the launch from the positions
        got_p = nha_hybrid_prologue(dev_parts[0], dev_parts[1], dev_parts[2], dev_parts[3] if gates else None, None, None,
                                    positions=pos.expand(B, T).cuda(), inv_freq=inv.cuda(), num_heads=HQ, num_kv_heads=H,
                                    head_dim=D, num_slots=M, q_weight=None if qw is None else qw.cuda(),
                                    k_weight=None if kw is None else kw.cuda(), eps=1e-6, mask=None if mask is None else mask.cuda())
        for name, a, b in zip(("q", "sq", "k", "sk", "v", "g", "s"), got_p, ref):
            close(f"{name} from positions B{B} T{T}", a, b, dt)
        # one table for every sequence ([1, T, D]) and no s (what a decode step asks for)
        if B > 1:
            pos1 = torch.arange(T)[None] + 11
            ang = pos1.float()[..., None] * inv
            c1, s1 = torch.cat([ang, ang], -1).cos().to(dt), torch.cat([ang, ang], -1).sin().to(dt)
            ref1 = chain(parts[0], parts[1], parts[2], parts[3] if gates else None, c1.expand(B, -1, -1), s1.expand(B, -1, -1),
                         qw, kw, 1e-6, None, HQ, H, D, M)
            got1 = nha_hybrid_prologue(dev_parts[0], dev_parts[1], dev_parts[2], dev_parts[3] if gates else None, c1.cuda(),
                                       s1.cuda(), num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=M,
                                       q_weight=None if qw is None else qw.cuda(), k_weight=None if kw is None else kw.cuda(),
                                       eps=1e-6, want_s=False)
            assert got1[6] is None
            close(f"sq shared table B{B}", got1[1], ref1[1], dt)
            close(f"sk shared table B{B}", got1[3], ref1[3], dt)


def test_block_with_fused_glue_matches_block_on_the_tensor_op_chain():
    """The MoE-flavour block at its model's head shape: prompt and two decode steps with the fused projection + glue
    launch against the same module on the tensor-op chain (`fuse_glue = False`)."""
    from nha_amd import NHACache
    from nha_amd.hybrid import HybridNHAConfig, Qwen3MoeNativeHybridAttention
    cfg = HybridNHAConfig(hidden_size=512, num_attention_heads=32, num_key_value_heads=4, head_dim=128, num_slots=64,
                          window_size=64, attention_bias=True)
    torch.manual_seed(3)
    m = Qwen3MoeNativeHybridAttention(cfg, 0).to(torch.bfloat16).cuda().eval()
    with torch.no_grad():
        m.q_norm.weight.add_(0.1 * torch.randn_like(m.q_norm.weight))
        for lin in (m.q_proj, m.k_proj, m.v_proj):
            lin.bias.normal_(0, 0.1)
    x = torch.randn(2, 150, 512, device="cuda").to(torch.bfloat16)
    mask = torch.ones(2, 152, dtype=torch.long, device="cuda")
    mask[1, :20] = 0
    pos = (mask.cumsum(1) - 1).clamp(min=0)
    outs = []
    for fuse in (True, False):
        m.fuse_glue = fuse
        cache = NHACache()
        with torch.no_grad():
            a, _ = m(x, attention_mask=mask[:, :150], position_ids=pos[:, :150], past_key_value=cache, use_cache=True)
            steps = []
            for t in (150, 151):
                xs = torch.randn(2, 1, 512, device="cuda", generator=torch.Generator("cuda").manual_seed(t)).to(torch.bfloat16)
                b, _ = m(xs, attention_mask=mask[:, :t + 1], position_ids=pos[:, t:t + 1], past_key_value=cache, use_cache=True)
                steps.append(b)
        outs.append((a, steps))
    # rotary tables handed in by the caller (`position_embeddings`, as the decoder models do) instead of formed in the launch
    m.fuse_glue = True
    with torch.no_grad():
        tables = m.rotary_emb(x, pos[:, :150])
        a2, _ = m(x, attention_mask=mask[:, :150], position_embeddings=tables)
    (a1, s1), (a0, s0) = outs
    assert float((a2[0] - a1[0]).abs().max()) <= 1e-2 * float(a1[0].abs().max())
    scale = float(a0[1, 20:].abs().max())
    assert float((a1[0] - a0[0]).abs().max()) <= 2e-2 * scale and float((a1[1, 20:] - a0[1, 20:]).abs().max()) <= 2e-2 * scale
    for x1, x0 in zip(s1, s0):
        assert float((x1 - x0).abs().max()) <= 2e-2 * float(x0.abs().max())


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_zero_sink_rescale_matches_the_log_space_formula(dt, D):
    """o * (e^lse + M) / (e^lse + clamp(W - 1 - t, 0, M)) in place, against float64, with window log-sum-exps from
    -100 to +100 (e^-lse outside fp32) and every sink count from M down to 0."""
    from nha_amd.ops import nha_zero_sink_rescale_
    gen = torch.Generator().manual_seed(D)
    B, T, HQ, W, M = 2, 90, 3, 70, 16
    o = torch.randn(B, T, HQ, D, generator=gen).to(dt)
    lse = torch.randn(B, T, HQ, generator=gen) * 3
    lse[0, ::7] = -100.0
    lse[1, ::5] = 100.0
    lse[0, 3] = -88.5
    got = nha_zero_sink_rescale_(o.clone().cuda(), lse.cuda(), W, M).cpu()
    n0 = (W - 1 - torch.arange(T)).clamp(0, M).double()[None, :, None]
    e = torch.exp(lse.double())
    fac = (e + M) / (e + n0)
    ref = o.double() * fac[..., None]
    fin = torch.isfinite(ref) & (ref.abs() < 1e38)      # rows whose exact value no float holds (no sink in view, lse = -100) aside
    assert torch.isfinite(got[fin]).all() and not torch.isnan(got).any()
    tol = 1e-2 if dt == torch.bfloat16 else 1e-5
    err = ((got.double() - ref).abs() / ref.abs().clamp(min=1e-30))[fin]
    assert float(err.max()) <= tol, float(err.max())
    # rows with every sink still in view are left bit-identical
    assert torch.equal(got[:, : W - 1 - M], o[:, : W - 1 - M])


@pytest.mark.parametrize("window", [64, 2048])
def test_recorded_decode_step_replays_match_eager_steps(window):
    """A block's decode step recorded into a HIP graph: twelve replays, with eager work of the same program and a
    synchronisation between them, each against the eager step of a second cache that took the same prompt; the ring
    contents and counters agree at the end.  An NHA layer (window 64: pops start at once after a 100-token prompt)
    and a zero-sink layer."""
    from nha_amd import NHACache
    from nha_amd.hybrid import HybridNHAConfig, Qwen3MoeNativeHybridAttention
    cfg = HybridNHAConfig(hidden_size=256, num_attention_heads=8, num_key_value_heads=2, head_dim=128, num_slots=64,
                          window_size=64, block_size=1 if window == 2048 else None, transformer_idx=0 if window == 2048 else None)
    torch.manual_seed(11)
    m = Qwen3MoeNativeHybridAttention(cfg, 0).to(torch.bfloat16).cuda().eval()
    assert m.window_size == window
    B, T0 = 3, 100
    x0 = torch.randn(B, T0, 256, device="cuda").to(torch.bfloat16)
    pos0 = torch.arange(T0, device="cuda")[None].expand(B, -1)
    eager, rec = NHACache(), NHACache()
    with torch.no_grad():
        m(x0, position_ids=pos0, past_key_value=eager, use_cache=True)
        m(x0, position_ids=pos0, past_key_value=rec, use_cache=True)
    step = m.record_decode_step(rec, B)
    assert rec.layer_tokens(0) == T0 and int(rec.states[0].count[0]) == T0     # recording leaves the cache as it was
    gen = torch.Generator("cuda").manual_seed(5)
    for t in range(T0, T0 + 12):
        xs = torch.randn(B, 1, 256, device="cuda", generator=gen).to(torch.bfloat16)
        pos = torch.full((B, 1), t, device="cuda")
        with torch.no_grad():
            want, _ = m(xs, position_ids=pos, past_key_value=eager, use_cache=True)
        if t % 2:
            got = step.step(xs, pos).clone()
        else:                                   # the caller writes into the graph's own input buffers: no copies
            step.x.copy_(xs)
            step.pos.copy_(pos)
            got = step.step(step.x, step.pos).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), (t, float((got.float() - want.float()).abs().max()))
        _ = (xs.float() @ xs.float().transpose(1, 2)).sum().item()      # eager work and a sync between replays
    assert rec.layer_tokens(0) == eager.layer_tokens(0) == T0 + 12
    a, b = eager.states[0], rec.states[0]
    assert torch.equal(a.count, b.count)
    for name in ("hk", "hv", "ring_k", "ring_kg", "ring_v", "ring_g"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name
    # an eager step on the recorded cache moves its counters to the other array: the recording refuses to go on
    with torch.no_grad():
        m(xs, position_ids=pos + 1, past_key_value=rec, use_cache=True)
    with pytest.raises(RuntimeError, match="record again"):
        step.step(xs, pos + 2)


@pytest.mark.parametrize("HQ,H,D", [(8, 2, 128), (4, 1, 64), (16, 2, 128)])
def test_zero_sink_attention_matches_the_restated_module_path(HQ, H, D):
    """nha_sink_window_fwd (the prefill's window loop alone, sinks in the denominator) against the oracle's restatement
    of the reference's zero-prefix sliding-window attention (pinned by brute force on the CPU), bf16: sequences shorter
    and longer than the window, windows shorter than a 32-key unit, not a multiple of it, and 2048; packed sequences;
    the returned log-denominator against the same softmax."""
    from nha_amd.ops import zero_sink_attention
    gen = torch.Generator().manual_seed(HQ + D)
    bf = torch.bfloat16
    for B, T, W, M in ((2, 300, 96, 64), (1, 700, 256, 64), (2, 130, 2048, 64), (1, 90, 20, 16), (3, 64, 33, 64)):
        q = (torch.randn(B, T, HQ, D, generator=gen) * D ** -0.25).to(bf)
        k = (torch.randn(B, T, H, D, generator=gen) * D ** -0.25).to(bf)
        v = torch.randn(B, T, H, D, generator=gen).to(bf)
        ref = zero_sink_attention_ref(q.double(), k.double(), v.double(), W, M)
        got, lse = zero_sink_attention(q.cuda(), k.cuda(), v.cuda(), W, M, output_lse=True)
        close(f"o B{B} T{T} W{W}", got, ref, bf)
        # the denominator: log(sum over the window of e^(scale q.k) + sinks in view)
        G = HQ // H
        kk = k.double().repeat_interleave(G, 2)
        sc = torch.einsum("bthd,bnhd->bhtn", q.double(), kk) / D ** 0.5
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        vis = (j <= i) & (j > i - W)
        e = torch.exp(sc.masked_fill(~vis[None, None], -1e30)).sum(-1).transpose(1, 2)          # [B, T, HQ]
        n0 = (W - 1 - torch.arange(T)).clamp(0, M).double()[None, :, None]
        assert torch.allclose(lse.double().cpu(), torch.log(e + n0), atol=2e-2, rtol=1e-2)
    # packed sequences (one of a single token, one ending mid-chunk)
    cu = [0, 1, 130, 451]
    q = (torch.randn(1, cu[-1], HQ, D, generator=gen) * D ** -0.25).to(bf)
    k = (torch.randn(1, cu[-1], H, D, generator=gen) * D ** -0.25).to(bf)
    v = torch.randn(1, cu[-1], H, D, generator=gen).to(bf)
    got = zero_sink_attention(q.cuda(), k.cuda(), v.cuda(), 100, 64, cu_seqlens=torch.tensor(cu, dtype=torch.int32).cuda())
    for a, b in zip(cu[:-1], cu[1:]):
        ref = zero_sink_attention_ref(q[:, a:b].double(), k[:, a:b].double(), v[:, a:b].double(), 100, 64)
        close(f"packed [{a},{b})", got[:, a:b], ref, bf)


def test_zero_sink_attention_rows_far_from_the_fixed_reference_take_the_exact_pass():
    """Scale 1 with unnormalised q / k: window scores of a few hundred above and below those of a row's nearest keys, so
    rows whose sums leave the fp32 range around the fixed softmax reference are recomputed by the exact pass.  Finite
    everywhere, relative L2 within 3e-2 (logits of this size make the softmax one-hot: single outputs move by more than
    the element-wise bar under bf16 rounding of the scores)."""
    from nha_amd.ops import zero_sink_attention
    gen = torch.Generator().manual_seed(9)
    bf = torch.bfloat16
    B, T, HQ, H, D, W, M = 2, 200, 8, 2, 128, 100, 64
    for qk in (1.0, 3.0):
        q = (torch.randn(B, T, HQ, D, generator=gen) * qk).to(bf)
        k = (torch.randn(B, T, H, D, generator=gen) * qk).to(bf)
        v = torch.randn(B, T, H, D, generator=gen).to(bf)
        got = zero_sink_attention(q.cuda(), k.cuda(), v.cuda(), W, M, scale=1.0).double().cpu()
        qq, kk, vv = q.double(), k.double().repeat_interleave(HQ // H, 2), v.double().repeat_interleave(HQ // H, 2)
        sc = torch.einsum("bthd,bnhd->bhtn", qq, kk)
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        vis = (j <= i) & (j > i - W)
        sc = sc.masked_fill(~vis[None, None], -float("inf"))
        n0 = (W - 1 - torch.arange(T)).clamp(0, M).double()
        mx = torch.maximum(sc.amax(-1), torch.zeros(()).double())
        e = torch.exp(sc - mx[..., None])
        den = e.sum(-1) + n0[None, None] * torch.exp(-mx)
        ref = torch.einsum("bhtn,bnhd->bthd", e / den[..., None], vv)
        assert torch.isfinite(got).all()
        rel = ((got - ref).norm() / ref.norm()).item()
        assert rel <= 3e-2, (qk, rel)
