"""The hybrid decoder models' attention blocks (nha_amd/hybrid.py) against the CPU restatement of the
reference's modules (oracle/hybrid_attention_ref.py): the parity tool's end-to-end case -- a 4-layer
stack, 128-token prompt, 16 single-token steps, batch 1 and 4, all-NHA and mixed layer assignments
(scripts/verify_opt_parity.py:592-694) -- plus the pins of that restatement, which run on the CPU."""
import pytest
import torch
import torch.nn.functional as F

from oracle.hybrid_attention_ref import HybridAttentionRef, zero_sink_attention_ref, _rope_tables, _rotate_half
from oracle.nha_ref import prefill_ref

F64 = torch.float64


# ----------------------------------------------------------------------------- CPU: pins of the restatement
def test_zero_sink_attention_matches_a_softmax_over_explicit_sinks():
    """Brute force: query t attends its W-wide causal window of real keys plus clamp(W-1-t, 0, M) keys of
    logit 0 and value 0 (the closed form nha_amd.hybrid.zero_sink_count states)."""
    from nha_amd.hybrid import zero_sink_count
    gen = torch.Generator().manual_seed(0)
    B, T, HQ, H, D, M, W = 2, 40, 4, 2, 8, 5, 12
    sq = torch.randn(B, T, HQ, D, generator=gen, dtype=F64)
    sk = torch.randn(B, T, H, D, generator=gen, dtype=F64)
    v = torch.randn(B, T, H, D, generator=gen, dtype=F64)
    got = zero_sink_attention_ref(sq, sk, v, W, M)
    n0 = zero_sink_count(T, W, M, "cpu")
    assert n0[0] == M and n0[W - 1 - M] == M and n0[W - 2] == 1 and n0[W - 1] == 0 and n0[-1] == 0
    G = HQ // H
    for b in range(B):
        for t in range(T):
            for h in range(HQ):
                lo = max(0, t - W + 1)
                logits = (sk[b, lo:t + 1, h // G] @ sq[b, t, h]) / D ** 0.5
                e = torch.exp(logits)
                o = (e[:, None] * v[b, lo:t + 1, h // G]).sum(0) / (e.sum() + float(n0[t]))
                assert torch.allclose(got[b, t, h], o, atol=1e-12), (b, t, h)


def test_pool_k_to_g_is_average_pooling_over_rows():
    """The library routine the reference calls (training/convert_weight.py:15-21): avg_pool1d over the
    row axis of the transposed weight."""
    from nha_amd.hybrid import pool_k_to_g
    gen = torch.Generator().manual_seed(1)
    w = torch.randn(64, 24, generator=gen)
    for rows in (64, 32, 16, 8):
        ref = F.avg_pool1d(w.T[:, None, :], kernel_size=64 // rows, stride=64 // rows)[:, 0].T
        assert torch.allclose(pool_k_to_g(w, rows), ref, atol=1e-6)
    with pytest.raises(ValueError, match="must be divisible"):
        pool_k_to_g(w, 24)


def _weights(gen, hidden, HQ, H, D, M, qk_norm, dtype=torch.bfloat16, bias=False):
    r = lambda *s, sc=1.0: (torch.randn(*s, generator=gen) * sc).to(dtype)
    w = {"q_proj.weight": r(HQ * D, hidden, sc=hidden ** -0.5), "k_proj.weight": r(H * D, hidden, sc=hidden ** -0.5),
         "v_proj.weight": r(H * D, hidden, sc=hidden ** -0.5), "g_proj.weight": r(H * M, hidden, sc=2 * hidden ** -0.5),
         "o_proj.weight": r(hidden, HQ * D, sc=(HQ * D) ** -0.5)}
    if qk_norm:
        w["q_norm.weight"] = (1 + 0.1 * torch.randn(D, generator=gen)).to(dtype)
        w["k_norm.weight"] = (1 + 0.1 * torch.randn(D, generator=gen)).to(dtype)
    if bias:
        for n, rows in (("q_proj", HQ * D), ("k_proj", H * D), ("v_proj", H * D), ("o_proj", hidden)):
            w[n + ".bias"] = r(rows, sc=0.1)
    return w


@pytest.mark.parametrize("window,T", [(8, 29), (96, 20)])
def test_restated_block_prompt_then_step_equals_longer_prompt(window, T):
    """Invariant of the model: the output for token T of a (T+1)-token prompt equals the output of one
    decode step after a T-token prompt -- through the pop, the window rule of the cache, the window
    positions of the rotary tables and the state hand-over.  (A zero-sink layer keeps all its sinks in
    decode but only clamp(W-1-t, 0, M) of them in a prompt, so its case stays below W-1-M tokens.)"""
    gen = torch.Generator().manual_seed(2)
    hidden, HQ, H, D, M = 32, 4, 2, 8, 4
    blk = HybridAttentionRef(_weights(gen, hidden, HQ, H, D, M, True, dtype=F64), num_heads=HQ, num_kv_heads=H,
                             head_dim=D, num_slots=M, window_size=window, qk_norm=True)
    x = torch.randn(2, T + 3, hidden, generator=gen, dtype=F64)
    pos = torch.arange(T + 3)[None].expand(2, -1)
    cache = {}
    blk.forward(x[:, :T], pos[:, :T], cache)
    for t in range(T, T + 3):
        step = blk.forward(x[:, t:t + 1], pos[:, t:t + 1], cache)
        whole = blk.forward(x[:, :t + 1], pos[:, :t + 1], {})
        assert torch.allclose(step[:, 0], whole[:, -1], atol=1e-10), (t, (step[:, 0] - whole[:, -1]).abs().max())
        assert cache["k"].shape[1] == min(t + 1, window)


def test_ring_cache_counts_layers_and_windows_per_layer():
    from nha_amd.cache import NHARingCache
    c = NHARingCache(window_size=32)
    assert not c.has_ring(0) and c.layer_tokens(0) == 0 and c.get_seq_length(0) == 0


def test_cache_under_the_reference_name_takes_the_reference_constructor():
    """`NHACache()` / `NHACache(seen_tokens)` / `NHACache.from_legacy_cache(None)` as the reference's callers build it
    (scripts/verify_opt_parity.py:671; nha_cache.py:20-29, :167-182), then the window rule through `update` and
    `get_pop_kvf` with the window size passed per call, as qwennha.py:151-176 does."""
    from nha_fla.models.nha_cache import NHACache
    W, H, D, M = 4, 2, 3, 5
    for cache in (NHACache(), NHACache.from_legacy_cache(None), NHACache(0)):
        assert cache.window_size is None and cache.seen_tokens == 0 and len(cache) == 0
        gen = torch.Generator().manual_seed(0)
        rows = [tuple(torch.randn(1, 1, H * d, generator=gen) for d in (D, D, M)) for _ in range(7)]
        for t, row in enumerate(rows):
            pop = cache.get_pop_kvf(0, W)
            if t < W:
                assert pop == (None, None, None)
            else:                                     # the entry that leaves is the oldest one held
                assert all(torch.equal(a, b) for a, b in zip(pop, rows[t - W]))
            held = cache.update(attn_state=row, layer_idx=0, offset=1, cache_kwargs=dict(window_size=W))["attn_state"]
            assert held[0].shape[-2] == min(t + 1, W) and torch.equal(held[0][..., -1:, :], row[0])
        assert cache.seen_tokens == 7 and cache.get_seq_length(0) == 6
    assert NHACache(5).seen_tokens == 5 and NHACache(5).window_size is None
    with pytest.raises(ValueError, match="window size"):
        c = NHACache()
        c.update(attn_state=rows[0], layer_idx=0)
        c.get_pop_kvf(0)


def test_zero_sink_rescale_stays_finite_for_strongly_negative_window_scores():
    """(e^lse + M) / (e^lse + n0) against float64 at lse = +-100, where e^-lse is outside fp32."""
    from nha_amd.hybrid import zero_sink_rescale
    lse = torch.tensor([-100.0, -100.0, -88.5, -30.0, 0.0, 3.0, 100.0, 100.0])
    n0 = torch.tensor([3.0, 64.0, 1.0, 0.0, 7.0, 0.0, 0.0, 64.0])
    got = zero_sink_rescale(lse, 64, n0)
    ref = (torch.exp(lse.double()) + 64) / (torch.exp(lse.double()) + n0.double())
    assert torch.isfinite(got).all()
    assert torch.allclose(got.double(), ref, rtol=1e-5), (got, ref)
    # no sink in view and a window weight below fp32: the ratio is capped, and a zero output row stays zero
    capped = zero_sink_rescale(torch.tensor([-100.0]), 64, torch.tensor([0.0]))
    assert torch.isfinite(capped).all() and float(capped * 0.0) == 0.0


def test_reference_import_paths_resolve_to_these_modules():
    from nha_fla.models.qwen3_moe_nha.qwennha import Qwen3MoeNativeHybridAttention as A
    from nha_fla.models.llama3_nha.llamanha import LlamaNativeHybridAttention as B_
    from nha_fla.models.nha_cache import NHACache
    from nha_fla.ops.nha.chunk_fused import fused_chunk_nha_prefill as f
    import nha_amd
    assert A is nha_amd.Qwen3MoeNativeHybridAttention and B_ is nha_amd.LlamaNativeHybridAttention
    assert NHACache is nha_amd.NHACache and issubclass(NHACache, nha_amd.NHARingCache) and f is nha_amd.fused_chunk_nha_prefill
    m = A(nha_amd.HybridNHAConfig(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16, num_slots=8,
                                  block_size=2, transformer_idx=1), layer_idx=3)
    assert m.window_size == 2048 and not m.is_nha_layer and sorted(n for n, _ in m.named_parameters()) == [
        "g_proj.weight", "k_norm.weight", "k_proj.weight", "o_proj.weight", "q_norm.weight", "q_proj.weight", "v_proj.weight"]
    with pytest.raises(TypeError, match="NHARingCache"):
        m(torch.zeros(1, 2, 64), past_key_value=object())


# ----------------------------------------------------------------------------- GPU: the end-to-end case
# (q heads, kv heads, head size, slots, window of the NHA layers).  "small" runs the generic kernels; the other two are
# head shapes of the converted models (eight / four query heads per kv-head at head size 128, 64 slots, window 64:
# qwen3_moe_nha and llama3_nha), which the LDS-direct prefill, the matrix-core decode step and the hand-over of that
# prefill's final state to the ring buffers serve.
SHAPES = {"small": (8, 2, 32, 16, 32), "moe_heads": (32, 4, 128, 64, 64), "dense_heads": (8, 2, 128, 64, 64)}


def _stack(tag, flavour, dev, shape="small"):
    from nha_amd.hybrid import HybridNHAConfig, Qwen3MoeNativeHybridAttention, LlamaNativeHybridAttention
    HQ, H, D, M, W = SHAPES[shape]
    cfg = HybridNHAConfig(hidden_size=256, num_attention_heads=HQ, num_key_value_heads=H, head_dim=D, num_slots=M,
                          window_size=W, max_position_embeddings=4096,
                          block_size=2 if tag == "mixed" else None, transformer_idx=1 if tag == "mixed" else None)
    cls = Qwen3MoeNativeHybridAttention if flavour == "moe" else LlamaNativeHybridAttention
    gen = torch.Generator().manual_seed(1234)
    layers, refs = [], []
    for i in range(4):
        w = _weights(gen, 256, HQ, H, D, M, flavour == "moe")
        m = cls(cfg, layer_idx=i).to(torch.bfloat16)
        m.load_state_dict(w, strict=True)
        layers.append(m.to(dev).eval())
        refs.append(HybridAttentionRef(w, num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=M, window_size=m.window_size,
                                       qk_norm=flavour == "moe", round_to=torch.bfloat16))
    return cfg, layers, refs


def _rms(x, dtype=None):
    y = x.float()
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + 1e-6)
    return y.to(x.dtype) if dtype is None else y.to(dtype).to(x.dtype)


def _run_stack(layers, x, pos, cache, mask=None):
    """x <- x + attention(rmsnorm(x)) per layer, in the tensors' dtype."""
    for m in layers:
        a, _ = m(_rms(x), attention_mask=mask, position_ids=pos, past_key_value=cache, use_cache=True)
        x = x + a
    return x


def _run_ref_stack(refs, x, pos, caches, mask=None):
    r = lambda t: t.to(torch.bfloat16).to(F64)
    for blk, c in zip(refs, caches):
        h = r(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6))
        x = r(x + blk.forward(h, pos, c, attention_mask=mask))
    return x


def _close(name, got, ref, tol=2.5e-2):
    got, ref = got.detach().double().cpu(), ref.double()
    assert torch.isfinite(got).all(), name
    scale = ref.abs().max().item()
    err = (got - ref).abs()
    assert err.max().item() <= tol * scale, f"{name}: max err {err.max().item():.3e} vs scale {scale:.3e}"
    assert err.mean().item() <= 0.2 * tol * scale, f"{name}: mean err {err.mean().item():.3e} vs scale {scale:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("tag,flavour,B,shape", [
    ("nha", "moe", 1, "small"), ("nha", "moe", 4, "small"), ("mixed", "moe", 1, "small"), ("mixed", "moe", 4, "small"),
    ("nha", "dense", 4, "small"), ("mixed", "dense", 1, "small"),
    ("nha", "moe", 2, "moe_heads"), ("mixed", "moe", 1, "moe_heads"), ("mixed", "dense", 2, "dense_heads")])
def test_stack_prompt_128_then_16_steps_matches_restated_modules(tag, flavour, B, shape):
    from nha_amd import NHACache, NHARingCache
    dev = torch.device("cuda:0")
    cfg, layers, refs = _stack(tag, flavour, dev, shape)
    gen = torch.Generator().manual_seed(99)
    x_pre = torch.randn(B, 128, 256, generator=gen).to(torch.bfloat16)
    x_dec = torch.randn(B, 16, 256, generator=gen).to(torch.bfloat16)
    # the cache under the reference's name and constructor for the model head shapes, the ring cache's own otherwise
    cache = NHACache() if shape != "small" else NHARingCache(cfg.window_size)
    ref_caches = [{} for _ in refs]
    with torch.no_grad():
        pos = torch.arange(128)[None].expand(B, -1)
        got = _run_stack(layers, x_pre.to(dev), pos.to(dev), cache)
        ref = _run_ref_stack(refs, x_pre.to(F64), pos, ref_caches)
        _close("prompt", got, ref)
        for t in range(16):
            pos = torch.full((B, 1), 128 + t)
            got = _run_stack(layers, x_dec[:, t:t + 1].to(dev), pos.to(dev), cache)
            ref = _run_ref_stack(refs, x_dec[:, t:t + 1].to(F64), pos, ref_caches)
            _close(f"step {t}", got, ref)
    assert cache.seen_tokens == 144 and cache.get_seq_length(0) == 144
    # the caches agree: slot states of the NHA layers, time-ordered windows of every layer
    for i, (m, rc) in enumerate(zip(layers, refs)):
        entry = cache[i]
        k, v, g = cache.window(i)
        n = min(144, m.window_size)
        pos = torch.arange(144 - n, 144)[None].expand(B, -1)
        cos, sin = (t.to(torch.bfloat16).to(F64) for t in _rope_tables(pos, cfg.head_dim, 10000.0))
        _close(f"layer {i} window keys", k, _rotate_half(ref_caches[i]["k"], cos, sin))
        _close(f"layer {i} window values", v, ref_caches[i]["v"])
        if m.is_nha_layer:
            _close(f"layer {i} hk", entry["recurrent_state"][0], ref_caches[i]["hk"])
            _close(f"layer {i} hv", entry["recurrent_state"][1], ref_caches[i]["hv"])
        else:
            assert float(entry["recurrent_state"][0].abs().max()) == 0.0


@pytest.mark.gpu
@pytest.mark.parametrize("grad", [False, True])
@pytest.mark.parametrize("HQ,H,D", [(4, 2, 64), (8, 2, 128)])
def test_zero_sink_layer_prompt_longer_than_its_window(grad, HQ, H, D):
    """A layer of the zero-sink kind whose window (96) the prompt (300 tokens) outgrows: the number of
    visible sinks falls from M to 0 along the prompt, which the per-query rescaling has to follow.  With
    gradients enabled the same numbers come out of the differentiable op.  The second head shape (four query
    heads per kv-head at head size 128) is served by the LDS-direct prefill kernel."""
    from nha_amd.hybrid import HybridNHAConfig, Qwen3MoeNativeHybridAttention
    dev = torch.device("cuda:0")
    cfg = HybridNHAConfig(hidden_size=128, num_attention_heads=HQ, num_key_value_heads=H, head_dim=D, num_slots=64, window_size=32)
    gen = torch.Generator().manual_seed(5)
    w = _weights(gen, 128, HQ, H, D, 64, True, bias=True)
    cfg.attention_bias = True
    m = Qwen3MoeNativeHybridAttention(cfg, 0).to(torch.bfloat16)
    m.load_state_dict(w)
    m = m.to(dev).eval()
    m.window_size = 96
    ref = HybridAttentionRef(w, num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=64, window_size=96, qk_norm=True,
                             round_to=torch.bfloat16)
    x = (torch.randn(2, 300, 128, generator=gen) * 2).to(torch.bfloat16)
    pos = torch.arange(300)[None].expand(2, -1)
    with torch.set_grad_enabled(grad):
        xin = x.to(dev).requires_grad_(grad)
        got, _ = m(xin, position_ids=pos.to(dev))
        if grad:
            got.float().sum().backward()
            assert torch.isfinite(xin.grad).all() and float(xin.grad.abs().max()) > 0
    _close("zero-sink prompt", got, ref.forward(x, pos))


@pytest.mark.gpu
def test_left_padded_prompt_and_steps():
    """Left padding (attention_mask): padded tokens write nothing into the slots and carry zero values
    (qwennha.py:133-144); prompt of 70 with 0 / 9 padded tokens, then 4 steps."""
    from nha_amd import NHARingCache
    from nha_amd.hybrid import HybridNHAConfig, LlamaNativeHybridAttention
    dev = torch.device("cuda:0")
    cfg = HybridNHAConfig(hidden_size=128, num_attention_heads=4, num_key_value_heads=4, head_dim=32, num_slots=16, window_size=16)
    gen = torch.Generator().manual_seed(6)
    w = _weights(gen, 128, 4, 4, 32, 16, False)
    m = LlamaNativeHybridAttention(cfg, 0).to(torch.bfloat16)
    m.load_state_dict(w)
    m = m.to(dev).eval()
    ref = HybridAttentionRef(w, num_heads=4, num_kv_heads=4, head_dim=32, num_slots=16, window_size=16, qk_norm=False,
                             round_to=torch.bfloat16)
    x = torch.randn(2, 74, 128, generator=gen).to(torch.bfloat16)
    mask = torch.ones(2, 74, dtype=torch.long)
    mask[1, :9] = 0
    pos = (mask.cumsum(1) - 1).clamp(min=0)
    cache, rc = NHARingCache(16), {}
    with torch.no_grad():
        got, _ = m(x[:, :70].to(dev), attention_mask=mask[:, :70].to(dev), position_ids=pos[:, :70].to(dev), past_key_value=cache,
                   use_cache=True)
        want = ref.forward(x[:, :70], pos[:, :70], rc, attention_mask=mask[:, :70])
        _close("prompt without padding", got[0], want[0])
        _close("padded prompt", got[1, 9:], want[1, 9:])
        for t in range(70, 74):
            # steps 70 and 72 pass the mask in its four-dimensional form [batch, 1, queries, tokens] (qwennha.py:133-136)
            mk = mask[:, :t + 1] if t % 2 else mask[:, None, None, :t + 1]
            got, _ = m(x[:, t:t + 1].to(dev), attention_mask=mk.to(dev), position_ids=pos[:, t:t + 1].to(dev),
                       past_key_value=cache, use_cache=True)
            _close(f"padded step {t}", got, ref.forward(x[:, t:t + 1], pos[:, t:t + 1], rc, attention_mask=mask[:, :t + 1]))


def test_gate_initialisation_from_keys_on_a_module():
    from nha_amd.hybrid import HybridNHAConfig, LlamaNativeHybridAttention, init_gates_from_keys
    cfg = HybridNHAConfig(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=32, num_slots=16, window_size=16)
    m = LlamaNativeHybridAttention(cfg, 0)
    assert init_gates_from_keys(m) == 1
    ref = F.avg_pool1d(m.k_proj.weight.detach().T[:, None, :], kernel_size=2, stride=2)[:, 0].T
    assert torch.allclose(m.g_proj.weight.detach(), ref, atol=1e-6)
