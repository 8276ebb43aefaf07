"""Pins for oracle/nha_ref.py: each check compares the oracle with something that is NOT a
retyping of its own formula (library routine, explicit closed form, algebraic identity, an
independent evaluation order), chosen so that a dropped term, a wrong sign/index or a transposed
operand fails at least one of them."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import nha_ref as R

torch.manual_seed(0)
DT = torch.float64


def make(B, T, HQ, H, K, V, M, seed=0, gate_div=1.0, gate_mean=0.0):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=DT)
    q_swa, q_gsa = r(B, T, HQ, K), r(B, T, HQ, K)
    k_swa, k_gsa = r(B, T, H, K), r(B, T, H, K)
    v = r(B, T, H, V)
    g = F.logsigmoid(r(B, T, H, M) + gate_mean) / gate_div
    s = 1 - g.exp()
    return q_swa, k_swa, q_gsa, k_gsa, v, s, g


# ---------------------------------------------------------------------------------------------
# 1. library routine: with s == 0 and no initial state the slots are M zero-logit / zero-value
#    sinks, so the op is SDPA over [M zero keys | causal sliding window]
#    (the reference's own W>64 "zero-prefix" path, models/llama3_nha/llamanha.py:205-216)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("wl,shift", [(7, 8), (8, 0), (-1, 0), (0, 1), (100, 0)])
@pytest.mark.parametrize("NG", [1, 2])
def test_zero_slots_reduce_to_sdpa(wl, shift, NG):
    B, T, H, K, V, M = 2, 29, 2, 8, 6, 5
    HQ = H * NG
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = make(B, T, HQ, H, K, V, M, seed=1)
    s = torch.zeros_like(s)
    scale = 0.37
    o, lse_swa, lse_gsa, hk, hv = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g,
                                                 window_size_left=wl, gsa_kv_shift=shift, scale=scale)
    kk = torch.cat([torch.zeros(B, M, HQ, K, dtype=DT), k_swa.repeat_interleave(NG, 2)], 1)
    vv = torch.cat([torch.zeros(B, M, HQ, V, dtype=DT), v.repeat_interleave(NG, 2)], 1)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    win = (j <= i) & ((j >= i - wl) if wl >= 0 else (j <= i))
    mask = torch.cat([torch.ones(T, M, dtype=torch.bool), win], 1)
    ref = F.scaled_dot_product_attention(q_swa.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2),
                                         attn_mask=mask, scale=scale).transpose(1, 2)
    assert torch.allclose(o, ref, atol=1e-12, rtol=1e-10)
    assert torch.allclose(lse_gsa, torch.full_like(lse_gsa, math.log(M)), atol=1e-12)
    assert hk.abs().max() == 0 and hv.abs().max() == 0
    # lse_swa against an explicit masked logsumexp
    logits = torch.einsum("bihk,bjhk->bihj", q_swa, k_swa.repeat_interleave(NG, 2)) * scale
    logits = logits.masked_fill(~win[None, :, None, :], float("-inf"))
    assert torch.allclose(lse_swa, torch.logsumexp(logits, -1), atol=1e-12)


# ---------------------------------------------------------------------------------------------
# 2. closed form of the gated recurrence (no recursion): after absorbing tokens 0..n-1,
#    hk = h0*exp(G_n) + sum_j exp(G_n - G_{j+1}) k_j s_j^T,   G_i = sum_{l<i} g_l
# ---------------------------------------------------------------------------------------------
def closed_form_state(k, v, s, g, hk0, hv0, n):
    B, T, H, K = k.shape
    G = torch.cat([torch.zeros_like(g[:, :1]), g.cumsum(1)], 1)        # G[:, i] = sum_{l<i} g_l
    w = torch.exp(G[:, n:n + 1] - G[:, 1:n + 1])                       # [B,n,H,M]
    hk = hk0 * G[:, n].exp()[:, :, None, :] + torch.einsum("bjhk,bjhm->bhkm", k[:, :n], s[:, :n] * w)
    hv = hv0 * G[:, n].exp()[:, :, :, None] + torch.einsum("bjhm,bjhv->bhmv", s[:, :n] * w, v[:, :n])
    return hk, hv


@pytest.mark.parametrize("shift", [0, 5, 40])
def test_final_state_closed_form(shift):
    B, T, H, NG, K, V, M = 2, 37, 2, 2, 6, 5, 4
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = make(B, T, H * NG, H, K, V, M, seed=2)
    gen = torch.Generator().manual_seed(5)
    hk0 = torch.randn(B, H, K, M, generator=gen, dtype=DT)
    hv0 = torch.randn(B, H, M, V, generator=gen, dtype=DT)
    _, _, _, hk, hv = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=3,
                                    gsa_kv_shift=shift, initial_state=(hk0, hv0))
    n = max(0, T - shift)                                               # tokens 0..T-1-shift absorbed
    hk_c, hv_c = closed_form_state(k_gsa, v, s, g, hk0, hv0, n)
    assert torch.allclose(hk, hk_c, atol=1e-12) and torch.allclose(hv, hv_c, atol=1e-12)


def test_slot_logits_and_read_closed_form():
    """o and lse_gsa at one row against the explicit (non-recursive) state, window disabled via
    a -inf-like construction: with wl=0 the window is the token itself; subtract its known term."""
    B, T, H, NG, K, V, M = 1, 23, 2, 2, 5, 4, 3
    HQ = H * NG
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = make(B, T, HQ, H, K, V, M, seed=3)
    scale = 0.5
    shift = 2
    o, lse_swa, lse_gsa, _, _ = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=0,
                                               gsa_kv_shift=shift, scale=scale)
    z = torch.zeros
    for t in (0, 1, 2, 7, T - 1):
        n = max(0, t - shift + 1)
        hk, hv = closed_form_state(k_gsa, v, s, g, z(B, H, K, M, dtype=DT), z(B, H, M, V, dtype=DT), n)
        for hq in range(HQ):
            h = hq // NG
            ok = scale * q_gsa[0, t, hq] @ hk[0, h]                       # [M]
            sw = scale * (q_swa[0, t, hq] @ k_swa[0, t, h])               # own token only
            p = torch.softmax(torch.cat([ok, sw[None]]), 0)
            ref = p[:M] @ hv[0, h] + p[M] * v[0, t, h]
            assert torch.allclose(o[0, t, hq], ref, atol=1e-12)
            assert torch.allclose(lse_gsa[0, t, hq], torch.logsumexp(ok, 0), atol=1e-12)
            assert torch.allclose(lse_swa[0, t, hq], sw, atol=1e-12)


# ---------------------------------------------------------------------------------------------
# 3. special cases of the slot write
# ---------------------------------------------------------------------------------------------
def test_noop_pop_and_full_forget_and_ema():
    gen = torch.Generator().manual_seed(4)
    hk = torch.randn(2, 3, 4, dtype=DT, generator=gen)
    hv = torch.randn(2, 4, 5, dtype=DT, generator=gen)
    k = torch.randn(2, 3, dtype=DT, generator=gen)
    v = torch.randn(2, 5, dtype=DT, generator=gen)
    zero = torch.zeros(2, 4, dtype=DT)
    # dummy pop (models/qwen3_moe_nha/qwennha.py:153-160): exact no-op
    a, b = R.gsa_step(hk, hv, torch.zeros_like(k), torch.zeros_like(v), zero, zero)
    assert torch.equal(a, hk) and torch.equal(b, hv)
    # g -> -inf: the state becomes the last outer product
    g = torch.full((2, 4), -1e4, dtype=DT)
    a, b = R.gsa_step(hk, hv, k, v, 1 - g.exp(), g)
    assert torch.allclose(a, k[:, :, None].expand(2, 3, 4)) and torch.allclose(b, v[:, None, :].expand(2, 4, 5))
    # M == 1, K == V == 1: scalar EMA  h <- a h + (1-a) x
    h = torch.tensor([[[0.3]]], dtype=DT)
    x = torch.tensor([[2.0]], dtype=DT)
    gg = torch.tensor([[math.log(0.25)]], dtype=DT)
    a, _ = R.gsa_step(h, h.clone(), x, x, 1 - gg.exp(), gg)
    assert abs(a.item() - (0.25 * 0.3 + 0.75 * 2.0)) < 1e-15


# ---------------------------------------------------------------------------------------------
# 4. chunk form (independent evaluation order + two-branch LSE merge) == recurrence
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,BT", [(50, 16), (64, 64), (97, 64), (130, 32)])
@pytest.mark.parametrize("wl,shift", [(15, 16), (16, 0), (70, 0), (-1, 3)])
def test_chunked_equals_recurrent(T, BT, wl, shift):
    B, H, NG, K, V, M = 2, 2, 2, 8, 8, 6
    x = make(B, T, H * NG, H, K, V, M, seed=T + BT)
    gen = torch.Generator().manual_seed(9)
    h0 = (torch.randn(B, H, K, M, generator=gen, dtype=DT), torch.randn(B, H, M, V, generator=gen, dtype=DT))
    a = R.prefill_ref(*x, window_size_left=wl, gsa_kv_shift=shift, initial_state=h0)
    b = R.prefill_chunked_ref(*x, window_size_left=wl, gsa_kv_shift=shift, initial_state=h0, chunk_size=BT)
    for u, w in zip(a, b):
        assert torch.allclose(u, w, atol=1e-10, rtol=1e-10)


def test_strong_gates_do_not_overflow():
    """g as low as -10 per token: every decay exponent used must be non-positive."""
    B, T, H, NG, K, V, M = 1, 130, 1, 1, 8, 8, 4
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = make(B, T, H * NG, H, K, V, M, seed=11)
    g = g * 0 - 10.0 + torch.rand_like(g)
    s = 1 - g.exp()
    a = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=8, gsa_kv_shift=0)
    b = R.prefill_chunked_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=8, gsa_kv_shift=0)
    for u, w in zip(a, b):
        assert torch.isfinite(u).all() and torch.allclose(u, w, atol=1e-10, rtol=1e-9)


# ---------------------------------------------------------------------------------------------
# 5. varlen packing == each sequence on its own
# ---------------------------------------------------------------------------------------------
def test_packed_equals_per_sequence():
    lens = [1, 20, 3, 2, 33]                                # incl. lengths 1, 2 (tests/test_varlen.py:66,73)
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    T, H, NG, K, V, M = cu[-1], 2, 2, 6, 6, 5
    x = make(1, T, H * NG, H, K, V, M, seed=12)
    gen = torch.Generator().manual_seed(13)
    N = len(lens)
    h0 = (torch.randn(N, H, K, M, generator=gen, dtype=DT), torch.randn(N, H, M, V, generator=gen, dtype=DT))
    o, ls, lg, hk, hv = R.prefill_ref(*x, window_size_left=4, gsa_kv_shift=5, cu_seqlens=cu, initial_state=h0)
    for n in range(N):
        sl = slice(cu[n], cu[n + 1])
        xs = [t[:, sl] for t in x]
        o1, ls1, lg1, hk1, hv1 = R.prefill_ref(*xs, window_size_left=4, gsa_kv_shift=5,
                                                initial_state=(h0[0][n:n + 1], h0[1][n:n + 1]))
        assert torch.equal(o[:, sl], o1) and torch.equal(hk[n], hk1[0]) and torch.equal(hv[n], hv1[0])
    # a sequence no longer than the shift leaves its state untouched (ops/nha/chunk.py:75-76)
    assert torch.equal(hk[0], h0[0][0]) and torch.equal(hk[2], h0[0][2]) and torch.equal(hk[3], h0[0][3])


# ---------------------------------------------------------------------------------------------
# 6. decode == last row of a prefill in the shifted convention (window W, slots <= t-W)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,W", [(20, 6), (6, 6), (5, 6)])
def test_decode_matches_prefill_last_row(T, W):
    B, H, NG, K, V, M = 2, 2, 3, 8, 5, 4
    HQ = H * NG
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = make(B, T, HQ, H, K, V, M, seed=20 + T)
    full = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=W - 1, gsa_kv_shift=W)
    xs = [t[:, :T - 1] for t in (q_swa, k_swa, q_gsa, k_gsa, v, s, g)]
    _, _, _, hk, hv = R.prefill_ref(*xs, window_size_left=W - 1, gsa_kv_shift=W)
    t = T - 1
    lo = max(0, t - W + 1)
    if t - W >= 0:
        kp, vp, gp = k_gsa[:, t - W:t - W + 1], v[:, t - W:t - W + 1], g[:, t - W:t - W + 1]
    else:
        kp, vp, gp = torch.zeros(B, 1, H, K, dtype=DT), torch.zeros(B, 1, H, V, dtype=DT), torch.zeros(B, 1, H, M, dtype=DT)
    o, hk1, hv1, pm, pw = R.decode_ref(q_gsa[:, t:t + 1], kp, vp, gp, k_swa[:, lo:t + 1], v[:, lo:t + 1],
                                       sq=q_swa[:, t:t + 1], initial_state=(hk, hv))
    assert torch.allclose(o[:, 0], full[0][:, t], atol=1e-12)
    assert torch.allclose(hk1, full[3], atol=1e-12) and torch.allclose(hv1, full[4], atol=1e-12)
    assert torch.allclose(pm.sum(-1) + pw.sum(-1), torch.ones(B, HQ, dtype=DT), atol=1e-12)


def test_ring_decode_matches_prefill():
    """Run T tokens through the ring-buffer step from an empty cache == prefill rows."""
    B, T, W, H, NG, K, V, M = 2, 19, 5, 2, 2, 6, 4, 3
    HQ = H * NG
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = make(B, T, HQ, H, K, V, M, seed=31)
    full = R.prefill_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, window_size_left=W - 1, gsa_kv_shift=W)
    z = lambda *sh: torch.zeros(*sh, dtype=DT)
    rings = (z(B, W, H, K), z(B, W, H, K), z(B, W, H, V), z(B, W, H, M))
    hk, hv = z(B, H, K, M), z(B, H, M, V)
    for t in range(T):
        o, hk, hv, rings = R.decode_ring_ref(q_gsa[:, t], q_swa[:, t], k_swa[:, t], k_gsa[:, t], v[:, t], g[:, t],
                                             *rings, [t] * B, hk, hv)
        assert torch.allclose(o, full[0][:, t], atol=1e-12)
    assert torch.allclose(hk, full[3], atol=1e-12) and torch.allclose(hv, full[4], atol=1e-12)


# ---------------------------------------------------------------------------------------------
# 7. RoPE: rotate-half with duplicated halves == complex rotation of (x_j, x_{j+K/2}) pairs
# ---------------------------------------------------------------------------------------------
def test_rope_is_complex_rotation_and_decode_rotary_mode():
    B, W, H, NG, K, V, M = 2, 7, 2, 2, 8, 4, 3
    HQ = H * NG
    gen = torch.Generator().manual_seed(40)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=DT)
    inv = 1.0 / (10000.0 ** (torch.arange(0, K, 2, dtype=DT) / K))
    pos = torch.arange(100, 100 + W, dtype=DT)
    fr = torch.outer(pos, inv)
    emb = torch.cat([fr, fr], -1)
    cos, sin = emb.cos()[None], emb.sin()[None]
    x = r(B, W, H, K)
    y = R.rope_rotate_half(x, cos, sin)
    xc = torch.complex(x[..., :K // 2], x[..., K // 2:]) * torch.polar(torch.ones_like(fr), fr)[None, :, None, :]
    assert torch.allclose(y, torch.cat([xc.real, xc.imag], -1), atol=1e-12)
    # rotary mode of decode == eager mode on pre-rotated tensors; relative-position property
    q, k, v, g = r(B, 1, HQ, K), r(B, 1, H, K), r(B, 1, H, V), F.logsigmoid(r(B, 1, H, M))
    sw_v = r(B, W, H, V)
    h0 = (r(B, H, K, M), r(B, H, M, V))
    a = R.decode_ref(q, k, v, g, x, sw_v, cos=cos, sin=sin, initial_state=h0)
    sq = R.rope_rotate_half(q, cos[:, -1:], sin[:, -1:])
    b = R.decode_ref(q, k, v, g, y, sw_v, sq=sq, initial_state=h0)
    assert torch.allclose(a[0], b[0], atol=1e-12)
    emb2 = torch.cat([torch.outer(pos + 17, inv)] * 2, -1)       # shifting all positions: same logits
    c = R.decode_ref(q, k, v, g, x, sw_v, cos=emb2.cos()[None], sin=emb2.sin()[None], initial_state=h0)
    assert torch.allclose(a[0], c[0], atol=1e-9)


# ---------------------------------------------------------------------------------------------
# 8. fused_recurrent (caller-supplied window logits) == decode with those logits
# ---------------------------------------------------------------------------------------------
def test_fused_recurrent_consistent_with_decode():
    B, W, H, NG, K, V, M = 2, 6, 2, 2, 8, 4, 5
    HQ = H * NG
    gen = torch.Generator().manual_seed(50)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=DT)
    q, sq, k, v = r(B, 1, HQ, K), r(B, 1, HQ, K), r(B, 1, H, K), r(B, 1, H, V)
    g = F.logsigmoid(r(B, 1, H, M)); s = 1 - g.exp()
    swk, swv = r(B, W, H, K), r(B, W, H, V)
    h0 = (r(B, H, K, M), r(B, H, M, V))
    scale = K ** -0.5
    o, hk, hv, pm, pw = R.decode_ref(q, k, v, g, swk, swv, sq=sq, s=s, initial_state=h0)
    logits = torch.einsum("bqk,bwqk->bqw", sq[:, 0] * scale, swk.repeat_interleave(NG, 2))[:, None]
    o2, p2, hk2, hv2 = R.fused_recurrent_ref(q, k, v, logits, s, g, initial_state=h0)
    assert torch.allclose(p2[:, 0], pw, atol=1e-12)
    o_full = o2[:, 0] + torch.einsum("bqw,bwqv->bqv", p2[:, 0], swv.repeat_interleave(NG, 2))
    assert torch.allclose(o_full, o[:, 0], atol=1e-12) and torch.allclose(hk, hk2) and torch.allclose(hv, hv2)


@pytest.mark.parametrize("wl,shift,varlen", [(2, 3, False), (3, 0, False), (-1, 1, False), (2, 3, True), (4, 0, True)])
def test_gradients_match_finite_differences(wl, shift, varlen):
    """prefill_grad_ref against central differences of prefill_ref (the forward is pinned above;
    this pins the plumbing of the gradient oracle: cotangents of o, both LSEs and the final states,
    every input incl. the initial state, batched and packed).  A dropped cotangent, a wrong
    sequence slice or a missing un-shift fails it."""
    torch.manual_seed(11)
    f64 = torch.float64
    HQ, H, K, V, M = 4, 2, 4, 6, 3
    if varlen:
        cu, B, T = [0, 5, 6, 13], 1, 13        # one sequence shorter than the shift
        N = 3
    else:
        cu, B, T = None, 2, 9
        N = B
    r = lambda *s: torch.randn(*s, dtype=f64)
    g = F.logsigmoid(r(B, T, H, M))
    x = [r(B, T, HQ, K), r(B, T, H, K), r(B, T, HQ, K), r(B, T, H, K), r(B, T, H, V), 1 - g.exp() + 0.1 * r(B, T, H, M), g]
    h0 = (r(N, H, K, M), r(N, H, M, V))
    do, dl1, dl2 = r(B, T, HQ, V), r(B, T, HQ), r(B, T, HQ)
    dht = (r(N, H, K, M), r(N, H, M, V))
    kw = dict(window_size_left=wl, gsa_kv_shift=shift, cu_seqlens=cu)
    G = R.prefill_grad_ref(*x, do, initial_state=h0, dlse_swa=dl1, dlse_gsa=dl2, dht=dht, **kw)

    def f(xs, h):
        o, ls, lg, hk, hv = R.prefill_ref(*xs, initial_state=h, **kw)
        return float((o * do).sum() + (ls * dl1).sum() + (lg * dl2).sum() + (hk * dht[0]).sum() + (hv * dht[1]).sum())

    eps = 1e-6
    names = ["q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g"]
    gen = torch.Generator().manual_seed(5)
    for i, nm in enumerate(names + ["h0k", "h0v"]):
        tgt = x[i] if i < 7 else h0[i - 7]
        for _ in range(6):
            idx = tuple(int(torch.randint(0, d, (1,), generator=gen)) for d in tgt.shape)
            xp, xm = [t.clone() for t in x], [t.clone() for t in x]
            hp, hm = [t.clone() for t in h0], [t.clone() for t in h0]
            (xp[i] if i < 7 else hp[i - 7])[idx] += eps
            (xm[i] if i < 7 else hm[i - 7])[idx] -= eps
            fd = (f(xp, tuple(hp)) - f(xm, tuple(hm))) / (2 * eps)
            an = float(G["d" + nm][idx])
            assert abs(fd - an) <= 1e-6 * max(1.0, abs(fd)), (nm, idx, fd, an)
    if varlen and shift >= 1:
        # tokens of a sequence no longer than the shift never reach the slots: no slot-branch gradient
        assert G["dk_gsa"][0, 5:6].abs().max() == 0 and G["dg"][0, 5:6].abs().max() == 0


def test_layer_glue_against_library_routines_and_invariants():
    """Pins layer_prologue_ref / layer_epilogue_ref without retyping them: torch's sigmoid and
    rms_norm routines, the complex-number form of RoPE, its norm and relative-position invariants."""
    torch.manual_seed(11)
    B, T, HQ, H, K, V, M = 2, 9, 4, 2, 8, 6, 5
    r = lambda *s: torch.randn(*s, dtype=DT)
    q, k, v, f = r(B, T, HQ, K), r(B, T, H, K), r(B, T, H, V), 3 * r(B, T, H, M)
    pos = torch.arange(T) + 7
    q_swa, k_swa, q_gsa, k_gsa, vo, s, g = R.layer_prologue_ref(q, k, v, f, feature_map="swish", gate_logit_normalizer=8,
                                                                positions=pos, rope_theta=10000.0)
    # gates: exp(normalizer * g) is the library sigmoid, s + exp(g) = 1, g <= 0
    assert torch.allclose((8 * g).exp(), torch.sigmoid(f), atol=1e-12)
    assert torch.allclose(s + g.exp(), torch.ones_like(s), atol=1e-14) and (g <= 0).all() and (s >= 0).all()
    assert torch.allclose(vo, v * torch.sigmoid(v), atol=1e-12) and torch.allclose(q_gsa, q * torch.sigmoid(q), atol=1e-12)
    assert torch.equal(R.layer_prologue_ref(q, k, v, f, feature_map="relu", gate_logit_normalizer=8, positions=pos)[3],
                       k.clamp_min(0))
    assert R.layer_prologue_ref(q, k, v, f, feature_map=None, gate_logit_normalizer=8, positions=pos)[2] is q
    # RoPE: (x1 + i x2) * exp(i * pos * theta^(-2j/K)), norms kept, scores depend on pos differences only
    inv = 10000.0 ** (-torch.arange(0, K, 2, dtype=DT) / K)
    z = torch.complex(q[..., : K // 2], q[..., K // 2:]) * torch.polar(torch.ones(T, K // 2, dtype=DT),
                                                                        (pos[:, None].float() * inv.float()).double())[None, :, None, :]
    assert torch.allclose(torch.cat([z.real, z.imag], -1), q_swa, atol=1e-12)
    assert torch.allclose(q_swa.norm(dim=-1), q.norm(dim=-1), atol=1e-12)
    q2, k2 = R.layer_prologue_ref(q, k, v, f, feature_map=None, gate_logit_normalizer=8, positions=pos + 100)[:2]
    sc1 = torch.einsum("bihk,bjhk->bhij", q_swa[:, :, :H], k_swa)
    sc2 = torch.einsum("bihk,bjhk->bhij", q2[:, :, :H], k2)
    assert torch.allclose(sc1, sc2, atol=1e-4)             # the angle is formed in float32: 1e-5-level drift at pos ~100
    # epilogue: torch's rms_norm on silu(o)
    o, w, b = r(B, T, HQ * V), r(HQ * V), r(HQ * V)
    ref = F.rms_norm(F.silu(o), (HQ * V,), weight=w, eps=1e-5) + b
    assert torch.allclose(R.layer_epilogue_ref(o, w, b, 1e-5), ref, atol=1e-12)
    y = R.layer_epilogue_ref(o, None, None, 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(B, T, dtype=DT), atol=1e-12)


@pytest.mark.parametrize("wl,shift,varlen,NG", [(15, 16, False, 2), (16, 0, True, 1), (-1, 3, True, 4), (0, 1, False, 1)])
def test_c_restatement_matches_torch_oracle(wl, shift, varlen, NG):
    """oracle/nha_ref_c.c (plain C, written independently of the torch code: explicit loops, one task
    per q-head carrying its kv-head's recurrence) against prefill_ref on random cases: both
    conventions, GQA, packed sequences shorter and longer than window and shift, initial states.
    float32 in and out, so agreement to float32 rounding."""
    from oracle.nha_ref_c import prefill_ref_c
    torch.manual_seed(7)
    H, K, V, M = 2, 12, 10, 7
    HQ = H * NG
    B, T = (1, 90) if varlen else (2, 45)
    cu = [0, 3, 40, 41, 90] if varlen else None
    N = 4 if varlen else B
    r = lambda *s: torch.randn(*s, dtype=torch.float32)
    g = F.logsigmoid(r(B, T, H, M))
    x = [r(B, T, HQ, K), r(B, T, H, K), r(B, T, HQ, K), r(B, T, H, K), r(B, T, H, V), 1 - g.exp(), g]
    h0 = (r(N, H, K, M), r(N, H, M, V))
    kw = dict(window_size_left=wl, gsa_kv_shift=shift, cu_seqlens=cu, initial_state=h0, scale=0.3)
    ref = R.prefill_ref(*x, **kw)
    got = prefill_ref_c(*x, **kw)
    for name, a, b in zip(("o", "lse_swa", "lse_gsa", "hkt", "hvt"), got, ref):
        assert a.dtype == torch.float32 and a.shape == b.shape, name
        assert (a.double() - b).abs().max() <= 2e-6 * max(1.0, b.abs().max().item()), name
    # zero slots and zero initial state: plain banded softmax attention from the library routine
    if wl >= 0 and not varlen:
        z = [x[0], x[1], x[2], x[3], x[4], torch.zeros_like(x[5]), x[6]]
        o = prefill_ref_c(*z, window_size_left=wl, gsa_kv_shift=shift, scale=0.3)[0]
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        band = (j <= i) & (j >= i - wl)
        kx = torch.cat([torch.zeros(B, M, H, K), x[1]], 1).repeat_interleave(NG, 2)     # M zero-logit, zero-value sinks
        vx = torch.cat([torch.zeros(B, M, H, V), x[4]], 1).repeat_interleave(NG, 2)
        mask = torch.cat([torch.ones(T, M, dtype=torch.bool), band], 1)
        sd = F.scaled_dot_product_attention(x[0].transpose(1, 2).double(), kx.transpose(1, 2).double(),
                                            vx.transpose(1, 2).double(), attn_mask=mask, scale=0.3).transpose(1, 2)
        assert (o.double() - sd).abs().max() <= 2e-6
