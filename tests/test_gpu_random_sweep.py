"""Seeded random sweeps of the three ops against the fp64 oracle, through the C ABI: head sizes, groupings, batch and
packed layouts, sequence lengths around the chunk edges (1, 2, 15..17, 63..65, 127..129, ...), windows and slot shifts
around the tile edges, gate distributions, initial states, call forms.  The draws are fixed by the seeds, so a failure
names its case; the grids of the other test files cover the reference's own cases, this file the combinations between
them.  (The reference has no counterpart: scripts/verify_opt_parity.py walks fixed grids only.)"""
import random

import numpy as np
import pytest
import torch

from oracle import nha_ref as R
from tests.test_gpu_decode import decode_inputs
from tests.test_gpu_prefill import run_case
from tests.util import assert_close, prefill_inputs

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
KEYS = ["q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g"]
EDGE_LENS = [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129]


def _layout(rnd, max_len, batches):
    """(B, T, cu, N): a batch of equal sequences, or one packed row of ragged ones."""
    nseq = rnd.choice([1, 1, 2, 3, 5])
    lens = [rnd.choice(EDGE_LENS + [255, 256, 257, rnd.randint(1, max_len)]) for _ in range(nseq)]
    if rnd.random() < 0.6:
        return 1, sum(lens), [0] + [int(x) for x in np.cumsum(lens)], nseq
    B = rnd.choice(batches)
    return B, lens[0], None, B


def test_prefill_forward_sweep():
    for i in range(160):
        rnd = random.Random(i)
        D = rnd.choice([64, 128, 128, 256])
        NG = rnd.choice([1, 2, 3, 4, 8])
        H = rnd.choice([1, 2, 3])
        B, T, cu, N = _layout(rnd, 700, [1, 2, 3])
        wl = rnd.choice([-1, 0, 1, 15, 31, 32, 63, 64, 65, 99, 127, 128, 255, 256, 511, 512, rnd.randint(0, 800)])
        shift = rnd.choice([0, 0, (wl + 1) if wl >= 0 else 0, rnd.randint(0, 300), 1, 64])
        gate_div = rnd.choice([8.0, 8.0, 1.0])
        gate_mean = rnd.choice([0.0, -1.0, -4.0]) if gate_div == 1.0 else 0.0
        with_state = rnd.random() < 0.5
        scale = rnd.choice([None, None, D ** -0.5 * 0.7])
        d = prefill_inputs(10_000 + i, B, T, H * NG, H, D, D, 64, dtype=BF, with_state=with_state, N=N, gate_div=gate_div,
                           gate_mean=gate_mean, qk_scale=D ** -0.5 if scale is None else 1.0, state_scale=0.3)
        run_case(f"sweep {i}: D{D} NG{NG} H{H} B{B} T{T} cu{cu} wl{wl} shift{shift} gates/{gate_div}{gate_mean:+} h0={with_state} "
                 f"scale={scale}", d, wl=wl, shift=shift, dtype=BF, impl="mfma", cu=cu, scale=scale)


def test_decode_sweep():
    """Both call forms of fused_recurrent_nha_decode (pre-rotated; raw keys + cos / sin tables) and the logits form, bf16
    and fp32, windows of 1 .. 3000 rows: every kernel of the decode dispatch, the rotary form of the matrix-core kernel
    over many blocks per wave included."""
    from nha_amd import fused_recurrent_nha, fused_recurrent_nha_decode
    for i in range(400):
        rnd = random.Random(i)
        dtype = rnd.choice([BF, BF, torch.float32])
        NG = rnd.choice([1, 2, 3, 4, 8])
        H = rnd.choice([1, 2, 3])
        K = rnd.choice([64, 128, 128, 256])
        M = rnd.choice([16, 32, 64, 64, 64, 80, 128])
        B = rnd.choice([1, 2, 3, 5])
        W = rnd.choice([1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 128, 255, 256, 257, 512, rnd.randint(1, 1200), rnd.randint(1, 3000)])
        tag = f"sweep {i}: {str(dtype)[6:]} NG{NG} H{H} K{K} M{M} B{B} W{W}"
        print("case", tag, flush=True)
        d = decode_inputs(30_000 + i, B, H, NG, K, K, M, W, dtype)
        c = {k: v.cuda() for k, v in d.items()}
        h0 = (d["hk0"], d["hv0"])
        o, (hk, hv) = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], s=c["s"], sw_k=c["sk"], sw_v=c["vw"],
                                                 initial_state=(c["hk0"].clone(), c["hv0"].clone()), output_final_state=True)
        ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sk"], d["vw"], sq=d["sq"], s=d["s"], initial_state=h0)
        assert_close(tag + " o", o, ro, dtype)
        assert_close(tag + " hk", hk, rhk, dtype)
        assert_close(tag + " hv", hv, rhv, dtype)
        o, (hk, hv) = fused_recurrent_nha_decode(q=c["q"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sw_k_raw"], sw_v=c["vw"], cos=c["cos"],
                                                 sin=c["sin"], initial_state=(c["hk0"].clone(), c["hv0"].clone()), output_final_state=True)
        ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sw_k_raw"], d["vw"], cos=d["cos"], sin=d["sin"], initial_state=h0)
        assert_close(tag + " rotary o", o, ro, dtype)
        assert_close(tag + " rotary hk", hk, rhk, dtype)
        assert_close(tag + " rotary hv", hv, rhv, dtype)
        o, p, (hk, hv) = fused_recurrent_nha(c["q"], c["k"], c["v"], c["sliding_window"], c["s"], c["g"],
                                             initial_state=(c["hk0"].clone(), c["hv0"].clone()), output_final_state=True)
        ro, rp, rhk, rhv = R.fused_recurrent_ref(d["q"], d["k"], d["v"], d["sliding_window"], d["s"], d["g"], initial_state=h0)
        assert_close(tag + " logits o", o, ro, dtype)
        assert_close(tag + " logits p", p, rp, dtype)
        assert_close(tag + " logits hk", hk, rhk, dtype)


@pytest.mark.parametrize("NG,H,K,B,W", [(8, 3, 64, 2, 256), (4, 2, 64, 5, 257), (3, 2, 128, 5, 1815), (4, 2, 128, 2, 256), (1, 3, 64, 3, 450)])
def test_decode_rotary_form_over_many_blocks(NG, H, K, B, W):
    """The table form at windows of several 32-row blocks per wave: each block's cos / sin pieces are requested one
    block ahead into a per-wave LDS area, and must have landed before the block's keys are rotated."""
    from nha_amd import fused_recurrent_nha_decode
    d = decode_inputs(4300 + NG + W, B, H, NG, K, K, 64, W, BF)
    c = {k: v.cuda() for k, v in d.items()}
    ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sw_k_raw"], d["vw"], cos=d["cos"], sin=d["sin"],
                                      initial_state=(d["hk0"], d["hv0"]))
    for rep in range(3):
        o, (hk, hv) = fused_recurrent_nha_decode(q=c["q"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sw_k_raw"], sw_v=c["vw"], cos=c["cos"],
                                                 sin=c["sin"], initial_state=(c["hk0"].clone(), c["hv0"].clone()), output_final_state=True)
        assert_close(f"rotary o (call {rep})", o, ro, BF)
        assert_close(f"rotary hv (call {rep})", hv, rhv, BF)


def _grad_close(name, got, ref, bar):
    got = got.detach().double().cpu()
    ref = ref.detach().double()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = (got - ref).norm().item()
    # a gradient that is zero in exact arithmetic comes out as rounding noise of its cancelling terms
    assert err <= bar * ref.norm().item() + 1e-5, f"{name}: |got - ref| = {err:.3e}, |ref| = {ref.norm().item():.3e}"


def test_prefill_backward_sweep():
    """Relative L2 per gradient: 1e-2 for the window gradients, dv and ds, as in the backward's own tests.  The slot
    queries' and keys' gradients and dg get 4e-2 here: the draws include windows of one or two keys and sequences of one
    or two tokens, where those gradients are small differences of the rounded terms (bf16 o, do and probabilities) and
    the fp32-math kernels on the same bf16 tensors are as far from the fp64 oracle (1e-2 .. 2.5e-2)."""
    from nha_amd import chunk_nha
    for i in range(80):
        rnd = random.Random(1000 + i)
        D = rnd.choice([64, 128, 128, 256])
        NG = rnd.choice([1, 2, 4, 4, 8, 3])
        H = rnd.choice([1, 2])
        B, T, cu, N = _layout(rnd, 500, [1, 2])
        wl = rnd.choice([-1, 0, 1, 31, 32, 63, 64, 65, 127, 128, 200, 255, 256, 300, rnd.randint(0, 600)])
        shift = rnd.choice([0, 0, (wl + 1) if wl >= 0 else 0, rnd.randint(0, 200), 1, 64])
        gate_div = rnd.choice([8.0, 8.0, 1.0])
        gate_mean = rnd.choice([0.0, -1.0]) if gate_div == 1.0 else 0.0
        with_state, with_lse, with_dht = rnd.random() < 0.5, rnd.random() < 0.4, rnd.random() < 0.4
        tag = (f"sweep {i}: D{D} NG{NG} H{H} B{B} T{T} cu{cu} wl{wl} shift{shift} gates/{gate_div}{gate_mean:+} h0={with_state} "
               f"dlse={with_lse} dht={with_dht}")
        print("case", tag, flush=True)
        HQ = H * NG
        d = prefill_inputs(20_000 + i, B, T, HQ, H, D, D, 64, dtype=BF, with_state=with_state, N=N, gate_div=gate_div,
                           gate_mean=gate_mean, qk_scale=1.0, state_scale=0.3)
        gen = torch.Generator().manual_seed(i)
        do = torch.randn(B, T, HQ, D, generator=gen).to(BF)
        dl1 = torch.randn(B, T, HQ, generator=gen) if with_lse else None
        dl2 = torch.randn(B, T, HQ, generator=gen) if with_lse else None
        dht = (torch.randn(N, H, D, 64, generator=gen), torch.randn(N, H, 64, D, generator=gen)) if with_dht else None
        h0 = d.get("h0")
        x = [d[k].cuda().requires_grad_(True) for k in KEYS]
        h0c = None if h0 is None else tuple(t.cuda().requires_grad_(True) for t in h0)
        out = chunk_nha(*x, cu_seqlens=None if cu is None else torch.tensor(cu, dtype=torch.int32).cuda(), scale=D ** -0.5,
                        window_size_left=wl, gsa_kv_shift=shift, initial_state=h0c, output_final_state=with_dht)
        loss = (out[0].float() * do.cuda().float()).sum()
        if with_lse:
            loss = loss + (out[1] * dl1.cuda()).sum() + (out[2] * dl2.cuda()).sum()
        if with_dht:
            loss = loss + (out[3][0] * dht[0].cuda()).sum() + (out[3][1] * dht[1].cuda()).sum()
        loss.backward()
        G = R.prefill_grad_ref(*[d[k] for k in KEYS], do, window_size_left=wl, gsa_kv_shift=shift, cu_seqlens=cu, initial_state=h0,
                               scale=D ** -0.5, dlse_swa=dl1, dlse_gsa=dl2, dht=dht)
        for k, t in zip(KEYS, x):
            _grad_close(f"{tag} d{k}", t.grad, G["d" + k], 4e-2 if k in ("q_gsa", "k_gsa", "g") else 1e-2)
        if h0 is not None:
            _grad_close(f"{tag} dh0k", h0c[0].grad, G["dh0k"], 1e-2)
            _grad_close(f"{tag} dh0v", h0c[1].grad, G["dh0v"], 1e-2)


def test_ring_decode_sweep():
    """Ring-buffer steps from drawn fill levels (empty, one short of full, full, wrapped several times), four steps
    each, every step and the final rings, counters and states against the oracle's ring recurrence."""
    import torch.nn.functional as F
    from nha_amd import NHARingState, ring_decode_step
    from tests.util import randn
    for i in range(120):
        rnd = random.Random(i)
        dtype = rnd.choice([BF, BF, torch.float32])
        NG, H, K = rnd.choice([1, 2, 3, 4, 8]), rnd.choice([1, 2, 3]), rnd.choice([32, 64, 128, 128, 256])
        M, B = rnd.choice([16, 64, 64, 64, 80]), rnd.choice([1, 2, 3, 4])
        W = rnd.choice([1, 2, 16, 31, 32, 33, 63, 64, 65, 128, 256, rnd.randint(1, 700)])
        HQ, V = H * NG, K
        gen = torch.Generator().manual_seed(40_000 + i)
        st = NHARingState.empty(B, H, K, V, M, W, dtype=dtype)
        st.hk.copy_(randn(gen, B, H, K, M, dtype=torch.float32, scale=0.1))
        st.hv.copy_(randn(gen, B, H, M, V, dtype=torch.float32, scale=0.1))
        st.ring_k.copy_(randn(gen, B, W, H, K, dtype=dtype))
        st.ring_kg.copy_(randn(gen, B, W, H, K, dtype=dtype))
        st.ring_v.copy_(randn(gen, B, W, H, V, dtype=dtype))
        st.ring_g.copy_((F.logsigmoid(torch.randn(B, W, H, M, generator=gen)) / 8).to(dtype))
        counts = torch.tensor([rnd.choice([0, 1, max(W - 2, 0), max(W - 1, 0), W, W + 1, 5 * W + 3, rnd.randint(0, 3 * W)])
                               for _ in range(B)], dtype=torch.int32)
        st.count.copy_(counts)
        tag = f"sweep {i}: {str(dtype)[6:]} NG{NG} H{H} K{K} M{M} B{B} W{W} counts{counts.tolist()}"
        print("case", tag, flush=True)
        ref = dict(hk=st.hk.cpu().double(), hv=st.hv.cpu().double(),
                   rings=tuple(x.cpu().double() for x in (st.ring_k, st.ring_kg, st.ring_v, st.ring_g)), count=counts.clone())
        for step in range(4):
            q, sq = randn(gen, B, HQ, K, dtype=dtype), randn(gen, B, HQ, K, dtype=dtype)
            kn, kgn, vn = randn(gen, B, H, K, dtype=dtype), randn(gen, B, H, K, dtype=dtype), randn(gen, B, H, V, dtype=dtype)
            gn = (F.logsigmoid(torch.randn(B, H, M, generator=gen)) / 8).to(dtype)
            o = ring_decode_step(st, q.cuda(), sq.cuda(), kn.cuda(), kgn.cuda(), vn.cuda(), gn.cuda())
            ro, ref["hk"], ref["hv"], ref["rings"] = R.decode_ring_ref(q, sq, kn, kgn, vn, gn, *ref["rings"], ref["count"],
                                                                       ref["hk"], ref["hv"])
            ref["count"] += 1
            assert_close(f"{tag} step {step} o", o, ro, dtype)
        assert torch.equal(st.count.cpu(), ref["count"])
        assert_close(tag + " hk", st.hk, ref["hk"], dtype)
        assert_close(tag + " hv", st.hv, ref["hv"], dtype)
        for got, want in zip((st.ring_k, st.ring_kg, st.ring_v, st.ring_g), ref["rings"]):
            assert torch.equal(got.cpu().double(), want), tag


def test_zero_sink_attention_sweep():
    """nha_sink_window_fwd against the restated zero-prefix window attention: windows of 1 .. 2048 keys, 0 .. 100 sinks,
    batches and packed sequences, four to twelve query heads per kv-head."""
    from nha_amd.ops import zero_sink_attention
    from oracle.hybrid_attention_ref import zero_sink_attention_ref
    for i in range(150):
        rnd = random.Random(i)
        D, H, NG = rnd.choice([64, 128, 128]), rnd.choice([1, 2, 3]), rnd.choice([4, 8, 4, 12])
        HQ = H * NG
        nseq = rnd.choice([1, 1, 2, 3, 4])
        lens = [rnd.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, rnd.randint(1, 600)]) for _ in range(nseq)]
        packed = rnd.random() < 0.5
        W = rnd.choice([1, 2, 20, 31, 32, 33, 63, 64, 65, 96, 100, 128, 255, 256, 257, 2048, rnd.randint(1, 700)])
        M = rnd.choice([0, 1, 16, 64, 64, 100])
        gen = torch.Generator().manual_seed(60_000 + i)
        if packed:
            cu = [0] + [int(x) for x in np.cumsum(lens)]
            B, T = 1, cu[-1]
        else:
            B, T, cu = rnd.choice([1, 2, 3]), lens[0], None
        tag = f"sweep {i}: D{D} H{H} NG{NG} B{B} T{T} cu{cu} W{W} sinks{M}"
        print("case", tag, flush=True)
        q = (torch.randn(B, T, HQ, D, generator=gen) * D ** -0.25).to(BF)
        k = (torch.randn(B, T, H, D, generator=gen) * D ** -0.25).to(BF)
        v = torch.randn(B, T, H, D, generator=gen).to(BF)
        got = zero_sink_attention(q.cuda(), k.cuda(), v.cuda(), W, M,
                                  cu_seqlens=None if cu is None else torch.tensor(cu, dtype=torch.int32).cuda())
        for a, b in [(0, T)] if cu is None else zip(cu[:-1], cu[1:]):
            ref = zero_sink_attention_ref(q[:, a:b].double(), k[:, a:b].double(), v[:, a:b].double(), W, M)
            assert_close(f"{tag} [{a},{b})", got[:, a:b], ref, BF)


def test_hybrid_block_stack_sweep():
    """Two-block stacks of the hybrid decoders' attention modules (both flavours; all-NHA and NHA + zero-sink; head shapes
    on the generic, the matrix-core and the LDS-direct kernels; zero-sink windows shorter than the prompt; left padding):
    a prompt, then single-token steps on the ring cache, against the restated modules."""
    from nha_amd import NHARingCache
    from nha_amd.hybrid import HybridNHAConfig, LlamaNativeHybridAttention, Qwen3MoeNativeHybridAttention
    from oracle.hybrid_attention_ref import HybridAttentionRef
    from tests.test_hybrid_modules import F64, _close, _run_ref_stack, _run_stack, _weights
    dev = torch.device("cuda:0")
    hidden = 128
    for i in range(60):
        rnd = random.Random(i)
        flavour = rnd.choice(["moe", "dense"])
        HQ, H, D, M = rnd.choice([(8, 2, 32, 16), (32, 4, 128, 64), (8, 2, 128, 64), (4, 4, 64, 64), (4, 2, 64, 64), (2, 2, 256, 64),
                                  (6, 2, 64, 64), (16, 2, 128, 64)])
        W = rnd.choice([16, 32, 64, 64, 48])
        mixed = rnd.random() < 0.5
        sink_window = rnd.choice([2048, 96, 40])
        B, T0, steps = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 17, 63, 64, 65, 128, rnd.randint(1, 300)]), rnd.choice([1, 3, 6])
        pad = rnd.random() < 0.4 and B > 1 and T0 > 4
        tag = f"sweep {i}: {flavour} HQ{HQ} H{H} D{D} M{M} W{W} mixed={mixed} sink window {sink_window} B{B} prompt {T0} steps {steps} pad={pad}"
        print("case", tag, flush=True)
        cfg = HybridNHAConfig(hidden_size=hidden, num_attention_heads=HQ, num_key_value_heads=H, head_dim=D, num_slots=M, window_size=W,
                              max_position_embeddings=4096, block_size=2 if mixed else None, transformer_idx=1 if mixed else None)
        cls = Qwen3MoeNativeHybridAttention if flavour == "moe" else LlamaNativeHybridAttention
        gen = torch.Generator().manual_seed(100_000 + i)
        layers, refs = [], []
        for li in range(2):
            w = _weights(gen, hidden, HQ, H, D, M, flavour == "moe")
            m = cls(cfg, layer_idx=li).to(BF)
            m.load_state_dict(w, strict=True)
            if not m.is_nha_layer:
                m.window_size = sink_window
            layers.append(m.to(dev).eval())
            refs.append(HybridAttentionRef(w, num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=M, window_size=m.window_size,
                                           qk_norm=flavour == "moe", round_to=BF))
        x = torch.randn(B, T0 + steps, hidden, generator=gen).to(BF)
        mask = torch.ones(B, T0 + steps, dtype=torch.long)
        if pad:
            mask[-1, : rnd.randint(1, T0 // 2)] = 0
        npad = int((mask[-1] == 0).sum())
        pos = (mask.cumsum(1) - 1).clamp(min=0)
        cache, ref_caches = NHARingCache(W), [{} for _ in refs]
        with torch.no_grad():
            mk = mask[:, :T0] if pad else None
            got = _run_stack(layers, x[:, :T0].to(dev), pos[:, :T0].to(dev), cache, None if mk is None else mk.to(dev))
            ref = _run_ref_stack(refs, x[:, :T0].to(F64), pos[:, :T0], ref_caches, mk)
            if B > 1:
                _close(tag + " prompt", got[:-1], ref[:-1])
            _close(tag + " prompt, last row", got[-1, npad:], ref[-1, npad:])
            for t in range(T0, T0 + steps):
                mk = mask[:, :t + 1] if pad else None
                got = _run_stack(layers, x[:, t:t + 1].to(dev), pos[:, t:t + 1].to(dev), cache, None if mk is None else mk.to(dev))
                ref = _run_ref_stack(refs, x[:, t:t + 1].to(F64), pos[:, t:t + 1], ref_caches, mk)
                _close(f"{tag} step {t}", got, ref)
