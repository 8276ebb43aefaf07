"""GPU parity of the decode kernels (through the C ABI via nha_amd.ops / nha_amd.ring) against
the fp64 oracle, on the reference's own case grid (scripts/verify_opt_parity.py:278-285, :322-329)."""
import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import nha_ref as R
from tests.util import assert_close, randn

pytestmark = pytest.mark.gpu

GRID = list(itertools.product((1, 4, 8), (16, 64, 80), (32, 64), (64, 128), (1, 4)))


def decode_inputs(seed, B, H, NG, K, V, M, W, dtype):
    gen = torch.Generator().manual_seed(seed)
    HQ = H * NG
    d = dict(q=randn(gen, B, 1, HQ, K, dtype=dtype), k=randn(gen, B, 1, H, K, dtype=dtype),
             v=randn(gen, B, 1, H, V, dtype=dtype), sliding_window=randn(gen, B, 1, HQ, W, dtype=dtype),
             hk0=randn(gen, B, H, K, M, dtype=torch.float32, scale=0.5),
             hv0=randn(gen, B, H, M, V, dtype=torch.float32, scale=0.5))
    d["g"] = (F.logsigmoid(torch.randn(B, 1, H, M, generator=gen)) / 8.0).to(dtype)
    d["s"] = (1 - d["g"].float().exp()).to(dtype)
    d["sw_k_raw"] = randn(gen, B, W, H, K, dtype=dtype)
    d["vw"] = randn(gen, B, W, H, V, dtype=dtype)
    inv = 1.0 / (10000.0 ** (torch.arange(0, K, 2, dtype=torch.float32) / K))
    fr = torch.outer(torch.arange(100, 100 + W, dtype=torch.float32), inv)
    emb = torch.cat([fr, fr], -1)
    d["cos"], d["sin"] = emb.cos().to(dtype)[None], emb.sin().to(dtype)[None]
    d["sq"] = R.rope_rotate_half(d["q"].float(), d["cos"][:, -1:].float(), d["sin"][:, -1:].float()).to(dtype)
    d["sk"] = R.rope_rotate_half(d["sw_k_raw"].float(), d["cos"].float(), d["sin"].float()).to(dtype)
    return d


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_grid(dtype):
    from nha_amd import fused_recurrent_nha, fused_recurrent_nha_decode
    dev = "cuda"
    for idx, (NG, M, W, K, B) in enumerate(GRID):
        H, V = 2, K
        d = decode_inputs(2000 + idx, B, H, NG, K, V, M, W, dtype)
        c = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}
        tag = f"ng{NG}_m{M}_w{W}_k{K}_b{B}"
        print("case", tag, dtype, flush=True)
        # eager mode: pre-rotated sq / sk, caller-supplied s
        o, (hkt, hvt) = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], s=c["s"],
                                                   sw_k=c["sk"], sw_v=c["vw"],
                                                   initial_state=(c["hk0"].clone(), c["hv0"].clone()),
                                                   output_final_state=True)
        ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sk"], d["vw"], sq=d["sq"], s=d["s"],
                                          initial_state=(d["hk0"], d["hv0"]))
        assert_close(tag + " o", o, ro, dtype)
        assert_close(tag + " hk", hkt, rhk, torch.float32 if dtype == torch.float32 else dtype)
        assert_close(tag + " hv", hvt, rhv, torch.float32 if dtype == torch.float32 else dtype)
        # rotary mode: raw q / keys + cos/sin, s recomputed in-kernel
        o2, (hk2, hv2) = fused_recurrent_nha_decode(q=c["q"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sw_k_raw"],
                                                    sw_v=c["vw"], cos=c["cos"], sin=c["sin"],
                                                    initial_state=(c["hk0"].clone(), c["hv0"].clone()),
                                                    output_final_state=True)
        ro2, rhk2, rhv2, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sw_k_raw"], d["vw"], cos=d["cos"],
                                             sin=d["sin"], initial_state=(d["hk0"], d["hv0"]))
        assert_close(tag + " rot o", o2, ro2, dtype)
        assert_close(tag + " rot hk", hk2, rhk2, torch.float32 if dtype == torch.float32 else dtype)
        # caller-supplied window logits
        o3, sc, (hk3, hv3) = fused_recurrent_nha(c["q"], c["k"], c["v"], c["sliding_window"], c["s"], c["g"],
                                                 initial_state=(c["hk0"].clone(), c["hv0"].clone()),
                                                 output_final_state=True)
        ro3, rsc, rhk3, rhv3 = R.fused_recurrent_ref(d["q"], d["k"], d["v"], d["sliding_window"], d["s"], d["g"],
                                                     initial_state=(d["hk0"], d["hv0"]))
        assert_close(tag + " fr o", o3, ro3, dtype)
        assert_close(tag + " fr p", sc, rsc, dtype)
        assert_close(tag + " fr hv", hv3, rhv3, torch.float32 if dtype == torch.float32 else dtype)


@pytest.mark.parametrize("B,H", [(16, 8), (8, 3), (24, 2), (5, 8)])
def test_decode_rotary_tables_of_their_own_per_sequence(B, H):
    """cos / sin tables [B, W, K] with different positions in every sequence (what a model's position embeddings
    are): the matrix-core kernel places all kv-heads of a sequence on one XCD when the batch is a multiple of 8 (its
    workgroups then read a sequence's table rows through one L2), so a wrong (sequence, head) of a workgroup would
    rotate with another sequence's rows.  Against the oracle, bf16, four query heads per kv-head."""
    from nha_amd import fused_recurrent_nha_decode
    dtype, NG, K, M, W = torch.bfloat16, 4, 128, 64, 200
    d = decode_inputs(4100 + B, B, H, NG, K, K, M, W, dtype)
    inv = 1.0 / (10000.0 ** (torch.arange(0, K, 2, dtype=torch.float32) / K))
    start = torch.arange(B, dtype=torch.float32) * 37.0 + 5.0          # first position of the window, per sequence
    pos = start[:, None] + torch.arange(W, dtype=torch.float32)[None]
    fr = pos[:, :, None] * inv[None, None]
    emb = torch.cat([fr, fr], -1)
    d["cos"], d["sin"] = emb.cos().to(dtype), emb.sin().to(dtype)
    c = {k: v.cuda() for k, v in d.items()}
    o, (hkt, hvt) = fused_recurrent_nha_decode(q=c["q"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sw_k_raw"], sw_v=c["vw"],
                                               cos=c["cos"], sin=c["sin"], initial_state=(c["hk0"], c["hv0"]),
                                               output_final_state=True)
    ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sw_k_raw"], d["vw"], cos=d["cos"], sin=d["sin"],
                                      initial_state=(d["hk0"], d["hv0"]))
    assert_close("per-sequence rotary o", o, ro, dtype)
    assert_close("per-sequence rotary hk", hkt, rhk, dtype)
    assert_close("per-sequence rotary hv", hvt, rhv, dtype)


def test_decode_long_window_streaming_kernel():
    """Long windows: the matrix-core kernel (bf16, M == 64, pre-rotated query) and, for the other
    cases, the single-pass streaming kernel that serves windows too long for logits in LDS."""
    from nha_amd import fused_recurrent_nha_decode
    for dtype, NG, W, K, M, rot in ((torch.bfloat16, 4, 3000, 128, 64, False), (torch.bfloat16, 2, 3000, 128, 32, False),
                                    (torch.bfloat16, 8, 2500, 64, 64, False), (torch.float32, 2, 5000, 64, 64, True)):
        print("case", dtype, NG, W, K, M, rot, flush=True)
        d = decode_inputs(77, 2, 2, NG, K, K, M, W, dtype)
        c = {k: v.cuda() for k, v in d.items()}
        if rot:
            o, (hkt, hvt) = fused_recurrent_nha_decode(q=c["q"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sw_k_raw"],
                                                       sw_v=c["vw"], cos=c["cos"], sin=c["sin"],
                                                       initial_state=(c["hk0"], c["hv0"]), output_final_state=True)
            ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sw_k_raw"], d["vw"], cos=d["cos"],
                                              sin=d["sin"], initial_state=(d["hk0"], d["hv0"]))
        else:
            o, (hkt, hvt) = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sk"],
                                                       sw_v=c["vw"], initial_state=(c["hk0"], c["hv0"]),
                                                       output_final_state=True)
            ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sk"], d["vw"], sq=d["sq"],
                                              initial_state=(d["hk0"], d["hv0"]))
        assert_close("long-window o", o, ro, dtype)
        assert_close("long-window hv", hvt, rhv, dtype)


@pytest.mark.parametrize("NG,W,B", [(1, 512, 3), (1, 31, 2), (2, 100, 2), (8, 64, 1)])
def test_decode_head_size_256(NG, W, B):
    """Head size 256 (the 340M layers: one query head per kv-head) in the window form with a pre-rotated query:
    served by the matrix-core kernel with one block of loads per wave and four waves per workgroup."""
    from nha_amd import fused_recurrent_nha_decode
    dtype, K, M = torch.bfloat16, 256, 64
    d = decode_inputs(4100 + NG + W, B, 2, NG, K, K, M, W, dtype)
    c = {k: v.cuda() for k, v in d.items()}
    o, (hkt, hvt) = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], s=c["s"], sw_k=c["sk"],
                                               sw_v=c["vw"], initial_state=(c["hk0"].clone(), c["hv0"].clone()),
                                               output_final_state=True)
    ro, rhk, rhv, _, _ = R.decode_ref(d["q"], d["k"], d["v"], d["g"], d["sk"], d["vw"], sq=d["sq"], s=d["s"],
                                      initial_state=(d["hk0"], d["hv0"]))
    assert_close("d256 o", o, ro, dtype)
    assert_close("d256 hk", hkt, rhk, dtype)
    assert_close("d256 hv", hvt, rhv, dtype)


def test_decode_state_aliasing_and_errors():
    from nha_amd import fused_recurrent_nha, fused_recurrent_nha_decode
    d = decode_inputs(7, 2, 2, 1, 64, 64, 16, 32, torch.bfloat16)
    c = {k: v.cuda() for k, v in d.items()}
    hk0, hv0 = c["hk0"].clone(), c["hv0"].clone()
    o, (hkt, hvt) = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sk"],
                                               sw_v=c["vw"], initial_state=(hk0, hv0), output_final_state=True)
    assert hkt.data_ptr() == hk0.data_ptr() and hvt.data_ptr() == hv0.data_ptr()      # in place when NG == 1
    assert not torch.equal(hk0, c["hk0"])
    o2, st = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sk"],
                                        sw_v=c["vw"], initial_state=(c["hk0"], c["hv0"]))
    assert st == (None, None)
    with pytest.raises(ValueError):
        fused_recurrent_nha(c["q"].expand(-1, 2, -1, -1), c["k"], c["v"], c["sliding_window"], c["s"], c["g"])
    with pytest.raises(AssertionError):
        fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], sw_k=c["sk"], sw_v=c["vw"],
                                   cos=c["cos"], sin=c["sin"])


@pytest.mark.parametrize("NG,K,M,W", [(4, 128, 64, 48), (1, 64, 16, 8), (8, 64, 80, 33), (2, 64, 64, 300), (8, 128, 64, 130),
                                      (1, 128, 64, 1), (1, 256, 64, 200), (4, 256, 64, 70), (8, 256, 64, 33)])
def test_ring_decode_steps(NG, K, M, W):
    """Consecutive ring-buffer steps from random fill levels == the oracle's ring recurrence."""
    from nha_amd import NHARingState, ring_decode_step
    dtype, B, H, V = torch.bfloat16, 3, 2, K
    HQ = H * NG
    gen = torch.Generator().manual_seed(99)
    st = NHARingState.empty(B, H, K, V, M, W, dtype=dtype)
    st.hk.copy_(randn(gen, B, H, K, M, dtype=torch.float32, scale=0.1))
    st.hv.copy_(randn(gen, B, H, M, V, dtype=torch.float32, scale=0.1))
    st.ring_k.copy_(randn(gen, B, W, H, K, dtype=dtype))
    st.ring_kg.copy_(randn(gen, B, W, H, K, dtype=dtype))
    st.ring_v.copy_(randn(gen, B, W, H, V, dtype=dtype))
    st.ring_g.copy_((F.logsigmoid(torch.randn(B, W, H, M, generator=gen)) / 8).to(dtype))
    counts = torch.tensor([0, max(W - 2, 0), 5 * W + 3], dtype=torch.int32)
    st.count.copy_(counts)
    ref = dict(hk=st.hk.cpu().double(), hv=st.hv.cpu().double(),
               rings=tuple(x.cpu().double() for x in (st.ring_k, st.ring_kg, st.ring_v, st.ring_g)),
               count=counts.clone())
    for step in range(6):
        q, sq = randn(gen, B, HQ, K, dtype=dtype), randn(gen, B, HQ, K, dtype=dtype)
        kn, kgn, vn = randn(gen, B, H, K, dtype=dtype), randn(gen, B, H, K, dtype=dtype), randn(gen, B, H, V, dtype=dtype)
        gn = (F.logsigmoid(torch.randn(B, H, M, generator=gen)) / 8).to(dtype)
        o = ring_decode_step(st, q.cuda(), sq.cuda(), kn.cuda(), kgn.cuda(), vn.cuda(), gn.cuda())
        ro, ref["hk"], ref["hv"], ref["rings"] = R.decode_ring_ref(q, sq, kn, kgn, vn, gn, *ref["rings"], ref["count"],
                                                                   ref["hk"], ref["hv"])
        ref["count"] += 1
        assert_close(f"ring step {step} o", o, ro, dtype)
    assert torch.equal(st.count.cpu(), ref["count"])
    assert_close("ring hk", st.hk, ref["hk"], dtype)
    assert_close("ring hv", st.hv, ref["hv"], dtype)
    assert torch.equal(st.ring_k.cpu().double(), ref["rings"][0])
    assert torch.equal(st.ring_g.cpu().double(), ref["rings"][3])


@pytest.mark.parametrize("W,lens,NG,K", [(32, (70, 20, 32), 4, 128), (64, (130, 64, 1), 1, 64), (48, (200,), 8, 64)])
def test_prefill_hands_over_to_ring_decode(W, lens, NG, K):
    """Packed prefill of the prompts -> NHARingState.from_prefill -> decode steps == the oracle's
    prefill of the extended sequences, row by row (prompts shorter than, equal to and longer than
    the window)."""
    import nha_amd
    from nha_amd import NHARingState, ring_decode_step
    from tests.util import prefill_inputs
    dtype, H, M, steps = torch.bfloat16, 2, 64, 5
    HQ, V = H * NG, K
    names = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")
    full = [prefill_inputs(40 + n, 1, L + steps, HQ, H, K, V, M, dtype=dtype) for n, L in enumerate(lens)]
    refs = [R.prefill_ref(*[d[k] for k in names], window_size_left=W - 1, gsa_kv_shift=W)[0] for d in full]
    packed = {k: torch.cat([d[k][:, :L] for d, L in zip(full, lens)], 1).cuda() for k in names}
    cu = torch.tensor([0] + list(itertools.accumulate(lens)), dtype=torch.int32)
    o, _, _, (hk, hv) = nha_amd.chunk_nha(*[packed[k] for k in names], window_size_left=W - 1, gsa_kv_shift=W,
                                           cu_seqlens=cu.cuda(), output_final_state=True)
    assert_close("prompt o", o, torch.cat([r[:, :L] for r, L in zip(refs, lens)], 1), dtype)
    st = NHARingState.from_prefill(packed["k_swa"], packed["k_gsa"], packed["v"], packed["g"], (hk, hv), W,
                                   cu_seqlens=cu.cuda())
    assert st.count.tolist() == list(lens) and st.ring_k.shape == (len(lens), W, H, K)
    for i in range(steps):
        row = lambda k: torch.stack([d[k][0, L + i] for d, L in zip(full, lens)]).cuda().contiguous()
        oi = ring_decode_step(st, row("q_gsa"), row("q_swa"), row("k_swa"), row("k_gsa"), row("v"), row("g"))
        assert_close(f"decode step {i}", oi, torch.stack([r[0, L + i] for r, L in zip(refs, lens)]), dtype)
    assert st.count.tolist() == [L + steps for L in lens]


def test_ring_state_from_fixed_length_prefill():
    """from_prefill on a [B,T,...] batch (no cu_seqlens): ring slot j % W holds token j of the last W
    tokens, the state is the prefill's final state, and the next decode step matches the oracle."""
    import nha_amd
    from nha_amd import NHARingState, ring_decode_step
    from tests.util import prefill_inputs
    dtype, B, T, H, NG, K, M, W = torch.bfloat16, 3, 75, 2, 2, 64, 64, 32
    HQ, V = H * NG, K
    names = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")
    d = prefill_inputs(7, B, T + 1, HQ, H, K, V, M, dtype=dtype)
    ref = R.prefill_ref(*[d[k] for k in names], window_size_left=W - 1, gsa_kv_shift=W)[0]
    c = {k: d[k][:, :T].contiguous().cuda() for k in names}
    _, _, _, (hk, hv) = nha_amd.chunk_nha(*[c[k] for k in names], window_size_left=W - 1, gsa_kv_shift=W,
                                          output_final_state=True)
    st = NHARingState.from_prefill(c["k_swa"], c["k_gsa"], c["v"], c["g"], (hk, hv), W)
    assert st.count.tolist() == [T] * B
    for j in range(T - W, T):
        assert torch.equal(st.ring_k[:, j % W], c["k_swa"][:, j]) and torch.equal(st.ring_g[:, j % W], c["g"][:, j])
    row = lambda k: d[k][:, T].contiguous().cuda()
    o = ring_decode_step(st, row("q_gsa"), row("q_swa"), row("k_swa"), row("k_gsa"), row("v"), row("g"))
    assert_close("first decode step", o, ref[:, T], dtype)
    with pytest.raises(ValueError):
        NHARingState.from_prefill(c["k_swa"], c["k_gsa"], c["v"], c["g"], (hk[:1], hv[:1]), W)


def test_ring_cache_follows_the_cat_shift_cache():
    """NHARingCache against a plain restatement of the reference cache's window semantics
    (nha_fla/models/nha_cache.py:87-131, :143-154): the time-ordered window is the last W tokens, the
    popped entry is the oldest one once the window is full, and the outputs equal the oracle's."""
    import nha_amd
    from nha_amd import NHARingCache
    from tests.util import prefill_inputs
    dtype, B, T0, steps, H, NG, K, M, W = torch.bfloat16, 2, 20, 30, 2, 2, 64, 64, 32
    HQ, V = H * NG, K
    names = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")
    d = prefill_inputs(3, B, T0 + steps, HQ, H, K, V, M, dtype=dtype)
    ref = R.prefill_ref(*[d[k] for k in names], window_size_left=W - 1, gsa_kv_shift=W)[0]
    c = {k: d[k][:, :T0].contiguous().cuda() for k in names}
    _, _, _, fs = nha_amd.chunk_nha(*[c[k] for k in names], window_size_left=W - 1, gsa_kv_shift=W, output_final_state=True)
    cache = NHARingCache(W)
    assert cache.get_seq_length(0) == 0 and cache.get_pop_kvf(0) == (None, None, None)
    cache.prefill(0, c["k_swa"], c["k_gsa"], c["v"], c["g"], fs)
    for i in range(steps):
        n = T0 + i                                            # tokens cached before this step
        assert cache.get_seq_length(0) == n
        lo = max(0, n - W)
        wk, wv, wg = cache.window(0)
        assert torch.equal(wk.cpu(), d["k_swa"][:, lo:n]) and torch.equal(wv.cpu(), d["v"][:, lo:n])
        pk, pv, pg = cache.get_pop_kvf(0, W)
        if n < W:
            assert pk is None
        else:                                                 # the oldest cached token leaves the window
            assert torch.equal(pk.cpu(), d["k_gsa"][:, lo:lo + 1].flatten(-2))
            assert torch.equal(pg.cpu(), d["g"][:, lo:lo + 1].flatten(-2))
        row = lambda k: d[k][:, n].contiguous().cuda()
        o = cache.decode(0, row("q_gsa"), row("q_swa"), row("k_swa"), row("k_gsa"), row("v"), row("g"))
        assert_close(f"cache step {i}", o, ref[:, n], dtype)
    legacy = cache.to_legacy_cache()
    assert legacy[0]["attn_state"][0].shape == (B, W, H * K) and legacy[0]["recurrent_state"][0].shape == (B, H, K, M)
    with pytest.raises(KeyError):
        cache[1]


def test_ring_decode_at_benchmark_shape():
    """Two steps of the benchmark's decode workload (B=128, 32/8 heads, D=128, M=64, W=1024: full
    windows at random ring positions) against the oracle's ring recurrence."""
    import bench
    from nha_amd import NHARingState, ring_decode_step
    cfg = bench.DECODE
    B, HQ, H, D, M, W = (cfg[k] for k in ("B", "HQ", "H", "D", "M", "W"))
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(21)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    st = NHARingState.empty(B, H, D, D, M, W, dtype=dtype)
    st.hk.copy_(r(B, H, D, M) * 0.1)
    st.hv.copy_(r(B, H, M, D) * 0.1)
    st.ring_k.copy_(r(B, W, H, D))
    st.ring_kg.copy_(r(B, W, H, D))
    st.ring_v.copy_(r(B, W, H, D))
    st.ring_g.copy_(F.logsigmoid(r(B, W, H, M)))
    counts = torch.randint(W, 3 * W, (B,), generator=gen, dtype=torch.int32)
    st.count.copy_(counts)
    ref = dict(hk=st.hk.cpu().double(), hv=st.hv.cpu().double(),
               rings=tuple(x.cpu().double() for x in (st.ring_k, st.ring_kg, st.ring_v, st.ring_g)), count=counts.clone())
    for step in range(2):
        q, sq = (r(B, HQ, D) * D ** -0.5).to(dtype), (r(B, HQ, D) * D ** -0.5).to(dtype)
        kn, kgn, vn = r(B, H, D).to(dtype), r(B, H, D).to(dtype), r(B, H, D).to(dtype)
        gn = F.logsigmoid(r(B, H, M)).to(dtype)
        o = ring_decode_step(st, q.cuda(), sq.cuda(), kn.cuda(), kgn.cuda(), vn.cuda(), gn.cuda())
        ro, ref["hk"], ref["hv"], ref["rings"] = R.decode_ring_ref(q, sq, kn, kgn, vn, gn, *ref["rings"], ref["count"],
                                                                   ref["hk"], ref["hv"])
        ref["count"] += 1
        assert_close(f"step {step} o", o, ro, dtype)
        rel = ((o.double().cpu() - ro).norm() / ro.norm()).item()
        assert rel <= 5e-3, f"step {step}: relative L2 error {rel:.3e}"
    assert_close("hk", st.hk, ref["hk"], dtype)
    assert_close("hv", st.hv, ref["hv"], dtype)


def test_ring_decode_benchmark_shape_partial_windows_16_steps():
    """The decode configuration as written: B=128 sequences, 32/8 heads, D=128, M=64, a W=1024 ring
    whose fill is drawn per sequence from [1, W] (some rings fill up and start popping within the
    run), state ~ N(0, 0.1), 16 consecutive steps, every step against the oracle's ring recurrence."""
    import bench
    from nha_amd import NHARingState, ring_decode_step
    cfg = bench.DECODE
    B, HQ, H, D, M, W = (cfg[k] for k in ("B", "HQ", "H", "D", "M", "W"))
    dtype, steps = torch.bfloat16, 16
    gen = torch.Generator().manual_seed(22)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    st = NHARingState.empty(B, H, D, D, M, W, dtype=dtype)
    st.hk.copy_(r(B, H, D, M) * 0.1)
    st.hv.copy_(r(B, H, M, D) * 0.1)
    st.ring_k.copy_(r(B, W, H, D))
    st.ring_kg.copy_(r(B, W, H, D))
    st.ring_v.copy_(r(B, W, H, D))
    st.ring_g.copy_(F.logsigmoid(r(B, W, H, M)))
    counts = torch.randint(0, W, (B,), generator=gen, dtype=torch.int32)    # fill after the first step in [1, W]
    counts[:8] = torch.tensor([0, 1, W - 1, W - 2, W - steps, W - 5, 63, 64], dtype=torch.int32)
    st.count.copy_(counts)
    ref = dict(hk=st.hk.cpu().double(), hv=st.hv.cpu().double(),
               rings=tuple(x.cpu().double() for x in (st.ring_k, st.ring_kg, st.ring_v, st.ring_g)), count=counts.clone())
    for step in range(steps):
        q, sq = (r(B, HQ, D) * D ** -0.5).to(dtype), (r(B, HQ, D) * D ** -0.5).to(dtype)
        kn, kgn, vn = r(B, H, D).to(dtype), r(B, H, D).to(dtype), r(B, H, D).to(dtype)
        gn = F.logsigmoid(r(B, H, M)).to(dtype)
        o = ring_decode_step(st, q.cuda(), sq.cuda(), kn.cuda(), kgn.cuda(), vn.cuda(), gn.cuda())
        ro, ref["hk"], ref["hv"], ref["rings"] = R.decode_ring_ref(q, sq, kn, kgn, vn, gn, *ref["rings"], ref["count"],
                                                                   ref["hk"], ref["hv"], dtype=torch.float32)
        ref["count"] += 1
        assert_close(f"step {step} o", o, ro, dtype)
        rel = ((o.double().cpu() - ro.double()).norm() / ro.double().norm()).item()
        assert rel <= 5e-3, f"step {step}: relative L2 error {rel:.3e}"
    assert torch.equal(st.count.cpu(), ref["count"])
    assert (ref["count"] > W).any() and (ref["count"] < W).any()
    assert_close("hk", st.hk, ref["hk"], dtype)
    assert_close("hv", st.hv, ref["hv"], dtype)
