"""Size-independent properties on the GPU, at shapes the CPU oracle cannot reach: the decode kernels
continue a prefill exactly where it stopped.  Prefill over T0 + n tokens must equal prefill over T0
tokens followed by n ring-buffer decode steps (outputs of the last n tokens and the final slot
states), in the shifted convention of the hybrid models (window = last W tokens, slots hold
everything older; nha_fla/ops/nha/chunk_fused.py:83-90, nha_fla/models/nha_cache.py:105-154)."""
import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_close

pytestmark = pytest.mark.gpu


def _inputs(seed, B, T, HQ, H, D, M):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, device="cuda", dtype=torch.float32)
    q_swa, q_gsa = (r(B, T, HQ, D).to(torch.bfloat16) for _ in range(2))
    k_swa, k_gsa, v = (r(B, T, H, D).to(torch.bfloat16) for _ in range(3))
    g = (F.logsigmoid(r(B, T, H, M)) / 8.0).to(torch.bfloat16)
    s = (1 - g.float().exp()).to(torch.bfloat16)
    return q_swa, k_swa, q_gsa, k_gsa, v, s, g


@pytest.mark.parametrize("B,HQ,H,D,M,W,T0,n", [
    (4, 32, 8, 128, 64, 256, 1024, 6),      # matrix-core decode kernel, 4 q-heads per kv-head
    (3, 8, 8, 64, 64, 100, 333, 5),         # one q-head per kv-head, ragged chunk and window sizes
    (2, 4, 2, 128, 32, 64, 200, 4),         # M != 64: VALU decode kernels, generic prefill kernels
    (128, 32, 8, 128, 64, 1024, 1088, 3),   # the decode benchmark's full shape
])
def test_decode_continues_prefill(B, HQ, H, D, M, W, T0, n):
    from nha_amd import NHARingState, chunk_nha, ring_decode_step
    T = T0 + n
    x = _inputs(1234 + B, B, T, HQ, H, D, M)
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = x
    o_full, _, _, (hk_full, hv_full) = chunk_nha(*x, window_size_left=W - 1, gsa_kv_shift=W, output_final_state=True)
    head = [t[:, :T0].contiguous() for t in x]
    _, _, _, (hk, hv) = chunk_nha(*head, window_size_left=W - 1, gsa_kv_shift=W, output_final_state=True)
    st = NHARingState.empty(B, H, D, D, M, W, dtype=torch.bfloat16)
    st.hk.copy_(hk)
    st.hv.copy_(hv)
    pos = torch.arange(T0 - W, T0, device="cuda")
    st.ring_k[:, pos % W] = k_swa[:, pos]
    st.ring_kg[:, pos % W] = k_gsa[:, pos]
    st.ring_v[:, pos % W] = v[:, pos]
    st.ring_g[:, pos % W] = g[:, pos]
    st.count.fill_(T0)
    for i in range(n):
        t = T0 + i
        o = ring_decode_step(st, q_gsa[:, t].contiguous(), q_swa[:, t].contiguous(), k_swa[:, t].contiguous(),
                             k_gsa[:, t].contiguous(), v[:, t].contiguous(), g[:, t].contiguous())
        assert_close(f"decode step {i} vs prefill row {t}", o, o_full[:, t], torch.bfloat16)
    assert int(st.count[0]) == T
    # bf16 chunk states inside the prefill against fp32 state updates in decode: relative to the
    # state's scale
    for name, a, b in (("hk", st.hk, hk_full), ("hv", st.hv, hv_full)):
        err = (a - b).abs().max().item()
        assert err <= 2e-2 * max(b.abs().max().item(), 1.0), f"{name}: {err}"


def test_workspace_cache_is_bounded_and_can_be_released():
    """The prefill workspace is one grow-only buffer per (device, stream): the cache keeps at most sixteen of them (least
    recently used leaves first) and `release_workspaces()` drops them all and reports what they held."""
    import nha_amd
    from nha_amd import ops
    from tests.util import prefill_inputs
    nha_amd.release_workspaces()
    d = prefill_inputs(1, 1, 200, 8, 2, 128, 128, 64, dtype=torch.bfloat16)
    keys = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")
    x = [d[k].cuda() for k in keys]
    ref = nha_amd.chunk_nha(*x, window_size_left=63, gsa_kv_shift=64)[0]
    assert len(ops._WORKSPACE) == 1
    streams = [torch.cuda.Stream() for _ in range(ops._WORKSPACE_MAX_STREAMS + 3)]
    for st in streams:
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            o = nha_amd.chunk_nha(*x, window_size_left=63, gsa_kv_shift=64)[0]
        torch.cuda.current_stream().wait_stream(st)
        assert torch.equal(o, ref)
    assert len(ops._WORKSPACE) == ops._WORKSPACE_MAX_STREAMS
    held = nha_amd.release_workspaces()
    assert held >= ops._WORKSPACE_MAX_STREAMS * (1 << 20) and len(ops._WORKSPACE) == 0
    assert torch.equal(nha_amd.chunk_nha(*x, window_size_left=63, gsa_kv_shift=64)[0], ref)


def test_float16_tensors_are_computed_in_float32():
    """float16 inputs (the reference's Triton kernels take them like any other dtype): the four stateless ops compute in
    float32 on the generic kernels and return o in float16.  Against the oracle on the float16 values: 2e-3 abs + 2e-3 rel
    (one float16 rounding of o), gradients in float16 within 1e-2 relative L2."""
    from nha_amd import chunk_nha, fused_chunk_nha_prefill, fused_recurrent_nha, fused_recurrent_nha_decode
    from oracle import nha_ref as R
    from tests.test_gpu_decode import decode_inputs
    from tests.util import prefill_inputs
    keys = ["q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g"]
    f16 = torch.float16

    def near(name, got, ref, atol=2e-3, rtol=2e-3):
        got, ref = got.detach().double().cpu(), ref.double()
        bad = (got - ref).abs() > atol + rtol * ref.abs()
        assert torch.isfinite(got).all() and not bad.any(), f"{name}: {int(bad.sum())} off, max {(got - ref).abs().max():.2e}"

    d = prefill_inputs(31, 2, 150, 8, 2, 64, 64, 64, dtype=torch.float32, qk_scale=64 ** -0.5, with_state=True)
    d = {k: (v.to(f16) if k in keys else v) for k, v in d.items()}
    x = [d[k].cuda().requires_grad_(True) for k in keys]
    h0 = tuple(t.cuda() for t in d["h0"])
    o, ls, lg, (hk, hv) = chunk_nha(*x, window_size_left=31, gsa_kv_shift=32, initial_state=h0, output_final_state=True)
    assert o.dtype == f16 and ls.dtype == torch.float32 and hk.dtype == torch.float32
    ro, rls, rlg, rhk, rhv = R.prefill_ref(*[d[k] for k in keys], window_size_left=31, gsa_kv_shift=32, initial_state=d["h0"])
    near("o", o, ro)
    near("lse_swa", ls, rls)
    near("lse_gsa", lg, rlg)
    near("hk", hk, rhk)
    near("hv", hv, rhv)
    gen = torch.Generator().manual_seed(1)
    do = torch.randn(o.shape, generator=gen).to(f16)
    (o.float() * do.cuda().float()).sum().backward()
    G = R.prefill_grad_ref(*[d[k] for k in keys], do, window_size_left=31, gsa_kv_shift=32, initial_state=d["h0"])
    for k, t in zip(keys, x):
        assert t.grad.dtype == f16
        rel = ((t.grad.double().cpu() - G["d" + k]).norm() / G["d" + k].norm()).item()
        assert rel <= 1e-2, (k, rel)
    with torch.no_grad():
        o2, (hk2, _) = fused_chunk_nha_prefill(x[2], x[3], x[4], x[0], x[1], x[5], x[6], window_size=32, initial_state=h0,
                                               output_final_state=True)
    assert o2.dtype == f16
    near("fused prefill o", o2, ro)
    near("fused prefill hk", hk2, rhk)
    # the single-token ops
    dd = decode_inputs(5, 2, 2, 4, 64, 64, 64, 40, torch.float32)
    dd = {k: (v.to(f16) if v.dtype == torch.float32 and k not in ("hk0", "hv0") else v) for k, v in dd.items()}
    c = {k: v.cuda() for k, v in dd.items()}
    o3, (hk3, hv3) = fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], s=c["s"], sw_k=c["sk"], sw_v=c["vw"],
                                                initial_state=(c["hk0"].clone(), c["hv0"].clone()), output_final_state=True)
    r3, rhk3, rhv3, _, _ = R.decode_ref(dd["q"], dd["k"], dd["v"], dd["g"], dd["sk"], dd["vw"], sq=dd["sq"], s=dd["s"],
                                        initial_state=(dd["hk0"], dd["hv0"]))
    assert o3.dtype == f16
    near("decode o", o3, r3)
    near("decode hv", hv3, rhv3)
    o4, p4, (hk4, hv4) = fused_recurrent_nha(c["q"], c["k"], c["v"], c["sliding_window"], c["s"], c["g"],
                                             initial_state=(c["hk0"].clone(), c["hv0"].clone()), output_final_state=True)
    r4, rp4, rhk4, rhv4 = R.fused_recurrent_ref(dd["q"], dd["k"], dd["v"], dd["sliding_window"], dd["s"], dd["g"],
                                                initial_state=(dd["hk0"], dd["hv0"]))
    assert o4.dtype == f16
    near("logits-form o", o4, r4)
    near("logits-form p", p4, rp4)
    near("logits-form hk", hk4, rhk4)


@pytest.mark.parametrize("NSEQ,HQ,H,D,W,parts,same_kernel", [
    (128, 32, 8, 128, 2048, 8, True),     # q, o: 8 GiB; k, v: 2 GiB -- the LDS-direct kernels with row addresses past 2^32 bytes
    (264, 32, 8, 128, 512, 11, False),    # k, v: 4.1 GiB -- past the LDS-direct kernels' 32-bit lane offsets: mfma_out_kernel
])
def test_calls_whose_tensors_pass_4_gib(NSEQ, HQ, H, D, W, parts, same_kernel):
    """Packed sequences of 8192 tokens, 1M and 2.2M tokens in one call, against the same sequences in calls of 16 / 24
    sequences each (sequences do not interact, so the split calls are the reference): bit-identical while the same
    kernels serve both, within one bf16 rounding of o where the large call falls back to the kernel with 64-bit
    offsets.  Inputs are drawn on the device."""
    from nha_amd import chunk_nha
    dev, L = "cuda:0", 8192
    T = NSEQ * L
    try:
        gen = torch.Generator(device=dev).manual_seed(NSEQ)

        def draw(width, scale):
            out = torch.empty(1, T, width[0], width[1], dtype=torch.bfloat16, device=dev)
            for a in range(0, T, T // 8):
                out[:, a:a + T // 8] = (torch.randn(1, T // 8, *width, device=dev, generator=gen) * scale).to(torch.bfloat16)
            return out
        q_swa, q_gsa = draw((HQ, D), D ** -0.5), draw((HQ, D), D ** -0.5)
        k_swa, k_gsa, v = draw((H, D), D ** -0.5), draw((H, D), D ** -0.5), draw((H, D), 1.0)
        g = (torch.nn.functional.logsigmoid(draw((H, 64), 1.0).float()) / 8).to(torch.bfloat16)
        s = (1 - g.float().exp()).to(torch.bfloat16)
        xs = (q_swa, k_swa, q_gsa, k_gsa, v, s, g)
        cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
        o, ls, lg, (hk, hv) = chunk_nha(*xs, cu_seqlens=cu, window_size_left=W - 1, gsa_kv_shift=W, output_final_state=True)
        per = NSEQ // parts
        cu_p = torch.arange(0, per * L + 1, L, dtype=torch.int32, device=dev)
        for pi in range(parts):
            a, b = pi * per * L, (pi + 1) * per * L
            o2, ls2, lg2, (hk2, hv2) = chunk_nha(*(x[:, a:b] for x in xs), cu_seqlens=cu_p, window_size_left=W - 1, gsa_kv_shift=W,
                                                 output_final_state=True)
            assert torch.equal(hk[pi * per:(pi + 1) * per], hk2) and torch.equal(hv[pi * per:(pi + 1) * per], hv2), pi
            if same_kernel:
                assert torch.equal(o[:, a:b], o2) and torch.equal(ls[:, a:b], ls2) and torch.equal(lg[:, a:b], lg2), pi
            else:
                assert (o[:, a:b].float() - o2.float()).abs().max().item() <= 4e-3, pi
                assert (ls[:, a:b] - ls2).abs().max().item() <= 2e-2 and (lg[:, a:b] - lg2).abs().max().item() <= 1e-4, pi
    except torch.cuda.OutOfMemoryError:
        pytest.skip("not enough free device memory for this case")
    finally:
        q_swa = q_gsa = k_swa = k_gsa = v = g = s = xs = o = ls = lg = hk = hv = None
        from nha_amd import release_workspaces
        release_workspaces()
        torch.cuda.empty_cache()


def test_ops_recorded_into_a_graph_replay_like_eager_calls():
    """The library issues kernels only (no allocation, copy, fill or synchronisation of its own), so the ops can be
    recorded into a HIP graph after one eager call (which builds the index tables and the workspace): a prefill with
    packed sequences and a decode step, five replays each on fresh input contents, with eager work and a
    synchronisation between replays, every replay bit-identical to the eager call on the same inputs."""
    from nha_amd import chunk_nha, fused_recurrent_nha_decode
    from tests.test_gpu_decode import decode_inputs
    from tests.util import prefill_inputs
    keys = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")
    cu = torch.tensor([0, 300, 301, 900], dtype=torch.int32, device="cuda")

    def fresh(seed):
        d = prefill_inputs(seed, 1, 900, 8, 2, 128, 128, 64, dtype=torch.bfloat16, qk_scale=128 ** -0.5, with_state=True, N=3)
        return [d[k].cuda() for k in keys], tuple(t.cuda() for t in d["h0"])

    def prefill(xs, h0):
        return chunk_nha(*xs, cu_seqlens=cu, window_size_left=199, gsa_kv_shift=200, initial_state=h0, output_final_state=True)

    xs, h0 = fresh(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        prefill(xs, h0)                                  # tables, workspace and kernel set-up outside the recording
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph):
        out = prefill(xs, h0)
    for rep in range(1, 6):
        ys, g0 = fresh(rep)
        with torch.no_grad():
            want = prefill(ys, g0)
        for a, b in zip(xs + list(h0), ys + list(g0)):
            a.copy_(b)
        graph.replay()
        torch.cuda.synchronize()
        got = (out[0], out[1], out[2], out[3][0], out[3][1])
        for name, x, y in zip(("o", "lse_swa", "lse_gsa", "hk", "hv"), got, (want[0], want[1], want[2], want[3][0], want[3][1])):
            assert torch.equal(x, y), (rep, name)
        _ = (ys[0].float().sum() + ys[4].float().sum()).item()      # eager work and a sync between replays

    def step(c):
        return fused_recurrent_nha_decode(q=c["q"], sq=c["sq"], k=c["k"], v=c["v"], g=c["g"], s=c["s"], sw_k=c["sk"], sw_v=c["vw"],
                                          initial_state=(c["hk0"], c["hv0"]), output_final_state=True)

    c = {k: v.cuda() for k, v in decode_inputs(50, 4, 2, 4, 128, 128, 64, 300, torch.bfloat16).items()}
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        step(c)
    torch.cuda.current_stream().wait_stream(side)
    graph2 = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph2):
        o, (hk, hv) = step(c)
    for rep in range(1, 6):
        d = {k: v.cuda() for k, v in decode_inputs(50 + rep, 4, 2, 4, 128, 128, 64, 300, torch.bfloat16).items()}
        with torch.no_grad():
            wo, (whk, whv) = step(d)
        for k in c:
            c[k].copy_(d[k])
        graph2.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, wo) and torch.equal(hk, whk) and torch.equal(hv, whv), rep
        _ = d["vw"].float().sum().item()
