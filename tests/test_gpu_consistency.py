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
