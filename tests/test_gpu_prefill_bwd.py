"""Backward of chunk_nha on the GPU (nha_prefill_bwd through autograd) against reverse-mode
differentiation of the fp64 recurrence (oracle.nha_ref.prefill_grad_ref, pinned by finite
differences on the CPU).  The inputs the oracle sees are the rounded tensors the kernels see.

Tolerances: fp32 tensors 1e-4 of each gradient's scale (max norm), as for the forward; bf16 tensors
(gradients are returned in bf16, o and do enter in bf16): relative L2 error <= 1e-2 -- half the
reference's own 2e-2 relative-L2 bar against fp64 (scripts/verify_opt_parity.py:753) -- and every
element within 3e-2 of the gradient's max norm."""
import pytest
import torch

from oracle import nha_ref as R
from tests.util import prefill_inputs

pytestmark = pytest.mark.gpu

KEYS = ["q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g"]
BF = torch.bfloat16


def check_grad(name, got, ref, dtype, rel_bar=1e-2):
    got = got.detach().double().cpu()
    ref = ref.detach().double()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    scale = max(ref.abs().max().item(), 1e-30)
    err = (got - ref).abs().max().item()
    if dtype == BF:
        rel = ((got - ref).norm() / max(ref.norm().item(), 1e-30)).item()
        assert rel <= rel_bar, f"{name}: relative L2 error {rel:.3e}"
        assert err <= 3e-2 * scale, f"{name}: max err {err:.3e} vs scale {scale:.3e}"
    else:
        assert err <= 1e-4 * scale, f"{name}: max err {err:.3e} vs scale {scale:.3e}"


def run_bwd_case(tag, d, *, wl, shift, dtype, cu=None, scale=None, with_lse=False, with_dht=False, impl=None, seed=0,
                 dg_bar=1e-2):
    from nha_amd import chunk_nha
    print("case", tag, dtype, flush=True)
    gen = torch.Generator().manual_seed(seed)
    B, T, HQ, _ = d["q_swa"].shape
    H, V, M = d["v"].shape[2], d["v"].shape[3], d["s"].shape[3]
    N = B if cu is None else len(cu) - 1
    K = d["q_swa"].shape[3]
    do = torch.randn(B, T, HQ, V, generator=gen).to(dtype)
    dl1 = torch.randn(B, T, HQ, generator=gen) if with_lse else None
    dl2 = torch.randn(B, T, HQ, generator=gen) if with_lse else None
    dht = (torch.randn(N, H, K, M, generator=gen), torch.randn(N, H, M, V, generator=gen)) if with_dht else None
    h0 = d.get("h0")
    x = [d[k].cuda().requires_grad_(True) for k in KEYS]
    h0c = None if h0 is None else tuple(t.cuda().requires_grad_(True) for t in h0)
    out = chunk_nha(*x, cu_seqlens=None if cu is None else torch.tensor(cu, dtype=torch.int32).cuda(), scale=scale,
                    window_size_left=wl, gsa_kv_shift=shift, initial_state=h0c, output_final_state=with_dht, impl=impl)
    loss = (out[0].float() * do.cuda().float()).sum()
    if with_lse:
        loss = loss + (out[1] * dl1.cuda()).sum() + (out[2] * dl2.cuda()).sum()
    if with_dht:
        loss = loss + (out[3][0] * dht[0].cuda()).sum() + (out[3][1] * dht[1].cuda()).sum()
    loss.backward()
    G = R.prefill_grad_ref(*[d[k] for k in KEYS], do, window_size_left=wl, gsa_kv_shift=shift, cu_seqlens=cu,
                           initial_state=h0, scale=scale, dlse_swa=dl1, dlse_gsa=dl2, dht=dht)
    for k, t in zip(KEYS, x):
        assert t.grad is not None and t.grad.dtype == dtype, k
        check_grad(f"{tag} d{k}", t.grad, G["d" + k], dtype, dg_bar if k == "g" else 1e-2)
    if h0 is not None:
        # fp32 tensors, but computed from the same rounded o / do as the other gradients
        check_grad(f"{tag} dh0k", h0c[0].grad, G["dh0k"], dtype)
        check_grad(f"{tag} dh0v", h0c[1].grad, G["dh0v"], dtype)


@pytest.mark.parametrize("dtype", [torch.float32, BF])
def test_bwd_small_grid(dtype):
    """Both call conventions, GQA and not, chunk-ragged lengths, with and without initial state."""
    seed = 7000
    for T, W, NG, M in ((63, 32, 1, 16), (130, 64, 4, 64), (257, 100, 2, 64)):
        H, K, V = 2, 64, 64
        d = prefill_inputs(seed, 2, T, H * NG, H, K, V, M, dtype=dtype, qk_scale=1.0, with_state=(T == 130))
        seed += 1
        run_bwd_case(f"T{T} shifted", d, wl=W - 1, shift=W, dtype=dtype, scale=K ** -0.5)
        run_bwd_case(f"T{T} layer", d, wl=W, shift=0, dtype=dtype, scale=K ** -0.5)


@pytest.mark.parametrize("dtype", [torch.float32, BF])
def test_bwd_all_cotangents_and_varlen(dtype):
    """Cotangents on both LSEs and on the final states, packed sequences (one shorter than the
    shift, one ending mid-chunk), initial states, K != V."""
    cu = [0, 70, 90, 300, 333]
    d = prefill_inputs(7100, 1, cu[-1], 4, 2, 32, 64, 32, dtype=dtype, qk_scale=1.0, with_state=True, N=4)
    run_bwd_case("varlen shifted", d, wl=31, shift=32, dtype=dtype, cu=cu, scale=32 ** -0.5, with_lse=True, with_dht=True)
    run_bwd_case("varlen layer", d, wl=48, shift=0, dtype=dtype, cu=cu, scale=32 ** -0.5, with_lse=True, with_dht=True)
    run_bwd_case("varlen unbounded window", d, wl=-1, shift=5, dtype=dtype, cu=cu, scale=32 ** -0.5, with_dht=True)


def test_bwd_head_dims_of_the_models():
    """D = 128 (hybrid LLM heads, 4 and 8 query heads per kv-head) and D = 256 (the 340M layer)."""
    d = prefill_inputs(7200, 1, 200, 8, 2, 128, 128, 64, dtype=BF, qk_scale=128 ** -0.5, gate_div=1.0, gate_mean=-1.0)
    run_bwd_case("D128 GQA", d, wl=63, shift=64, dtype=BF, impl="mfma")
    d = prefill_inputs(7201, 2, 150, 2, 2, 256, 256, 64, dtype=BF, qk_scale=256 ** -0.5)
    run_bwd_case("D256", d, wl=64, shift=0, dtype=BF, impl="mfma")
    # eight query heads per kv-head (the MoE hybrid's grouping), packed sequences that end inside a group of four
    # chunks, inside a chunk and on a chunk boundary: the window gradients come from the LDS-direct kernels
    cu = [0, 300, 364, 900]
    d = prefill_inputs(7202, 1, cu[-1], 16, 2, 128, 128, 64, dtype=BF, qk_scale=128 ** -0.5, gate_div=1.0, gate_mean=-1.0, N=3)
    run_bwd_case("D128 NG8 varlen", d, wl=200, shift=0, dtype=BF, impl="mfma", cu=cu)


@pytest.mark.parametrize("HQ,D,M", [(4, 64, 16), (8, 128, 64)])
@pytest.mark.parametrize("wl,shift", [(-1, 0), (5, 6), (31, 32), (45, 0), (63, 64), (64, 0), (200, 201), (1000, 0)])
def test_bwd_window_edges_on_the_matrix_cores(wl, shift, HQ, D, M):
    """bf16, K == V: the window gradients come from the matrix-core kernels (at D = 128 with four query
    heads per kv-head dq_swa comes from the kernel that streams the window through LDS-direct units).
    Packed ragged sequences (1 token, mid-chunk ends, longer than several key tiles), windows shorter
    than a 32-key half tile, not a multiple of it, longer than every sequence, and unbounded."""
    cu = [0, 1, 66, 130, 450, 519]
    d = prefill_inputs(7400 + wl + D, 1, cu[-1], HQ, 2, D, D, M, dtype=BF, qk_scale=1.0, with_state=True, N=5)
    run_bwd_case(f"window wl={wl} D={D}", d, wl=wl, shift=shift, dtype=BF, cu=cu, scale=D ** -0.5, with_dht=True)


@pytest.mark.parametrize("gate_mean", [-1.0, -2.0, -4.0])
def test_bwd_strong_gates(gate_mean):
    """Gate logits N(gate_mean, 1) -> logsigmoid without the /8: a 32-row half of a chunk decays by
    about e^-45 / e^-70 / e^-130.  Up to e^-70 the matrix-core slot kernels factor the decay
    around the half's start; beyond, the state export flags the chunk and the fp32 VALU kernels
    take it.  Mixed within one call for gate_mean = -2 (some slots cross the bound, most do not).
    dg is a telescoping sum (large per-row terms that cancel against the final-state term); with a
    cotangent on the final states and gates this strong its relative L2 error in bf16 reaches
    1.4e-2, so that one gradient is held to the reference's own 2e-2 bar
    (scripts/verify_opt_parity.py:753) in the first case; everything else stays at 1e-2."""
    cu = [0, 130, 300]
    d = prefill_inputs(7600, 1, cu[-1], 4, 2, 64, 64, 64, dtype=BF, qk_scale=64 ** -0.5, gate_div=1.0, gate_mean=gate_mean,
                       with_state=True, N=2)
    run_bwd_case(f"strong gates {gate_mean} shifted", d, wl=31, shift=32, dtype=BF, cu=cu, with_dht=True, dg_bar=2e-2)
    run_bwd_case(f"strong gates {gate_mean} layer", d, wl=40, shift=0, dtype=BF, cu=cu, with_lse=False)


def test_bwd_matrix_core_path_matches_fp32_path_at_size():
    """A size the CPU recurrence cannot differentiate in seconds (B=2, T=1536, 8/2 heads, D=128,
    W=512, both conventions): the bf16 call (matrix-core state recomputation and window kernels)
    against the fp32 call (generic kernels only) on the same bf16-rounded inputs and cotangent."""
    from nha_amd import chunk_nha
    B, T, HQ, H, D, M, W = 2, 1536, 8, 2, 128, 64, 512
    d = prefill_inputs(7500, B, T, HQ, H, D, D, M, dtype=BF, qk_scale=D ** -0.5, gate_div=1.0, gate_mean=-1.0)
    do = torch.randn(B, T, HQ, D, generator=torch.Generator().manual_seed(3)).to(BF)
    for wl, shift in ((W - 1, W), (W, 0)):
        grads = []
        for dt in (BF, torch.float32):
            x = [d[k].cuda().to(dt).requires_grad_(True) for k in KEYS]
            o = chunk_nha(*x, window_size_left=wl, gsa_kv_shift=shift)[0]
            o.backward(do.cuda().to(dt))
            grads.append([t.grad for t in x])
        for k, gb, gf in zip(KEYS, *grads):
            check_grad(f"size wl={wl} d{k}", gb, gf.double().cpu(), BF)


def test_bwd_window_longer_than_64_key_units_against_the_oracle():
    """wl = 2047 on a 2300-token sequence at head size 128 with four query heads per kv-head, against reverse-mode
    differentiation of the fp64 recurrence: the LDS-direct window-gradient kernels with a window of more than 64
    units of 32 keys (a workgroup of the key-side kernel owns four chunks and pairs the first and last query units
    of its range), rows with a full window and rows that still see the start of the sequence, a ragged last chunk."""
    T, W = 2300, 2048
    d = prefill_inputs(7700, 1, T, 4, 1, 128, 128, 64, dtype=BF, qk_scale=128 ** -0.5, gate_div=1.0, gate_mean=-1.0)
    run_bwd_case("wl 2047 shifted", d, wl=W - 1, shift=W, dtype=BF)


def test_bwd_long_context_heads_with_the_real_window_against_the_fp32_call():
    """The long-context head shape with its own window (32 / 8 heads, D = 128, M = 64, W = 2048, shifted convention,
    gate logits N(-1, 1), one 4096-token sequence): every gradient of the bf16 call (matrix-core kernels) against
    the fp32 call (generic fp32 kernels only) on the same bf16-rounded inputs and cotangent."""
    from nha_amd import chunk_nha
    B, T, HQ, H, D, M, W = 1, 4096, 32, 8, 128, 64, 2048
    d = prefill_inputs(7800, B, T, HQ, H, D, D, M, dtype=BF, qk_scale=D ** -0.5, gate_div=1.0, gate_mean=-1.0)
    do = torch.randn(B, T, HQ, D, generator=torch.Generator().manual_seed(4)).to(BF)
    grads = []
    for dt in (BF, torch.float32):
        x = [d[k].cuda().to(dt).requires_grad_(True) for k in KEYS]
        o = chunk_nha(*x, window_size_left=W - 1, gsa_kv_shift=W)[0]
        o.backward(do.cuda().to(dt))
        grads.append([t.grad for t in x])
        del x, o
    for k, gb, gf in zip(KEYS, *grads):
        check_grad(f"long context d{k}", gb, gf.double().cpu(), BF)


def test_bwd_rejects_unsupported_shapes():
    from nha_amd import NhaError, chunk_nha
    d = prefill_inputs(7300, 1, 64, 2, 2, 64, 64, 128, dtype=torch.float32)
    x = [d[k].cuda().requires_grad_(True) for k in KEYS]
    out = chunk_nha(*x, window_size_left=16, gsa_kv_shift=0)
    with pytest.raises(NhaError, match="M <= 64"):
        out[0].sum().backward()
