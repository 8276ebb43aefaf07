"""Shared helpers for the parity tests: seeded inputs with the reference's distributions
(scripts/verify_opt_parity.py:198-256) and the tolerance checks."""
import torch
import torch.nn.functional as F


def randn(gen, *shape, dtype=torch.bfloat16, scale=1.0):
    return (torch.randn(*shape, generator=gen, dtype=torch.float32) * scale).to(dtype)


def prefill_inputs(seed, B, T, HQ, H, K, V, M, dtype=torch.bfloat16, gate_div=8.0, gate_mean=0.0, qk_scale=1.0,
                   with_state=False, N=None, state_scale=0.5):
    gen = torch.Generator().manual_seed(seed)
    d = dict(
        q_gsa=randn(gen, B, T, HQ, K, dtype=dtype, scale=qk_scale),
        k_gsa=randn(gen, B, T, H, K, dtype=dtype, scale=qk_scale),
        v=randn(gen, B, T, H, V, dtype=dtype, scale=qk_scale),
        q_swa=randn(gen, B, T, HQ, K, dtype=dtype, scale=qk_scale),
        k_swa=randn(gen, B, T, H, K, dtype=dtype, scale=qk_scale),
    )
    g = (F.logsigmoid(torch.randn(B, T, H, M, generator=gen) + gate_mean) / gate_div).to(dtype)
    d["g"] = g
    d["s"] = (1 - g.float().exp()).to(dtype)
    if with_state:
        n = B if N is None else N
        d["h0"] = (randn(gen, n, H, K, M, dtype=torch.float32, scale=state_scale),
                   randn(gen, n, H, M, V, dtype=torch.float32, scale=state_scale))
    return d


def assert_close(name, got, ref, dtype):
    """bf16: 2e-2 abs / 1e-2 rel element by element.  fp32: 1e-4 relative element by element, with an
    absolute floor of 2e-6 of the tensor's largest magnitude (the rounding noise of fp32 sums of that
    size; elements that cancel to nearly zero have no meaningful relative error)."""
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    diff = (got - ref).abs()
    if dtype == torch.bfloat16:
        bad = diff > (2e-2 + 1e-2 * ref.abs())
        assert not bad.any(), f"{name}: {int(bad.sum())} elements out of tolerance, max abs err {diff.max():.3e}"
    else:
        scale = max(ref.abs().max().item(), 1e-30)
        bad = diff > (1e-4 * ref.abs() + 2e-6 * scale)
        assert not bad.any(), (f"{name}: {int(bad.sum())} elements out of tolerance, worst excess "
                               f"{(diff - 1e-4 * ref.abs()).max().item() / scale:.3e} of the scale {scale:.3e}")
    return diff.max().item()
