#!/usr/bin/env python3
"""Headline benchmark of the NHA hot path on ONE MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  `value` is prefill tokens/s of one NHA attention layer at the
long-context head shape (32 q heads, 8 kv heads, D=128, M=64 slots, W=2048, B=2) at T=8192,
bf16, whole op (state pass + output pass), inputs resident in HBM.  The same line carries the
decode leg (B=128 sequences, 32/8 heads, D=128, M=64, W=1024 ring buffer, 256 consecutive
steps, us/step), each with its roofline object, and the CPU baseline (the oracle's naive
per-token PyTorch recurrence timed on the host cores on a bounded sample).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_BF16_TFLOPS = 2500.0   # MI355X dense bf16
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E
# HBM bytes per launch of the two dominant kernels on the default workloads, from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE (KiB per dispatch) scaled by what the same counters read for a 256 MiB
# device-to-device copy (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0); the runs are summarised under
# profiles/.  Reported as `traffic` only while the workload is the one they were measured on.
TRAFFIC_BYTES = {
    "ring_out_kernel<128>": (256759.0 * 2.0 + 139275.0) * 1024,
    "decode_mfma_kernel<128,4,2>": (302939.0 * 2.0 + 67216.0) * 1024,
    "layer_prologue_kernel": (106610.8 * 2.0 + 393216.0) * 1024,
    "layer_epilogue_kernel": (65759.4 * 2.0 + 131072.0) * 1024,
}

# where each figure above comes from: the counters are read in separate rocprofv3 runs, not in this one
TRAFFIC_SOURCE = {
    "ring_out_kernel<128>": "profiles/ring_out_kernel_prefill_T8192.md (rocprofv3 --pmc, not measured in this run)",
    "decode_mfma_kernel<128,4,2>": "profiles/decode_mfma_kernel_B128_W1024.md (rocprofv3 --pmc, not measured in this run)",
}
OUT_KERNEL = "ring_out_kernel<128>"

# Seconds of back-to-back launches before every timed region, on top of the --warmup steps.  An idle
# MI355X parks its shader clock near 100 MHz and needs about a second of load to reach the level it then
# holds (2.3 GHz under the prefill here); the default 20 timed steps of 0.7 ms would otherwise be measured
# on the ramp (about 2.0 GHz on these boxes).  `--clock-warmup 0` switches it off.
CLOCK_WARM_S = 1.5


def keep_busy(torch, fn, seconds=None, batch=20):
    """Launch `fn` back to back for `seconds` of wall time (untimed)."""
    seconds = CLOCK_WARM_S if seconds is None else seconds
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(batch):
            fn()
        torch.cuda.synchronize()


PREFILL = dict(B=2, T=8192, HQ=32, H=8, D=128, M=64, W=2048)
DECODE = dict(B=128, HQ=32, H=8, D=128, M=64, W=1024, steps=256)
# the other prefill shapes of the reference's configurations (parity-test cases; `--workload NAME`
# times one of them with the same method as the headline).  wl/shift default to the shifted
# convention (W-1, W); "layer" = (W, 0).  cfg3 packs sequences of 64..4096 tokens into 32768.
# gate_mean: mean of the gate logits before logsigmoid (N(-1,1) for the long-context shapes, N(0,1)
# for the 340M-layer shapes); h0_std: standard deviation of the per-sequence initial slot states.
WORKLOADS = dict(
    headline=PREFILL,
    cfg2=dict(B=8, T=2048, HQ=4, H=4, D=256, M=64, W=512, wl=512, shift=0, gate_mean=0.0),
    cfg2_shifted=dict(B=8, T=2048, HQ=4, H=4, D=256, M=64, W=512, gate_mean=0.0),
    cfg3=dict(B=1, T=32768, HQ=4, H=4, D=256, M=64, W=512, wl=512, shift=0, varlen=True, gate_mean=0.0, h0_std=0.1),
    cfg5=dict(B=2, T=16384, HQ=32, H=8, D=128, M=64, W=2048),
    # the headline heads with the 64-token window of the hybrid models' NHA layers (the only regime of the
    # reference's fused inference prefill, which is limited to W <= 64)
    w64=dict(B=2, T=8192, HQ=32, H=8, D=128, M=64, W=64),
)


def w_eff(T, W):
    return sum(min(t + 1, W) for t in range(T)) / T


def prefill_flops(B, T, HQ, H, D, M, W):
    """Algorithmic (recurrent-form) flops: slot logits + slot read per q-head, window QK^T + PV
    per q-head over the in-window keys, slot write per kv-head."""
    return B * T * HQ * (2 * (D * M + M * D) + 2 * w_eff(T, W) * (D + D)) + B * T * H * 2 * (D * M + M * D)


def workload_lengths(torch, cfg):
    """Sequence lengths of a workload: B equal sequences, or (varlen) draws of 64..4096 tokens
    until T is filled, the last one truncated."""
    if not cfg.get("varlen"):
        return [cfg["T"]] * cfg["B"]
    gen = torch.Generator().manual_seed(0)
    lens = []
    while sum(lens) < cfg["T"]:
        lens.append(int(torch.randint(64, 4097, (1,), generator=gen)))
    lens[-1] -= sum(lens) - cfg["T"]
    return lens


def min_prefill_bytes(cfg, N):
    """Minimal HBM bytes of a prefill call: every operand read once, the output written once (bf16),
    initial states read when the workload has them."""
    B, T, HQ, H, D, M = (cfg[k] for k in ("B", "T", "HQ", "H", "D", "M"))
    b = 2 * B * T * (HQ * 3 * D + H * (3 * D + 2 * M))
    if cfg.get("h0_std"):
        b += 4 * N * H * 2 * D * M
    return b


def decode_bytes(B, HQ, H, D, M, W):
    """Algorithmic HBM bytes of one decode step: fp32 state read+write, bf16 K/V window read,
    q/o/new-token/popped-entry traffic."""
    state = 2 * 4 * B * H * (D * M + M * D)
    window = 2 * B * W * H * (D + D)
    small = 2 * B * (2 * HQ * D + HQ * D) + 2 * 2 * B * H * (3 * D + M)
    return state + window + small


def make_prefill_inputs(torch, cfg, device, seed=0, B=None, T=None):
    B = cfg["B"] if B is None else B
    T = cfg["T"] if T is None else T
    HQ, H, D, M = cfg["HQ"], cfg["H"], cfg["D"], cfg["M"]
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    q = (r(B, T, HQ, D) * D ** -0.5).to(torch.bfloat16)
    k = (r(B, T, H, D) * D ** -0.5).to(torch.bfloat16)
    v = (r(B, T, H, D) * D ** -0.5).to(torch.bfloat16)
    g = torch.nn.functional.logsigmoid(r(B, T, H, M) + cfg.get("gate_mean", -1.0)).to(torch.bfloat16)
    s = (1 - g.float().exp()).to(torch.bfloat16)
    # the window branch and the slot branch see different (rotated / raw) q and k in the hybrid
    # models; a second draw keeps the two operand streams distinct as they are in production
    q2 = (r(B, T, HQ, D) * D ** -0.5).to(torch.bfloat16)
    k2 = (r(B, T, H, D) * D ** -0.5).to(torch.bfloat16)
    return [x.to(device) for x in (q2, k2, q, k, v, s, g)]


def make_initial_state(torch, cfg, N, device, seed=4):
    """Per-sequence initial slot states ~ N(0, h0_std) of a workload that has them, else None."""
    if not cfg.get("h0_std"):
        return None
    gen = torch.Generator().manual_seed(seed)
    H, D, M = cfg["H"], cfg["D"], cfg["M"]
    return ((torch.randn(N, H, D, M, generator=gen) * cfg["h0_std"]).to(device),
            (torch.randn(N, H, M, D, generator=gen) * cfg["h0_std"]).to(device))


def bench_prefill(torch, steps, warmup, cfg=PREFILL, cold=False):
    """`cold`: no clock warm-up -- after a second of idling the same warm-up and timed steps start from the parked
    shader clock and are measured on its ramp (what a single call after a pause sees); returns the step time only."""
    import numpy as np
    from nha_amd import _lib
    from nha_amd.ops import prefill_tables, _ptr
    dev = torch.device("cuda:0")
    B, T, HQ, H, D, M, W = (cfg[k] for k in ("B", "T", "HQ", "H", "D", "M", "W"))
    wl, shift = cfg.get("wl", W - 1), cfg.get("shift", W)
    lens = workload_lengths(torch, cfg)
    xs = [x.reshape(B * T, *x.shape[2:]).contiguous() for x in make_prefill_inputs(torch, cfg, dev)]
    cu_host = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = len(lens)
    cu_d, idx_d, off_d, NT = prefill_tables(cu_host, dev)
    lib = _lib.load()
    o = torch.empty(B * T, HQ, D, dtype=torch.bfloat16, device=dev)
    lse_s = torch.empty(B * T, HQ, dtype=torch.float32, device=dev)
    lse_g = torch.empty(B * T, HQ, dtype=torch.float32, device=dev)
    hkt = torch.empty(N, H, D, M, dtype=torch.float32, device=dev)
    hvt = torch.empty(N, H, M, D, dtype=torch.float32, device=dev)
    a = _lib.NhaPrefillArgs()
    a.q_swa, a.k_swa, a.q_gsa, a.k_gsa, a.v, a.s, a.g = (_ptr(x) for x in xs)
    a.o, a.lse_swa, a.lse_gsa, a.hkt, a.hvt = _ptr(o), _ptr(lse_s), _ptr(lse_g), _ptr(hkt), _ptr(hvt)
    h0 = make_initial_state(torch, cfg, N, dev)
    if h0 is not None:
        a.h0k, a.h0v = _ptr(h0[0]), _ptr(h0[1])
    a.cu_seqlens, a.chunk_indices, a.chunk_offsets = _ptr(cu_d), _ptr(idx_d), _ptr(off_d)
    a.T_tot, a.N, a.NT, a.HQ, a.H, a.K, a.V, a.M = B * T, N, NT, HQ, H, D, D, M
    a.wl, a.shift, a.dtype, a.impl, a.scale = wl, shift, _lib.NHA_DTYPE_BF16, _lib.NHA_IMPL_MFMA, D ** -0.5
    stream = torch.cuda.current_stream(dev)
    a.stream = stream.cuda_stream
    nbytes = lib.nha_prefill_scratch_bytes(C.byref(a))
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    a.scratch, a.scratch_bytes = _ptr(scratch), nbytes

    # the library's measurement entry (exported, not in the public header): phase 1 = state pass, 2 = output pass
    lib.nha_internal_prefill_fwd_phase.restype = C.c_int
    lib.nha_internal_prefill_fwd_phase.argtypes = [C.c_void_p, C.c_int]

    def run(phase):
        if phase == 0:
            _lib.check(lib.nha_prefill_fwd(C.byref(a)))
        else:
            _lib.check(lib.nha_internal_prefill_fwd_phase(C.byref(a), phase))

    if cold:
        torch.cuda.synchronize()
        time.sleep(1.0)
    else:
        keep_busy(torch, lambda: run(0))
    for _ in range(warmup):
        run(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run(0)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    if cold:
        return dict(tokens_per_s=B * T / wall, ms_per_step=wall * 1e3)
    # per-kernel durations with events on the launch stream: state pass alone, output pass alone.  The
    # events of all steps are recorded before the host waits once, so the launches follow each other as
    # they do in the timed loop above
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for ev in evs:
        ev[0].record(stream)
        run(1)
        ev[1].record(stream)
        run(2)
        ev[2].record(stream)
    torch.cuda.synchronize()
    t_state = sum(ev[0].elapsed_time(ev[1]) for ev in evs) * 1e-3 / steps
    t_out = sum(ev[1].elapsed_time(ev[2]) for ev in evs) * 1e-3 / steps
    flops = sum(prefill_flops(1, L, HQ, H, D, M, wl + 1) for L in lens)
    # the output pass carries everything but the slot write (the state pass's flops)
    flops_out = flops - B * T * H * 2 * (D * M + M * D)
    return dict(tokens_per_s=B * T / wall, ms_per_step=wall * 1e3, t_state_ms=t_state * 1e3, t_out_ms=t_out * 1e3,
                flops=flops, achieved_tflops=flops_out / t_out / 1e12, whole_op_tflops=flops / wall / 1e12)


def bench_backward(torch, steps, warmup, cfg=PREFILL):
    """Backward of the prefill op (nha_prefill_bwd behind chunk_nha's autograd node) on the same
    synthetic inputs: milliseconds per call with HIP events on the launch stream.  Flops by the
    usual convention for attention backwards, 2.5 x the forward's (five matrix products for two)."""
    import numpy as np
    from nha_amd.ops import nha_prefill, nha_prefill_bwd
    dev = torch.device("cuda:0")
    B, T, HQ, H, D, M, W = (cfg[k] for k in ("B", "T", "HQ", "H", "D", "M", "W"))
    wl, shift = cfg.get("wl", W - 1), cfg.get("shift", W)
    lens = workload_lengths(torch, cfg)
    xs = [x.reshape(B * T, *x.shape[2:]).contiguous() for x in make_prefill_inputs(torch, cfg, dev)]
    cu_host = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    o, ls, lg, _, _ = nha_prefill(*xs, cu_host, wl=wl, shift=shift, scale=D ** -0.5, impl="mfma")
    gen = torch.Generator(device=dev).manual_seed(1)
    do = torch.randn(o.shape, generator=gen, device=dev, dtype=torch.float32).to(o.dtype)
    stream = torch.cuda.current_stream(dev)
    run = lambda: nha_prefill_bwd(*xs, o, ls, lg, do, cu_host, wl=wl, shift=shift, scale=D ** -0.5)
    keep_busy(torch, run, batch=5)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    tot = 0.0
    for _ in range(steps):
        ev[0].record(stream)
        run()
        ev[1].record(stream)
        torch.cuda.synchronize()
        tot += ev[0].elapsed_time(ev[1])
    ms = tot / steps
    flops = 2.5 * sum(prefill_flops(1, L, HQ, H, D, M, wl + 1) for L in lens)
    return dict(bwd_ms=ms, bwd_flops=flops, bwd_tflops=flops / (ms * 1e-3) / 1e12, bwd_tokens_per_s=B * T / (ms * 1e-3))


def bench_glue(torch, steps, warmup, cfg=PREFILL):
    """The two fused glue launches of the layer at the prefill workload's shape (raw projections ->
    op operands, op output -> input of the output projection): microseconds per launch with HIP
    events on the launch stream, and the algorithmic bytes (every element read / written once)."""
    from nha_amd.ops import nha_layer_epilogue, nha_layer_prologue
    dev = torch.device("cuda:0")
    B, T, HQ, H, D, M = (cfg[k] for k in ("B", "T", "HQ", "H", "D", "M"))
    gen = torch.Generator(device=dev).manual_seed(2)
    r = lambda *s: torch.randn(*s, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    q, k, v, f = r(B, T, HQ, D), r(B, T, H, D), r(B, T, H, D), r(B, T, H, M)
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32, device=dev) / D))
    o, w = r(B * T, HQ * D), torch.ones(HQ * D, device=dev)
    stream = torch.cuda.current_stream(dev)

    def timed(fn):
        keep_busy(torch, fn)
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record(stream)
        for _ in range(steps):
            fn()
        ev[1].record(stream)
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / steps * 1e3

    us_p = timed(lambda: nha_layer_prologue(q, k, v, f, inv, feature_map="swish", gate_logit_normalizer=8))
    us_e = timed(lambda: nha_layer_epilogue(o, w, None, 1e-5))
    by_p = 2 * (3 * q.numel() + 3 * k.numel() + 2 * v.numel() + 3 * f.numel())
    by_e = 2 * 2 * o.numel()
    return dict(prologue_us=us_p, prologue_bytes=by_p, prologue_gbs=by_p / us_p / 1e3,
                epilogue_us=us_e, epilogue_bytes=by_e, epilogue_gbs=by_e / us_e / 1e3)


def bench_layer(torch, steps, warmup):
    """NativeHybridAttention (hidden 1024, 4 heads of 256, 64 slots, window 512: the 340M layer) on
    B=8 T=2048 bf16: milliseconds per forward (autograd off) and per forward + backward, with the
    fused glue launches and with the tensor-op chain."""
    from nha_amd.layer import NativeHybridAttention
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    layer = NativeHybridAttention(hidden_size=1024, num_heads=4, num_kv_heads=4, num_slots=64, layer_idx=0,
                                  window_size=512).to(dev).to(torch.bfloat16)
    x = (torch.randn(8, 2048, 1024) * 0.5).to(torch.bfloat16).to(dev)
    stream = torch.cuda.current_stream(dev)

    def timed(fn):
        keep_busy(torch, fn)
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record(stream)
        for _ in range(steps):
            fn()
        ev[1].record(stream)
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / steps

    def fwd():
        with torch.no_grad():
            layer(x)

    def fwd_bwd():
        xg = x.detach().requires_grad_(True)
        y = layer(xg)[0]
        y.backward(torch.ones_like(y))

    out = {}
    for fuse in (True, False):
        layer.fuse_glue = fuse
        layer.eval()
        out[("fused" if fuse else "chain") + "_fwd_ms"] = timed(fwd)
        layer.train()
        layer._compression_stats = []
        out[("fused" if fuse else "chain") + "_fwd_bwd_ms"] = timed(fwd_bwd)
    return out


def bench_hybrid(torch, steps, warmup):
    """One attention block of the MoE-flavour hybrid decoder (hidden 2048, 32 query / 4 kv heads of 128, 64 slots),
    bf16, autograd off: the prompt (B=2, T=8192) through an NHA layer (window 64) and through a zero-sink layer
    (window 2048), and single-token steps at B=128 on the ring cache after a 256-token prompt -- each as the whole
    block (projection GEMMs, the glue launch, the attention kernels, the output projection) next to its parts timed
    alone, with the fused glue and with the tensor-op chain."""
    from nha_amd import NHACache, fused_chunk_nha_prefill
    from nha_amd.hybrid import HybridNHAConfig, Qwen3MoeNativeHybridAttention
    from nha_amd.ops import nha_hybrid_prologue
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream(dev)
    hidden, HQ, H, D, M = 2048, 32, 4, 128, 64

    def timed(fn, n=steps, busy=0.5):
        keep_busy(torch, fn, seconds=min(busy, CLOCK_WARM_S))
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record(stream)
        for _ in range(n):
            fn()
        ev[1].record(stream)
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / n

    out = {"shape": {"hidden": hidden, "HQ": HQ, "H": H, "D": D, "M": M, "prefill": "B=2 T=8192", "decode": "B=128"}}
    torch.manual_seed(0)
    for W, tag in ((64, "w64"), (2048, "w2048")):
        cfg = HybridNHAConfig(hidden_size=hidden, num_attention_heads=HQ, num_key_value_heads=H, head_dim=D, num_slots=M,
                              window_size=64, block_size=1 if W == 2048 else None, transformer_idx=0 if W == 2048 else None)
        blk = Qwen3MoeNativeHybridAttention(cfg, 0).to(torch.bfloat16).to(dev).eval()
        assert blk.window_size == W
        x = (torch.randn(2, 8192, hidden, device=dev) * 0.5).to(torch.bfloat16)
        pos = torch.arange(8192, device=dev)[None].expand(2, -1)
        res = {}
        with torch.no_grad():
            for fuse in (True, False):
                blk.fuse_glue = fuse
                ms = timed(lambda: blk(x, position_ids=pos), n=max(steps // 2, 4))
                res["block_ms" if fuse else "block_chain_ms"] = ms
            res["tokens_per_s"] = 2 * 8192 / (res["block_ms"] * 1e-3)
            # the parts of the fused block, each alone
            blk.fuse_glue = True
            nha = blk.is_nha_layer
            y = blk._fused_projection(x, nha)
            res["projection_ms"] = timed(lambda: blk._fused_projection(x, nha), n=max(steps // 2, 4))
            cos, sin = blk._tables(x, pos, None, None, 8192)
            o0, o1, o2 = HQ * D, HQ * D + H * D, HQ * D + 2 * H * D
            glue = lambda: nha_hybrid_prologue(y[..., :o0], y[..., o0:o1], y[..., o1:o2], y[..., o2:] if nha else None, cos, sin,
                                               num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=M,
                                               q_weight=blk.q_norm.weight, k_weight=blk.k_norm.weight, eps=1e-6)
            q, sq, k, sk, v, g, s_ = glue()
            res["glue_ms"] = timed(glue, n=max(steps // 2, 4))
            moved = 2 * 8192 * 2 * (3 * HQ * D + 3 * H * D + 2 * H * D + (3 if nha else 2) * H * M + 2 * D)
            res["glue_gbs"] = moved / (res["glue_ms"] * 1e-3) / 1e9
            if nha:
                op = lambda: fused_chunk_nha_prefill(q=q, k=k, v=v, rotary_q=sq, rotary_k=sk, s=s_, g=g, window_size=W,
                                                     scale=D ** -0.5)
            else:
                from nha_amd.ops import zero_sink_attention
                op = lambda: (zero_sink_attention(sq, sk, v, W, M, scale=D ** -0.5),)
            o = op()[0]
            res["attention_op_ms"] = timed(op, n=max(steps // 2, 4))
            res["o_proj_ms"] = timed(lambda: blk.o_proj(o.reshape(2, 8192, HQ * D)), n=max(steps // 2, 4))
            res["parts_sum_ms"] = res["projection_ms"] + res["glue_ms"] + res["attention_op_ms"] + res["o_proj_ms"]
        out["prefill_" + tag] = res
        # decode: B = 128 after a 256-token prompt (the NHA layer's window is full; the zero-sink layer holds 256 of 2048)
        B = 128
        xp = (torch.randn(B, 256, hidden, device=dev) * 0.5).to(torch.bfloat16)
        xs = (torch.randn(B, 1, hidden, device=dev) * 0.5).to(torch.bfloat16)
        dres = {}
        with torch.no_grad():
            for fuse in (True, False):
                blk.fuse_glue = fuse
                cache = NHACache()
                blk(xp, position_ids=torch.arange(256, device=dev)[None].expand(B, -1), past_key_value=cache, use_cache=True)
                pos1 = torch.full((B, 1), 256, device=dev)
                step = lambda: blk(xs, position_ids=pos1, past_key_value=cache, use_cache=True)
                dres["block_us" if fuse else "block_chain_us"] = timed(step, n=128, busy=0.2) * 1e3
                if fuse:
                    # the same step recorded into a HIP graph (no per-launch host work)
                    rec = blk.record_decode_step(cache, B)
                    dres["recorded_block_us"] = timed(lambda: rec.step(xs, pos1), n=128, busy=0.2) * 1e3
                    # the caller fills the graph's input buffers itself: the replay alone
                    dres["recorded_block_replay_only_us"] = timed(lambda: rec.step(rec.x, rec.pos), n=128, busy=0.2) * 1e3
                    del rec
            # the bare kernel step on the same cache, and the glue and GEMMs of a step alone
            from nha_amd import ring_decode_step
            blk.fuse_glue = True
            st = cache.states[0]
            y1 = blk._fused_projection(xs, nha)
            cos1, sin1 = blk._tables(xs, pos1, None, None, 1)
            glue1 = lambda: nha_hybrid_prologue(y1[..., :o0], y1[..., o0:o1], y1[..., o1:o2], y1[..., o2:] if nha else None, cos1,
                                                sin1, num_heads=HQ, num_kv_heads=H, head_dim=D, num_slots=M,
                                                q_weight=blk.q_norm.weight, k_weight=blk.k_norm.weight, eps=1e-6, want_s=False)
            q1, sq1, k1, sk1, v1, g1, _ = glue1()
            dres["ring_decode_step_us"] = timed(lambda: ring_decode_step(st, q1[:, 0], sq1[:, 0], sk1[:, 0], k1[:, 0], v1[:, 0],
                                                                         g1[:, 0], scale=D ** -0.5), n=128, busy=0.2) * 1e3
            dres["glue_us"] = timed(glue1, n=128, busy=0.2) * 1e3
            dres["projection_us"] = timed(lambda: blk._fused_projection(xs, nha), n=128, busy=0.2) * 1e3
            o1_ = torch.empty(B, 1, HQ * D, dtype=torch.bfloat16, device=dev)
            dres["o_proj_us"] = timed(lambda: blk.o_proj(o1_), n=128, busy=0.2) * 1e3
            dres["parts_sum_us"] = dres["ring_decode_step_us"] + dres["glue_us"] + dres["projection_us"] + dres["o_proj_us"]
            dres["block_over_bare_step"] = dres["block_us"] / dres["ring_decode_step_us"]
            dres["recorded_block_over_bare_step"] = dres["recorded_block_us"] / dres["ring_decode_step_us"]
        out["decode_" + tag] = dres
        del blk, cache
    return out


# the decode step at the 340M layers' heads (one query head per kv-head, head size 256, window 512)
DECODE_D256 = dict(B=128, HQ=4, H=4, D=256, M=64, W=512, steps=128)


def bench_decode(torch, warmup, cfg=DECODE):
    from nha_amd import NHARingState, ring_decode_step
    dev = torch.device("cuda:0")
    B, HQ, H, D, M, W, steps = (cfg[k] for k in ("B", "HQ", "H", "D", "M", "W", "steps"))
    gen = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    st = NHARingState.empty(B, H, D, D, M, W, dtype=torch.bfloat16, device=dev)
    st.hk.copy_(r(B, H, D, M) * 0.1)
    st.hv.copy_(r(B, H, M, D) * 0.1)
    st.ring_k.copy_(r(B, W, H, D))
    st.ring_kg.copy_(r(B, W, H, D))
    st.ring_v.copy_(r(B, W, H, D))
    st.ring_g.copy_(torch.nn.functional.logsigmoid(r(B, W, H, M)))
    # full windows at random ring positions
    st.count.copy_(torch.randint(W, 3 * W, (B,), generator=gen, dtype=torch.int32))
    pool = 8
    q = [(r(B, HQ, D) * D ** -0.5).to(torch.bfloat16).to(dev) for _ in range(pool)]
    sq = [(r(B, HQ, D) * D ** -0.5).to(torch.bfloat16).to(dev) for _ in range(pool)]
    kn = [r(B, H, D).to(torch.bfloat16).to(dev) for _ in range(pool)]
    kgn = [r(B, H, D).to(torch.bfloat16).to(dev) for _ in range(pool)]
    vn = [r(B, H, D).to(torch.bfloat16).to(dev) for _ in range(pool)]
    gn = [torch.nn.functional.logsigmoid(r(B, H, M)).to(torch.bfloat16).to(dev) for _ in range(pool)]
    o = torch.empty(B, HQ, D, dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream(dev)

    def loop(n, advance):
        for i in range(n):
            j = i % pool
            ring_decode_step(st, q[j], sq[j], kn[j], kgn[j], vn[j], gn[j], out=o, advance=advance)

    keep_busy(torch, lambda: loop(pool, False), batch=4)
    loop(warmup, True)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    loop(steps, True)
    e1.record(stream)
    torch.cuda.synchronize()
    us_step = e0.elapsed_time(e1) * 1e3 / steps
    # decode kernel alone, counters left where they are
    e0.record(stream)
    loop(steps, False)
    e1.record(stream)
    torch.cuda.synchronize()
    us_kernel = e0.elapsed_time(e1) * 1e3 / steps
    nbytes = decode_bytes(B, HQ, H, D, M, W)
    return dict(us_per_step=us_step, us_kernel=us_kernel, bytes=nbytes, achieved_gbs=nbytes / (us_kernel * 1e-6) / 1e9)


def bench_api(torch, steps, warmup):
    """The drop-in Python ops, called the way the reference's callers call them (outputs allocated per
    call, tables and workspace found in the ops' caches): milliseconds / microseconds per call with HIP
    events on the launch stream.  chunk_nha at the headline shape and on the packed varlen
    configuration (cu_seqlens tensor on the GPU, initial and final states); fused_recurrent_nha_decode
    in its window form (time-ordered [B,W,H,D] window tensors, explicit popped entry) at the decode
    configuration, once with a pre-rotated query and once with in-kernel rotary (cos / sin)."""
    import itertools
    from nha_amd import chunk_nha, fused_recurrent_nha_decode
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream(dev)

    def timed(fn, n):
        keep_busy(torch, fn)
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record(stream)
        for _ in range(n):
            fn()
        ev[1].record(stream)
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / n

    out = {}
    with torch.no_grad():
        cfg = PREFILL
        xs = make_prefill_inputs(torch, cfg, dev)
        W = cfg["W"]
        # the C-ABI call with pre-allocated outputs, timed right next to the op (the clock a box grants
        # moves by several per cent over a run; the ratio is taken between neighbours)
        out["abi_ms_adjacent"] = bench_prefill(torch, steps, warmup)["ms_per_step"]
        out["chunk_nha_ms"] = timed(lambda: chunk_nha(*xs, window_size_left=W - 1, gsa_kv_shift=W), steps)
        del xs
        cfg = WORKLOADS["cfg3"]
        lens = workload_lengths(torch, cfg)
        xs = make_prefill_inputs(torch, cfg, dev)
        cu = torch.tensor([0] + list(itertools.accumulate(lens)), dtype=torch.int32, device=dev)
        h0 = make_initial_state(torch, cfg, len(lens), dev)
        out["chunk_nha_varlen_cfg3_ms"] = timed(lambda: chunk_nha(*xs, cu_seqlens=cu, window_size_left=cfg["wl"],
                                                                  gsa_kv_shift=cfg["shift"], initial_state=h0,
                                                                  output_final_state=True), steps)
        del xs
        d = DECODE
        B, HQ, H, D, M, Wd = (d[k] for k in ("B", "HQ", "H", "D", "M", "W"))
        gen = torch.Generator().manual_seed(3)
        r = lambda *sh: torch.randn(*sh, generator=gen, dtype=torch.float32)
        bf = lambda x: x.to(torch.bfloat16).to(dev)
        q, sq = bf(r(B, 1, HQ, D) * D ** -0.5), bf(r(B, 1, HQ, D) * D ** -0.5)
        k, v = bf(r(B, 1, H, D)), bf(r(B, 1, H, D))
        g = bf(torch.nn.functional.logsigmoid(r(B, 1, H, M)))
        swk, swv = bf(r(B, Wd, H, D)), bf(r(B, Wd, H, D))
        hk, hv = (r(B, H, D, M) * 0.1).to(dev), (r(B, H, M, D) * 0.1).to(dev)
        pos = torch.arange(Wd, dtype=torch.float32)
        inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
        ang = torch.cat([pos[:, None] * inv[None], pos[:, None] * inv[None]], -1)[None]
        cos, sin = bf(ang.cos()), bf(ang.sin())
        n = d["steps"]
        out["decode_window_eager_us"] = 1e3 * timed(lambda: fused_recurrent_nha_decode(
            q, k, v, g, swk, swv, sq=sq, initial_state=(hk, hv), output_final_state=True), n)
        out["decode_window_rotary_us"] = 1e3 * timed(lambda: fused_recurrent_nha_decode(
            q, k, v, g, swk, swv, cos=cos, sin=sin, initial_state=(hk, hv), output_final_state=True), n)
        # tables with rows of their own per sequence ([B,W,D], what a model's position embeddings are)
        cos_b, sin_b = cos.expand(B, Wd, D).contiguous(), sin.expand(B, Wd, D).contiguous()
        out["decode_window_rotary_per_sequence_us"] = 1e3 * timed(lambda: fused_recurrent_nha_decode(
            q, k, v, g, swk, swv, cos=cos_b, sin=sin_b, initial_state=(hk, hv), output_final_state=True), n)
        del cos_b, sin_b
        # the call forms that the generic (vector-unit) decode kernels serve: caller-supplied window logits
        # (fused_recurrent_nha, the dense hybrids' step) and float32 tensors
        from nha_amd import fused_recurrent_nha
        logits = (r(B, 1, HQ, Wd)).to(torch.bfloat16).to(dev)
        s_ = (1 - g.float().exp()).to(torch.bfloat16)
        out["fused_recurrent_nha_logits_us"] = 1e3 * timed(lambda: fused_recurrent_nha(
            q, k, v, logits, s_, g, initial_state=(hk, hv), output_final_state=True), n)
        f32 = lambda x: x.float()
        q32, sq32, k32, v32, g32, swk32, swv32 = map(f32, (q, sq, k, v, g, swk, swv))
        out["decode_window_fp32_us"] = 1e3 * timed(lambda: fused_recurrent_nha_decode(
            q32, k32, v32, g32, swk32, swv32, sq=sq32, initial_state=(hk, hv), output_final_state=True), max(n // 4, 8))
    return out


def decode_call_forms(api):
    """The other call forms of the single-token ops at the decode workload's shape (Python ops, outputs allocated per
    call), each with the bytes its tensors hold and the share of the HBM peak that makes: window rows as a [B,W,H,D]
    tensor with a pre-rotated query, the same with cos / sin tables (shared [1,W,D] tables: their bytes are not
    counted; [B,W,D] tables with rows of their own per sequence: counted), float32 tensors, and caller-supplied window
    logits (no window rows at all)."""
    d = DECODE
    B, HQ, H, D, M, W = (d[k] for k in ("B", "HQ", "H", "D", "M", "W"))
    state = 2 * 2 * B * H * D * M * 4                      # hk and hv, read and written
    rows = lambda esz: (2 * B * W * H * D + 2 * B * HQ * D + 2 * B * H * D + B * H * M + B * HQ * D) * esz + state
    forms = {"window_prerotated": ("decode_window_eager_us", rows(2)), "window_cos_sin_tables": ("decode_window_rotary_us", rows(2)),
             "window_cos_sin_tables_per_sequence": ("decode_window_rotary_per_sequence_us", rows(2) + 2 * B * W * D * 2),
             "window_float32": ("decode_window_fp32_us", rows(4)),
             "caller_logits": ("fused_recurrent_nha_logits_us", state + B * HQ * W * (2 + 4) + (B * HQ * D * 2 + 2 * B * H * D + 2 * B * H * M) * 2)}
    out = {}
    for name, (key, nbytes) in forms.items():
        us = api[key]
        out[name] = {"us_per_step": us, "algorithmic_bytes": nbytes, "hbm_frac": nbytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBS}
    return out


def cpu_baseline(torch):
    """The oracle on the host cores, bounded sample: the plain-C restatement (oracle/nha_ref_c.c,
    OpenMP over sequences x q-heads, double arithmetic) for the prefill, the torch restatement for a
    few decode steps."""
    from oracle import nha_ref as R
    from oracle.nha_ref_c import prefill_ref_c
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    cfg = PREFILL
    W = cfg["W"]

    def timed(T, B=1):
        xs = make_prefill_inputs(torch, cfg, "cpu", B=B, T=T)
        t0 = time.perf_counter()
        prefill_ref_c(*xs, window_size_left=W - 1, gsa_kv_shift=W)
        return time.perf_counter() - t0

    t_probe = timed(512)
    # cost per token grows with the window fill; aim at 10-20 s of CPU work, at most the full T
    T = 512
    est = t_probe
    while T < cfg["T"]:
        grow = 4.0 if 2 * T <= W else 2.2
        if est * grow > 20.0:
            break
        T *= 2
        est *= grow
    Bs = cfg["B"] if (T == cfg["T"] and est * cfg["B"] <= 30.0) else 1   # the whole workload when it fits
    t = timed(T, Bs)
    what = "the whole workload" if Bs == cfg["B"] else f"B=1 slice, first {T} tokens of the T={cfg['T']} workload"
    pre = dict(value=Bs * T / t, unit="tokens/s", cores=cores, kind="port",
               sample=f"{what}, C restatement of the oracle (OpenMP, double arithmetic), {t:.1f} s")
    d = DECODE
    B, HQ, H, D, M, Wd = (d[k] for k in ("B", "HQ", "H", "D", "M", "W"))
    gen = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    args = dict(q=r(B, 1, HQ, D), k=r(B, 1, H, D), v=r(B, 1, H, D), g=torch.nn.functional.logsigmoid(r(B, 1, H, M)),
                sw_k=r(B, Wd, H, D), sw_v=r(B, Wd, H, D))
    h0 = (r(B, H, D, M) * 0.1, r(B, H, M, D) * 0.1)
    R.decode_ref(**args, sq=args["q"], initial_state=h0, dtype=torch.float32)
    t0 = time.perf_counter()
    nrep = 3
    for _ in range(nrep):
        R.decode_ref(**args, sq=args["q"], initial_state=h0, dtype=torch.float32)
    pre["decode_us_per_step"] = (time.perf_counter() - t0) / nrep * 1e6
    pre["decode_sample"] = f"{nrep} steps of the B={B} decode workload, fp32"
    pre["torch_naive"] = cpu_baseline_torch_naive(torch, cores, (args, h0))
    return pre


def cpu_baseline_torch_naive(torch, cores, decode_inputs):
    """The naive PyTorch per-token path (oracle.prefill_ref / oracle.decode_ref: the shape of computation of
    the reference's scripts/verify_opt_parity.py:88-191), fp32, all host cores: one warm-up, then the
    median of three runs, on a B=1 slice of the prefill workload sized to a few seconds per run."""
    import statistics
    from oracle import nha_ref as R
    cfg = PREFILL
    W = cfg["W"]
    keys = ("q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g")

    def run(T):
        xs = make_prefill_inputs(torch, cfg, "cpu", B=1, T=T)
        t0 = time.perf_counter()
        R.prefill_ref(*xs, window_size_left=W - 1, gsa_kv_shift=W, dtype=torch.float32)
        return time.perf_counter() - t0

    T = 256
    t = run(T)                                       # warm-up and probe
    while T < cfg["T"] and t * 2.5 <= 8.0:           # per-token cost grows until the window is full
        T *= 2
        t *= 2.5
    ts = sorted(run(T) for _ in range(3))
    a, h0 = decode_inputs
    R.decode_ref(**a, sq=a["q"], initial_state=h0, dtype=torch.float32)
    td = []
    for _ in range(3):
        t0 = time.perf_counter()
        R.decode_ref(**a, sq=a["q"], initial_state=h0, dtype=torch.float32)
        td.append(time.perf_counter() - t0)
    return dict(value=T / ts[1], unit="tokens/s", cores=cores, kind="port",
                sample=f"B=1 slice, first {T} tokens of the T={cfg['T']} workload, fp32 torch per-token loop, "
                       f"1 warm-up + median of 3 ({ts[1]:.1f} s)",
                decode_us_per_step=statistics.median(td) * 1e6,
                decode_sample=f"median of 3 steps after a warm-up, B={DECODE['B']} decode workload, fp32 torch")


def main():
    global CLOCK_WARM_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--clock-warmup", type=float, default=CLOCK_WARM_S,
                    help="seconds of untimed back-to-back launches before each timed region (the shader clock of an "
                         "idle GPU needs about a second of load to reach its sustained level); 0 = off")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one 256 MiB device-to-device copy (reference point for rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--only", choices=["prefill", "decode", "decode_d256", "glue", "layer", "hybrid"], default=None,
                    help="development aid: time one leg only and print its raw numbers")
    ap.add_argument("--backward", action="store_true",
                    help="with --workload: also time the backward of the prefill op")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default=None,
                    help="time the prefill of another of the reference's configurations and print its raw numbers")
    args = ap.parse_args()
    CLOCK_WARM_S = max(args.clock_warmup, 0.0)
    if args.gpus != 1:
        print("bench.py measures one GPU: this path shards by sequence / kv-head with no communication and "
              "no multi-GPU figure is produced (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the NHA ops have no CPU fallback)", file=sys.stderr)
        sys.exit(3)
    if args.copy_calibration:
        a = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0")
        b = torch.empty_like(a)
        b.copy_(a)
        torch.cuda.synchronize()
    if args.workload:
        cfg = WORKLOADS[args.workload]
        res = bench_prefill(torch, args.steps, args.warmup, cfg)
        res["workload"] = {k: v for k, v in cfg.items()}
        res["min_bytes"] = min_prefill_bytes(cfg, len(workload_lengths(torch, cfg)))
        res["min_bytes_gbs"] = res["min_bytes"] / (res["ms_per_step"] * 1e-3) / 1e9
        if args.backward:
            res.update(bench_backward(torch, args.steps, args.warmup, cfg))
        print(json.dumps(res))
        return
    if args.only:
        res = (bench_prefill(torch, args.steps, args.warmup) if args.only == "prefill" else
               bench_glue(torch, args.steps, args.warmup) if args.only == "glue" else
               bench_layer(torch, args.steps, args.warmup) if args.only == "layer" else
               bench_hybrid(torch, args.steps, args.warmup) if args.only == "hybrid" else
               bench_decode(torch, args.warmup, DECODE_D256) if args.only == "decode_d256" else bench_decode(torch, args.warmup))
        print(json.dumps(res))
        return
    pf_cold = bench_prefill(torch, args.steps, args.warmup, cold=True)
    pf = bench_prefill(torch, args.steps, args.warmup)
    bw = bench_backward(torch, max(args.steps // 2, 1), min(args.warmup, 2))
    dc = bench_decode(torch, args.warmup)
    dc256 = bench_decode(torch, args.warmup, DECODE_D256)
    gl = bench_glue(torch, args.steps, args.warmup)
    api = bench_api(torch, max(args.steps // 2, 1), min(args.warmup, 2))
    hyb = bench_hybrid(torch, max(args.steps // 2, 1), min(args.warmup, 2))
    others = {}
    for name in ("cfg2", "cfg3", "cfg5", "w64"):
        cfg = WORKLOADS[name]
        r = bench_prefill(torch, max(args.steps // 2, 1), min(args.warmup, 2), cfg)
        mb = min_prefill_bytes(cfg, len(workload_lengths(torch, cfg)))
        others[name] = {"ms": r["ms_per_step"], "state_pass_ms": r["t_state_ms"], "output_pass_ms": r["t_out_ms"],
                        "tokens_per_s": r["tokens_per_s"], "tflops": r["whole_op_tflops"],
                        "mfma_frac": r["whole_op_tflops"] / PEAK_MFMA_BF16_TFLOPS, "min_bytes": mb,
                        "min_bytes_gbs": mb / (r["ms_per_step"] * 1e-3) / 1e9,
                        "shape": {k: v for k, v in cfg.items()}}
    cpu = None if args.no_cpu_baseline else cpu_baseline(torch)
    out = {
        "metric": "NHA prefill tokens/s @T=8K bf16",
        "value": pf["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_warmup_s": CLOCK_WARM_S,
        "ms_per_step": pf["ms_per_step"],
        "cold_ms_per_step": pf_cold["ms_per_step"],
        "cold_note": "the same warm-up and timed steps without the clock warm-up, after one second of idling: measured "
                     "on the shader clock's ramp from its parked level",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "one NHA layer prefill, B=2 T=8192 HQ=32 H=8 D=128 M=64 W=2048 "
                               "(window W keys, slots hold tokens <= t-W), gate logits N(-1,1)->logsigmoid",
                   "decode_workload": "B=128 HQ=32 H=8 D=128 M=64 W=1024 ring buffer, full windows at random "
                                      "ring positions, 256 consecutive steps"},
        "roofline": {"bound": "mfma", "kernel": OUT_KERNEL, "achieved": pf["achieved_tflops"],
                     "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": pf["achieved_tflops"] / PEAK_MFMA_BF16_TFLOPS,
                     "traffic": TRAFFIC_BYTES[OUT_KERNEL], "traffic_source": TRAFFIC_SOURCE[OUT_KERNEL],
                     "kernel_ms": pf["t_out_ms"], "state_pass_ms": pf["t_state_ms"],
                     "whole_op_tflops": pf["whole_op_tflops"], "algorithmic_flop": pf["flops"]},
        "decode": {"metric": "decode step us @B=128", "value": dc["us_per_step"], "unit": "us/step",
                   "higher_is_better": False,
                   "roofline": {"bound": "hbm", "kernel": "decode_mfma_kernel<128,4,2>", "achieved": dc["achieved_gbs"],
                                "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": dc["achieved_gbs"] / PEAK_HBM_GBS,
                                "traffic": TRAFFIC_BYTES["decode_mfma_kernel<128,4,2>"],
                                "traffic_source": TRAFFIC_SOURCE["decode_mfma_kernel<128,4,2>"],
                                "kernel_us": dc["us_kernel"], "algorithmic_bytes": dc["bytes"]},
                   "other_shapes": {"d256": {"shape": {k: v for k, v in DECODE_D256.items() if k != "steps"},
                                             "us_per_step": dc256["us_per_step"], "kernel_us": dc256["us_kernel"],
                                             "kernel": "decode_mfma_kernel<256,1,4>", "algorithmic_bytes": dc256["bytes"],
                                             "achieved_gbs": dc256["achieved_gbs"],
                                             "hbm_frac": dc256["achieved_gbs"] / PEAK_HBM_GBS},
                                    "call_forms": decode_call_forms(api)}},
        "backward": {"metric": "backward of the same prefill call", "ms_per_call": bw["bwd_ms"], "unit": "ms",
                     "tokens_per_s": bw["bwd_tokens_per_s"], "tflops": bw["bwd_tflops"],
                     "flop": bw["bwd_flops"], "note": "2.5 x the forward's algorithmic flop"},
        "layer_glue": {"metric": "fused layer prologue / epilogue at the prefill shape", "unit": "us/launch",
                       "prologue_us": gl["prologue_us"], "epilogue_us": gl["epilogue_us"],
                       "roofline": {"bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                    "prologue": {"achieved": gl["prologue_gbs"], "frac": gl["prologue_gbs"] / PEAK_HBM_GBS,
                                                 "algorithmic_bytes": gl["prologue_bytes"],
                                                 "traffic": TRAFFIC_BYTES["layer_prologue_kernel"]},
                                    "epilogue": {"achieved": gl["epilogue_gbs"], "frac": gl["epilogue_gbs"] / PEAK_HBM_GBS,
                                                 "algorithmic_bytes": gl["epilogue_bytes"],
                                                 "traffic": TRAFFIC_BYTES["layer_epilogue_kernel"]}}},
        "api": {"note": "the drop-in Python ops as their callers use them (outputs allocated per call); the headline "
                        "value above times the C-ABI call with pre-allocated outputs",
                "chunk_nha_ms": api["chunk_nha_ms"], "abi_ms_adjacent": api["abi_ms_adjacent"],
                "chunk_nha_vs_abi": api["chunk_nha_ms"] / api["abi_ms_adjacent"],
                "chunk_nha_varlen_cfg3_ms": api["chunk_nha_varlen_cfg3_ms"],
                "fused_recurrent_nha_decode_window_eager_us": api["decode_window_eager_us"],
                "fused_recurrent_nha_decode_window_rotary_us": api["decode_window_rotary_us"],
                "fused_recurrent_nha_logits_mode_us": api["fused_recurrent_nha_logits_us"],
                "fused_recurrent_nha_decode_window_fp32_us": api["decode_window_fp32_us"]},
        "hybrid": hyb,
        "workloads": others,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
