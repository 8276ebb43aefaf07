"""CPU oracle for the NHA fused hybrid-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``nha_amd``) imports
this module; it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / CPU timing reference.

It restates, as plain PyTorch on CPU, the semantics of the reference op
(citations are relative to the reference checkout):

* slot write  (scripts/verify_opt_parity.py:76-85, nha_fla/ops/nha/fused_recurrent.py:88,142)
* slot read + window + ONE softmax over [M slots | window]
  (scripts/verify_opt_parity.py:147-191, nha_fla/ops/nha/fused_recurrent.py:342-349)
* the (window_size_left, gsa_kv_shift) generalisation of nha_fla/ops/nha/chunk.py:53-78,
  :401-470 (shift of the slot branch, causal left window of the SWA branch, LSE merge)
* single-token decode incl. rotate-half RoPE (scripts/verify_opt_parity.py:88-125,
  nha_fla/ops/nha/fused_recurrent.py:309-329)
* caller-supplied-window-logit step (scripts/verify_opt_parity.py:128-144)

A second, independent restatement of the prefill in plain C lives in nha_ref_c.c
(front: nha_ref_c.py); it is pinned against this module.

Pinning (see tests/test_oracle_pins.py): every function below is checked against
something that is *not* a retyping of its own formula -- torch's
scaled_dot_product_attention (slots degenerate to zero sinks), the explicit
double-sum closed form of the gated recurrence, the two-branch LSE merge of
chunk.py:459-470, an independent chunk-form evaluation, complex-number RoPE,
decode == last row of prefill, packed == per-sequence; the layer glue against
torch's sigmoid / rms_norm library routines, RoPE's norm and relative-position
invariants and s + exp(g) = 1.  What nothing in this
container pins: the exact bf16 rounding sequence of the Triton/fla chain and
flash-attn's window inclusivity for ``window_size_left`` (third-party documented
semantics: key j visible to query i iff i - wl <= j <= i).
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

__all__ = [
    "layer_prologue_ref",
    "layer_epilogue_ref",
    "rope_rotate_half",
    "gsa_step",
    "prefill_ref",
    "prefill_chunked_ref",
    "prefill_grad_ref",
    "decode_ref",
    "decode_ring_ref",
    "fused_recurrent_ref",
]


def rope_rotate_half(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """HF rotate-half RoPE on ``x [..., T, H, K]`` with duplicated-halves tables
    ``cos/sin [..., T, K]`` (scripts/verify_opt_parity.py:49-54)."""
    half = x.shape[-1] // 2
    rot = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos.unsqueeze(-2) + rot * sin.unsqueeze(-2)


def layer_prologue_ref(q, k, v, f, *, feature_map, gate_logit_normalizer, positions, rope_theta=10000.0):
    """The elementwise chain of nha_fla/layers/nha.py:214-237 in the dtype of the inputs (pass
    float64 for the checker): q [B,T,HQ,K], k [B,T,H,K], v [B,T,H,V], f [B,T,H,M],
    positions [B,T] or [T] (token index inside its sequence + seqlen_offset).
    Returns (q_swa, k_swa, q_gsa, k_gsa, v, s, g).  The rotary angle is formed in float32
    (position * inv_freq, as the rotary module's cos/sin cache is) and then widened."""
    K = q.shape[-1]
    fmap = {"swish": torch.nn.functional.silu, "relu": torch.relu, None: (lambda x: x)}[feature_map]
    inv = 1.0 / (rope_theta ** (torch.arange(0, K, 2, dtype=torch.float32) / K))
    ang = (positions.to(torch.float32)[..., None] * inv).to(q.dtype)          # [..., T, K/2]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    g = torch.nn.functional.logsigmoid(f) / gate_logit_normalizer
    return (rope_rotate_half(q, cos, sin), rope_rotate_half(k, cos, sin), fmap(q), fmap(k),
            torch.nn.functional.silu(v), 1 - g.exp(), g)


def layer_epilogue_ref(o, weight, bias, eps):
    """rms_norm(silu(o)) * weight (+ bias) over the last dim: the normalisation half of
    rms_norm_linear(F.silu(o), ...) at nha_fla/layers/nha.py:278."""
    y = torch.nn.functional.silu(o)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight
    if bias is not None:
        y = y + bias
    return y


def gsa_step(hk, hv, k, v, s, g):
    """One slot write.  hk [...,H,K,M], hv [...,H,M,V]; k [...,H,K], v [...,H,V],
    s,g [...,H,M] (scripts/verify_opt_parity.py:81-83)."""
    eg = g.exp()
    hk = hk * eg[..., None, :] + k[..., :, None] * s[..., None, :]
    hv = hv * eg[..., :, None] + s[..., :, None] * v[..., None, :]
    return hk, hv


def _expand(x: torch.Tensor, ng: int, dim: int) -> torch.Tensor:
    # q-head hq reads kv-head hq // ng (group-major, scripts/verify_opt_parity.py:43-46)
    return x if ng == 1 else x.repeat_interleave(ng, dim=dim)


def _prefill_equal_len(q_swa, k_swa, q_gsa, k_gsa, v, s, g, wl, shift, scale, hk, hv):
    """Per-token recurrence for a batch of equal-length sequences.
    q_* [B,T,HQ,K]; k_*, v, s, g [B,T,H,*]; hk [B,H,K,M]; hv [B,H,M,V] (working dtype)."""
    B, T, HQ, K = q_swa.shape
    H = k_swa.shape[2]
    M = s.shape[-1]
    V = v.shape[-1]
    NG = HQ // H
    o = q_swa.new_zeros(B, T, HQ, V)
    lse_swa = q_swa.new_zeros(B, T, HQ)
    lse_gsa = q_swa.new_zeros(B, T, HQ)
    for t in range(T):
        j = t - shift
        if j >= 0:
            hk, hv = gsa_step(hk, hv, k_gsa[:, j], v[:, j], s[:, j], g[:, j])
        ok = torch.einsum("bqk,bqkm->bqm", q_gsa[:, t] * scale, _expand(hk, NG, 1))
        lo = 0 if wl < 0 else max(0, t - wl)
        kw = _expand(k_swa[:, lo:t + 1], NG, 2)                       # [B,w,HQ,K]
        vw = _expand(v[:, lo:t + 1], NG, 2)
        sw = torch.einsum("bqk,bwqk->bqw", q_swa[:, t] * scale, kw)
        p = torch.softmax(torch.cat([ok, sw], dim=-1), dim=-1)
        o[:, t] = torch.einsum("bqm,bqmv->bqv", p[..., :M], _expand(hv, NG, 1)) \
            + torch.einsum("bqw,bwqv->bqv", p[..., M:], vw)
        lse_gsa[:, t] = torch.logsumexp(ok, dim=-1)
        lse_swa[:, t] = torch.logsumexp(sw, dim=-1)
    return o, lse_swa, lse_gsa, hk, hv


def prefill_ref(
    q_swa: torch.Tensor,
    k_swa: torch.Tensor,
    q_gsa: torch.Tensor,
    k_gsa: torch.Tensor,
    v: torch.Tensor,
    s: torch.Tensor,
    g: torch.Tensor,
    *,
    window_size_left: int,
    gsa_kv_shift: int = 0,
    cu_seqlens: Optional[Sequence[int]] = None,
    initial_state: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    scale: Optional[float] = None,
    dtype: torch.dtype = torch.float64,
):
    """Naive NHA prefill: per-token slot recurrence + clamped causal window, one softmax.

    Token t of a sequence sees window keys ``[max(0, t - wl), t]`` (all of
    ``[0, t]`` when ``wl < 0``) and slots that have absorbed tokens ``<= t - shift``.
    ``(wl, shift) = (W-1, W)`` is scripts/verify_opt_parity.py:147-191 exactly;
    ``(W, 0)`` is the layer's call (nha_fla/layers/nha.py:238-253).

    Shapes: q_* ``[B,T,HQ,K]``; k_*, v, s, g ``[B,T,H,*]`` with ``HQ % H == 0``.
    Varlen: ``B == 1`` and ``cu_seqlens`` of length N+1; states are ``[N,H,K,M]/[N,H,M,V]``.
    Returns ``(o [B,T,HQ,V], lse_swa [B,T,HQ], lse_gsa [B,T,HQ], hkt, hvt)`` in ``dtype``.
    """
    B, T, HQ, K = q_swa.shape
    H = k_swa.shape[2]
    M = s.shape[-1]
    V = v.shape[-1]
    assert HQ % H == 0
    if scale is None:
        scale = K ** -0.5                                    # nha_fla/ops/nha/chunk.py:648-649
    cast = lambda x: x.detach().to("cpu", dtype)
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = map(cast, (q_swa, k_swa, q_gsa, k_gsa, v, s, g))
    if cu_seqlens is None:
        N = B
        if initial_state is not None:
            hk, hv = cast(initial_state[0]).clone(), cast(initial_state[1]).clone()
        else:
            hk = torch.zeros(N, H, K, M, dtype=dtype)
            hv = torch.zeros(N, H, M, V, dtype=dtype)
        return _prefill_equal_len(q_swa, k_swa, q_gsa, k_gsa, v, s, g,
                                  window_size_left, gsa_kv_shift, scale, hk, hv)
    assert B == 1, "varlen packing requires B == 1"
    cu = [int(c) for c in cu_seqlens]
    N = len(cu) - 1
    o = torch.zeros(1, T, HQ, V, dtype=dtype)
    lse_swa = torch.zeros(1, T, HQ, dtype=dtype)
    lse_gsa = torch.zeros(1, T, HQ, dtype=dtype)
    hkt = torch.zeros(N, H, K, M, dtype=dtype)
    hvt = torch.zeros(N, H, M, V, dtype=dtype)
    for n in range(N):
        st, en = cu[n], cu[n + 1]
        if initial_state is not None:
            hk, hv = cast(initial_state[0][n:n + 1]).clone(), cast(initial_state[1][n:n + 1]).clone()
        else:
            hk = torch.zeros(1, H, K, M, dtype=dtype)
            hv = torch.zeros(1, H, M, V, dtype=dtype)
        sl = slice(st, en)
        oo, ls, lg, hk, hv = _prefill_equal_len(
            q_swa[:, sl], k_swa[:, sl], q_gsa[:, sl], k_gsa[:, sl], v[:, sl], s[:, sl], g[:, sl],
            window_size_left, gsa_kv_shift, scale, hk, hv)
        o[:, sl], lse_swa[:, sl], lse_gsa[:, sl] = oo, ls, lg
        hkt[n], hvt[n] = hk[0], hv[0]
    return o, lse_swa, lse_gsa, hkt, hvt


def prefill_chunked_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, *, window_size_left, gsa_kv_shift=0,
                        initial_state=None, scale=None, chunk_size=64, dtype=torch.float64):
    """Chunk-form evaluation of the same op for ONE batch of equal-length sequences.

    Follows the chunk algebra of nha_fla/ops/nha/chunk_fused.py:96-107 (state pass: chunk-local
    inclusive gate cumsum ``gc``, ``h <- h*exp(gc_last) + K^T (S*exp(gc_last-gc))``) and
    :186-222, :242-275 (slot logits / slot read with the decay ``exp(gc_i - gc_j)``, j <= i
    INCLUDED), with the branch-wise LSE merge of nha_fla/ops/nha/chunk.py:459-470.  Used to pin
    "chunked == recurrent" and as the executable statement of what the HIP kernels compute."""
    B, T, HQ, K = q_swa.shape
    H = k_swa.shape[2]
    M = s.shape[-1]
    V = v.shape[-1]
    NG = HQ // H
    BT = chunk_size
    if scale is None:
        scale = K ** -0.5
    cast = lambda x: x.detach().to("cpu", dtype)
    q_swa, k_swa, q_gsa, k_gsa, v, s, g = map(cast, (q_swa, k_swa, q_gsa, k_gsa, v, s, g))
    wl, shift = window_size_left, gsa_kv_shift

    def shifted(x):                                          # nha_fla/ops/nha/chunk.py:100-111
        y = torch.zeros_like(x)
        if shift <= 0:
            return x
        if T > shift:
            y[:, shift:] = x[:, :T - shift]
        return y

    kg, vg, sg_, gg = shifted(k_gsa), shifted(v), shifted(s), shifted(g)
    if initial_state is not None:
        hk, hv = cast(initial_state[0]).clone(), cast(initial_state[1]).clone()
    else:
        hk = torch.zeros(B, H, K, M, dtype=dtype)
        hv = torch.zeros(B, H, M, V, dtype=dtype)
    o = torch.zeros(B, T, HQ, V, dtype=dtype)
    lse_swa = torch.zeros(B, T, HQ, dtype=dtype)
    lse_gsa = torch.zeros(B, T, HQ, dtype=dtype)
    ex = lambda x: _expand(x, NG, 2)
    exd = lambda x: _expand(x, NG, 3)
    for c0 in range(0, T, BT):
        c1 = min(c0 + BT, T)
        n = c1 - c0
        gc = gg[:, c0:c1].cumsum(1)                          # [B,n,H,M]
        tri = torch.tril(torch.ones(n, n, dtype=dtype))      # j <= i
        # decay[b,i,j,h,m] = exp(gc_i - gc_j) for j <= i (non-positive exponent)
        dec = torch.exp((gc[:, :, None] - gc[:, None, :]).clamp(max=0.0)) * tri[None, :, :, None, None]
        qg = q_gsa[:, c0:c1] * scale
        A = torch.einsum("bihk,bjhk->bijh", qg, ex(kg[:, c0:c1]))
        ok = torch.einsum("bihk,bhkm->bihm", qg, _expand(hk, NG, 1)) * ex(gc).exp() \
            + torch.einsum("bijh,bijhm,bjhm->bihm", A, exd(dec), ex(sg_[:, c0:c1]))
        lg = torch.logsumexp(ok, -1)
        p = torch.softmax(ok, -1)
        Av = torch.einsum("bihm,bijhm,bjhm->bijh", p, exd(dec), ex(sg_[:, c0:c1]))
        o_gsa = torch.einsum("bihm,bhmv->bihv", p * ex(gc).exp(), _expand(hv, NG, 1)) \
            + torch.einsum("bijh,bjhv->bihv", Av, ex(vg[:, c0:c1]))
        # sliding-window branch for the rows of this chunk
        lo_all = 0 if wl < 0 else max(0, c0 - wl)
        kw, vw = ex(k_swa[:, lo_all:c1]), ex(v[:, lo_all:c1])
        sw = torch.einsum("bihk,bjhk->bihj", q_swa[:, c0:c1] * scale, kw)
        ii = torch.arange(c0, c1)[:, None]
        jj = torch.arange(lo_all, c1)[None, :]
        valid = (jj <= ii) & ((jj >= ii - wl) if wl >= 0 else torch.ones_like(jj <= ii))
        sw = sw.masked_fill(~valid[None, :, None, :], float("-inf"))
        ls = torch.logsumexp(sw, -1)
        o_swa = torch.einsum("bihj,bjhv->bihv", torch.softmax(sw, -1), vw)
        # two-branch merge, nha_fla/ops/nha/chunk.py:459-470
        mx = torch.maximum(ls, lg)
        w_s, w_g = torch.exp(ls - mx), torch.exp(lg - mx)
        o[:, c0:c1] = (w_s[..., None] * o_swa + w_g[..., None] * o_gsa) / (w_s + w_g)[..., None]
        lse_swa[:, c0:c1], lse_gsa[:, c0:c1] = ls, lg
        # state pass, nha_fla/ops/nha/chunk_fused.py:100-107
        glast = gc[:, -1]                                    # [B,H,M]
        sdec = sg_[:, c0:c1] * torch.exp(glast[:, None] - gc)
        hk = hk * glast.exp()[:, :, None, :] + torch.einsum("bjhk,bjhm->bhkm", kg[:, c0:c1], sdec)
        hv = hv * glast.exp()[:, :, :, None] + torch.einsum("bjhm,bjhv->bhmv", sdec, vg[:, c0:c1])
    return o, lse_swa, lse_gsa, hk, hv


def prefill_grad_ref(q_swa, k_swa, q_gsa, k_gsa, v, s, g, do, *, window_size_left, gsa_kv_shift=0,
                     cu_seqlens=None, initial_state=None, scale=None, dlse_swa=None, dlse_gsa=None,
                     dht=None, dtype=torch.float64):
    """Gradients of the prefill op: reverse-mode differentiation of the per-token recurrence of
    ``prefill_ref`` itself (no second formula), which is what
    ChunkNativeHybridAttentionFunction.backward (nha_fla/ops/nha/chunk.py:490-564) has to equal:
    window-branch gradients (:499-511), slot-branch gradients with the merged-softmax coupling
    (:514-530), un-shifting of the slot-branch gradients (:533-543), dv accumulated over both
    branches (:559), initial-state gradients.  The scalar differentiated is
    ``<o, do> + <lse_swa, dlse_swa> + <lse_gsa, dlse_gsa> + <hkt, dht[0]> + <hvt, dht[1]>``.
    Pinned by central finite differences of ``prefill_ref`` (tests/test_oracle_pins.py).

    Returns a dict with dq_swa, dk_swa, dq_gsa, dk_gsa, dv, ds, dg and, when an initial state is
    given, dh0k, dh0v (all ``dtype``, shapes of the corresponding inputs)."""
    B, T, HQ, K = q_swa.shape
    H = k_swa.shape[2]
    M = s.shape[-1]
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    leaf = lambda x: x.detach().to("cpu", dtype).clone().requires_grad_(True)
    names = ["q_swa", "k_swa", "q_gsa", "k_gsa", "v", "s", "g"]
    xs = [leaf(x) for x in (q_swa, k_swa, q_gsa, k_gsa, v, s, g)]
    h0 = None
    if initial_state is not None:
        h0 = (leaf(initial_state[0]), leaf(initial_state[1]))
    cu = [0, T] if cu_seqlens is None else [int(c) for c in cu_seqlens]
    total = torch.zeros((), dtype=dtype)
    seqs = [(b, 0, T, b) for b in range(B)] if cu_seqlens is None else \
        [(0, cu[n], cu[n + 1], n) for n in range(len(cu) - 1)]
    cst = lambda x: None if x is None else x.detach().to("cpu", dtype)
    do, dlse_swa, dlse_gsa = cst(do), cst(dlse_swa), cst(dlse_gsa)
    dht = None if dht is None else (cst(dht[0]), cst(dht[1]))
    for b, st, en, n in seqs:
        sl = slice(st, en)
        part = [x[b:b + 1, sl] for x in xs]
        if h0 is not None:
            hk, hv = h0[0][n:n + 1], h0[1][n:n + 1]
        else:
            hk = torch.zeros(1, H, K, M, dtype=dtype)
            hv = torch.zeros(1, H, M, V, dtype=dtype)
        o, ls, lg, hk, hv = _prefill_equal_len(*part, window_size_left, gsa_kv_shift, scale, hk, hv)
        total = total + (o * do[b:b + 1, sl]).sum()
        if dlse_swa is not None:
            total = total + (ls * dlse_swa[b:b + 1, sl]).sum()
        if dlse_gsa is not None:
            total = total + (lg * dlse_gsa[b:b + 1, sl]).sum()
        if dht is not None:
            total = total + (hk[0] * dht[0][n]).sum() + (hv[0] * dht[1][n]).sum()
    wrt = xs + (list(h0) if h0 is not None else [])
    grads = torch.autograd.grad(total, wrt, allow_unused=True)
    out = {"d" + nm: (gr if gr is not None else torch.zeros_like(x)) for nm, gr, x in zip(names, grads[:7], xs)}
    if h0 is not None:
        out["dh0k"], out["dh0v"] = grads[7], grads[8]
    return out


def decode_ref(q, k, v, g, sw_k, sw_v, *, sq=None, s=None, cos=None, sin=None,
               initial_state=None, scale=None, dtype=torch.float64):
    """One decode step (scripts/verify_opt_parity.py:88-125; API of
    nha_fla/ops/nha/fused_recurrent.py:431-445).

    q ``[B,1,HQ,K]`` raw; popped k/v/g ``[B,1,H,*]``; ``sw_k/sw_v [B,W,H,*]`` ascending in time
    with the query token's own entry as the last row; either ``sq`` (pre-rotated query, ``sw_k``
    pre-rotated) or ``cos/sin [B|1, W2>=W, K]`` whose last W rows are used (row W-1 = query
    position) with raw ``q``/``sw_k``.  ``s`` defaults to ``1 - exp(g)`` (fused_recurrent.py:282-285).
    Returns ``(o [B,1,HQ,V], hkt, hvt, p_slots [B,HQ,M], p_win [B,HQ,W])``."""
    B, _, HQ, K = q.shape
    W, H = sw_k.shape[1], sw_k.shape[2]
    M, V = g.shape[-1], v.shape[-1]
    NG = HQ // H
    if scale is None:
        scale = K ** -0.5
    cast = lambda x: x.detach().to("cpu", dtype)
    q, k, v, g, sw_k, sw_v = map(cast, (q, k, v, g, sw_k, sw_v))
    s = (1.0 - g.exp()) if s is None else cast(s)
    if cos is not None:
        assert sq is None
        cos, sin = cast(cos)[:, -W:], cast(sin)[:, -W:]
        sq_ = rope_rotate_half(q, cos[:, -1:], sin[:, -1:])
        sk_ = rope_rotate_half(sw_k, cos, sin)
    else:
        sq_, sk_ = cast(sq), sw_k
    if initial_state is not None and initial_state[0] is not None:
        hk, hv = cast(initial_state[0]), cast(initial_state[1])
    else:
        hk = torch.zeros(B, H, K, M, dtype=dtype)
        hv = torch.zeros(B, H, M, V, dtype=dtype)
    hk, hv = gsa_step(hk, hv, k[:, 0], v[:, 0], s[:, 0], g[:, 0])
    ok = torch.einsum("bqk,bqkm->bqm", q[:, 0] * scale, _expand(hk, NG, 1))
    sw = torch.einsum("bqk,bwqk->bqw", sq_[:, 0] * scale, _expand(sk_, NG, 2))
    p = torch.softmax(torch.cat([ok, sw], -1), -1)
    o = torch.einsum("bqm,bqmv->bqv", p[..., :M], _expand(hv, NG, 1)) \
        + torch.einsum("bqw,bwqv->bqv", p[..., M:], _expand(sw_v, NG, 2))
    return o[:, None], hk, hv, p[..., :M], p[..., M:]


def decode_ring_ref(q_gsa, q_swa, k_new, k_gsa_new, v_new, g_new, ring_k, ring_kg, ring_v, ring_g,
                    count, hk, hv, *, scale=None, dtype=torch.float64):
    """Decode step on a W-slot ring buffer (the layout the HIP decode kernel keeps resident).

    Per sequence b with ``c = count[b]`` tokens cached so far: the new token goes to slot
    ``c % W``; if ``c >= W`` that slot holds the oldest token, which is popped into the slots
    first (models/qwen3_moe_nha/qwennha.py:151-176: pop is read before the cache update; an
    absent pop is the exact no-op ``k=v=0, g=0, s=0``, :153-160).  The window is then the
    ``min(c+1, W)`` valid ring entries (any order: softmax is permutation invariant and the
    ring holds already-rotated keys).  ring_k: window keys, ring_kg: slot-branch keys,
    ring_v, ring_g ``[B,W,H,*]``.  Returns ``(o [B,HQ,V], hk, hv)`` and updates the rings
    (returned as new tensors)."""
    B, HQ, K = q_gsa.shape
    W, H = ring_k.shape[1], ring_k.shape[2]
    M, V = ring_g.shape[-1], ring_v.shape[-1]
    NG = HQ // H
    if scale is None:
        scale = K ** -0.5
    cast = lambda x: x.detach().to("cpu", dtype)
    q_gsa, q_swa, k_new, k_gsa_new, v_new, g_new = map(cast, (q_gsa, q_swa, k_new, k_gsa_new, v_new, g_new))
    rk, rkg, rv, rg = (cast(x).clone() for x in (ring_k, ring_kg, ring_v, ring_g))
    hk, hv = cast(hk).clone(), cast(hv).clone()
    o = torch.zeros(B, HQ, V, dtype=dtype)
    for b in range(B):
        c = int(count[b])
        slot = c % W
        if c >= W:
            gp = rg[b, slot]
            hk[b], hv[b] = gsa_step(hk[b], hv[b], rkg[b, slot], rv[b, slot], 1.0 - gp.exp(), gp)
        rk[b, slot], rkg[b, slot], rv[b, slot], rg[b, slot] = k_new[b], k_gsa_new[b], v_new[b], g_new[b]
        fill = min(c + 1, W)
        ok = torch.einsum("qk,qkm->qm", q_gsa[b] * scale, _expand(hk[b], NG, 0))
        sw = torch.einsum("qk,wqk->qw", q_swa[b] * scale, _expand(rk[b, :fill], NG, 1))
        p = torch.softmax(torch.cat([ok, sw], -1), -1)
        o[b] = torch.einsum("qm,qmv->qv", p[:, :M], _expand(hv[b], NG, 0)) \
            + torch.einsum("qw,wqv->qv", p[:, M:], _expand(rv[b, :fill], NG, 1))
    return o, hk, hv, (rk, rkg, rv, rg)


def fused_recurrent_ref(q, k, v, sliding_window, s, g, *, scale=None, initial_state=None,
                        dtype=torch.float64):
    """T == 1 step where the caller supplies the window logits
    (scripts/verify_opt_parity.py:128-144; nha_fla/ops/nha/fused_recurrent.py:587-682).
    Returns ``(o [B,1,HQ,V] slot part only, swa_score [B,1,HQ,W], hkt, hvt)``."""
    B, _, HQ, K = q.shape
    H = k.shape[2]
    M, V = s.shape[-1], v.shape[-1]
    NG = HQ // H
    if scale is None:
        scale = K ** -0.5                                    # fused_recurrent.py:661-662
    cast = lambda x: x.detach().to("cpu", dtype)
    q, k, v, sliding_window, s, g = map(cast, (q, k, v, sliding_window, s, g))
    if initial_state is not None and initial_state[0] is not None:
        hk, hv = cast(initial_state[0]), cast(initial_state[1])
    else:
        hk = torch.zeros(B, H, K, M, dtype=dtype)
        hv = torch.zeros(B, H, M, V, dtype=dtype)
    hk, hv = gsa_step(hk, hv, k[:, 0], v[:, 0], s[:, 0], g[:, 0])
    ok = torch.einsum("bqk,bqkm->bqm", q[:, 0] * scale, _expand(hk, NG, 1))
    p = torch.softmax(torch.cat([ok, sliding_window[:, 0]], -1), -1)
    o = torch.einsum("bqm,bqmv->bqv", p[..., :M], _expand(hv, NG, 1))
    return o[:, None], p[..., M:][:, None], hk, hv
