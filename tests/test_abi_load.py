"""CPU-side checks of the C-ABI library: it loads, exports every symbol include/nha_hip.h
declares, validates arguments, and its host-only varlen tables equal the integer oracle."""
import ctypes as C
import os
import random
import re

import numpy as np
import pytest

from nha_amd import _lib
from nha_amd.varlen import chunk_tables
from oracle import varlen_index as VI

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_header_symbols():
    lib = _lib.load()
    header = open(os.path.join(ROOT, "include", "nha_hip.h")).read()
    declared = set(re.findall(r"\b(nha_[a-z_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.nha_abi_version() == _lib.ABI_VERSION


def test_library_is_built_from_the_current_sources():
    """The build records a digest of csrc/ and the header after a successful link: a compile error that leaves the
    previous library in place (or an edit without a rebuild) must not pass for the current code."""
    from nha_amd import build
    _lib.load()
    assert os.path.exists(build.STAMP), "no build stamp: run python -m nha_amd.build"
    with open(build.STAMP) as fh:
        assert fh.read().strip() == build.sources_digest(), "libnha_hip.so is older than its sources: run python -m nha_amd.build"


def test_struct_sizes_match_the_header(tmp_path):
    """sizeof and the offsets of the ctypes mirrors against the C compiler's view of the header."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    probes = [("NhaPrefillArgs", f) for f in ("q_swa", "scratch_bytes", "T_tot", "impl", "scale", "stream")]
    probes += [("NhaDecodeArgs", f) for f in ("mode", "scale", "q", "cos_sb", "count", "o", "stream", "count_next")]
    probes += [("NhaPrefillBwdArgs", f) for f in ("q_swa", "o", "dout", "dhvt", "dq_swa", "dg", "dh0v", "cu_seqlens",
                                                  "scratch_bytes", "T_tot", "dtype", "scale", "stream")]
    probes += [("NhaLayerPrologueArgs", f) for f in ("q", "q_swa", "g", "inv_freq", "cu_seqlens", "T_tot", "M", "feature_map",
                                                     "seqlen_offset", "dtype", "gate_logit_normalizer", "stream")]
    probes += [("NhaLayerEpilogueArgs", f) for f in ("o", "y", "weight", "bias", "rows", "dim", "dtype", "eps", "stream")]
    probes += [("NhaLayerPrologueBwdArgs", f) for f in ("q", "dq_swa", "dg", "dq", "df", "inv_freq", "cu_seqlens", "T_tot",
                                                        "feature_map", "dtype", "gate_logit_normalizer", "stream")]
    probes += [("NhaLayerEpilogueBwdArgs", f) for f in ("o", "dy", "dout", "weight", "dweight_partial", "dbias_partial",
                                                        "rows", "dim", "dtype", "eps", "stream")]
    probes += [("NhaShortConvArgs", f) for f in ("x", "weight", "bias", "y", "cu_seqlens", "T_tot", "KS", "activation", "dtype",
                                                 "stream")]
    probes += [("NhaShortConvBwdArgs", f) for f in ("x", "dy", "dx", "dweight_partial", "dbias_partial", "cu_seqlens", "T_tot",
                                                    "KS", "activation", "dtype", "stream")]
    probes += [("NhaHybridPrologueArgs", f) for f in ("q", "f", "q_stride", "f_stride", "q_weight", "cos", "cs_batch_stride", "positions", "inv_freq", "mask",
                                                      "q_out", "s_out", "B", "M", "dtype", "eps", "gate_logit_normalizer", "stream")]
    probes += [("NhaSinkWindowArgs", f) for f in ("q", "o", "lse", "cu_seqlens", "scratch", "scratch_bytes", "T_tot", "D", "window",
                                                  "sinks", "dtype", "scale", "stream")]
    src = ['#include <stdio.h>', '#include <stddef.h>', '#include "nha_hip.h"', 'int main(void) {',
           'printf("%zu %zu %zu\\n", sizeof(NhaPrefillArgs), sizeof(NhaDecodeArgs), sizeof(NhaPrefillBwdArgs));',
           'printf("%zu %zu\\n", sizeof(NhaLayerPrologueArgs), sizeof(NhaLayerEpilogueArgs));',
           'printf("%zu %zu\\n", sizeof(NhaLayerPrologueBwdArgs), sizeof(NhaLayerEpilogueBwdArgs));',
           'printf("%zu %zu\\n", sizeof(NhaShortConvArgs), sizeof(NhaShortConvBwdArgs));',
           'printf("%zu %zu\\n", sizeof(NhaHybridPrologueArgs), sizeof(NhaSinkWindowArgs));']
    src += [f'printf("%zu\\n", offsetof({t}, {f}));' for t, f in probes]
    src += ['return 0; }']
    cfile = tmp_path / "probe.c"
    cfile.write_text("\n".join(src))
    exe = tmp_path / "probe"
    subprocess.run(["gcc", "-I", os.path.join(root, "include"), str(cfile), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert int(out[0]) == C.sizeof(_lib.NhaPrefillArgs) and int(out[1]) == C.sizeof(_lib.NhaDecodeArgs)
    assert int(out[2]) == C.sizeof(_lib.NhaPrefillBwdArgs)
    assert int(out[3]) == C.sizeof(_lib.NhaLayerPrologueArgs) and int(out[4]) == C.sizeof(_lib.NhaLayerEpilogueArgs)
    assert int(out[5]) == C.sizeof(_lib.NhaLayerPrologueBwdArgs) and int(out[6]) == C.sizeof(_lib.NhaLayerEpilogueBwdArgs)
    assert int(out[7]) == C.sizeof(_lib.NhaShortConvArgs) and int(out[8]) == C.sizeof(_lib.NhaShortConvBwdArgs)
    assert int(out[9]) == C.sizeof(_lib.NhaHybridPrologueArgs) and int(out[10]) == C.sizeof(_lib.NhaSinkWindowArgs)
    for (t, f), off in zip(probes, out[11:]):
        assert getattr(getattr(_lib, t), f).offset == int(off), (t, f)


def test_argument_validation_without_gpu():
    lib = _lib.load()
    a = _lib.NhaPrefillArgs()
    assert lib.nha_prefill_fwd(C.byref(a)) == _lib.NHA_ERR_INVALID
    assert b"non-positive" in lib.nha_last_error()
    b = _lib.NhaPrefillBwdArgs()
    assert lib.nha_prefill_bwd(C.byref(b)) == _lib.NHA_ERR_INVALID and b"non-positive" in lib.nha_last_error()
    b.T_tot, b.N, b.NT, b.HQ, b.H, b.K, b.V, b.M = 64, 1, 1, 3, 2, 64, 64, 64
    assert lib.nha_prefill_bwd(C.byref(b)) == _lib.NHA_ERR_INVALID and b"multiple" in lib.nha_last_error()
    assert lib.nha_prefill_bwd_scratch_bytes(C.byref(b)) == 0
    b.HQ = 4
    assert lib.nha_prefill_bwd(C.byref(b)) == _lib.NHA_ERR_INVALID and b"required" in lib.nha_last_error()
    assert lib.nha_prefill_bwd_scratch_bytes(C.byref(b)) > 0
    d = _lib.NhaDecodeArgs()
    assert lib.nha_decode_step(C.byref(d)) == _lib.NHA_ERR_INVALID
    d.B = d.H = d.K = d.V = d.M = d.W = 8
    d.HQ = 12
    assert lib.nha_decode_step(C.byref(d)) == _lib.NHA_ERR_INVALID and b"multiple" in lib.nha_last_error()
    lp = _lib.NhaLayerPrologueArgs()
    assert lib.nha_layer_prologue(C.byref(lp)) == _lib.NHA_ERR_INVALID and b"non-positive" in lib.nha_last_error()
    lp.T_tot, lp.N, lp.HQ, lp.H, lp.K, lp.V, lp.M = 10, 1, 2, 1, 7, 8, 8
    assert lib.nha_layer_prologue(C.byref(lp)) == _lib.NHA_ERR_INVALID and b"even" in lib.nha_last_error()
    lp.K, lp.feature_map = 8, 3
    assert lib.nha_layer_prologue(C.byref(lp)) == _lib.NHA_ERR_INVALID and b"feature_map" in lib.nha_last_error()
    lp.feature_map = 1
    assert lib.nha_layer_prologue(C.byref(lp)) == _lib.NHA_ERR_INVALID and b"required" in lib.nha_last_error()
    le = _lib.NhaLayerEpilogueArgs()
    assert lib.nha_layer_epilogue(C.byref(le)) == _lib.NHA_ERR_INVALID and b"non-positive" in lib.nha_last_error()
    le.rows, le.dim = 4, 64
    assert lib.nha_layer_epilogue(C.byref(le)) == _lib.NHA_ERR_INVALID and b"required" in lib.nha_last_error()
    lpb = _lib.NhaLayerPrologueBwdArgs()
    assert lib.nha_layer_prologue_bwd(C.byref(lpb)) == _lib.NHA_ERR_INVALID and b"non-positive" in lib.nha_last_error()
    leb = _lib.NhaLayerEpilogueBwdArgs()
    leb.rows, leb.dim = 4, 64
    assert lib.nha_layer_epilogue_bwd(C.byref(leb)) == _lib.NHA_ERR_INVALID and b"required" in lib.nha_last_error()
    assert lib.nha_layer_epilogue_bwd_parts(0) == 0 and lib.nha_layer_epilogue_bwd_parts(33) == 2
    sc = _lib.NhaShortConvArgs()
    assert lib.nha_short_conv(C.byref(sc)) == _lib.NHA_ERR_INVALID and b"non-positive" in lib.nha_last_error()
    sc.T_tot, sc.N, sc.C, sc.KS = 16, 1, 64, 4
    assert lib.nha_short_conv(C.byref(sc)) == _lib.NHA_ERR_INVALID and b"required" in lib.nha_last_error()
    scb = _lib.NhaShortConvBwdArgs()
    scb.T_tot, scb.N, scb.C, scb.KS = 16, 1, 60, 4
    assert lib.nha_short_conv_bwd(C.byref(scb)) == _lib.NHA_ERR_INVALID and b"required" in lib.nha_last_error()
    assert lib.nha_short_conv_bwd_parts(0) == 0 and lib.nha_short_conv_bwd_parts(33) == 2
    with pytest.raises(_lib.NhaError):
        chunk_tables([0, 5, 5])          # zero-length sequence
    with pytest.raises(_lib.NhaError):
        chunk_tables([1, 5])             # does not start at 0


def test_varlen_tables_bit_exact_vs_oracle():
    random.seed(0)
    cases = [[128] * 4, [128, 64, 200, 10], [4096, 2048, 1, 1024, 2],
             [random.randint(1, 100) for _ in range(256)], [1, 2000, 3, 50, 4, 3000, 2, 7], [1], [64], [65]]
    rng = np.random.default_rng(0)
    lens, tot = [], 0
    while tot < 32768:                       # the varlen benchmark config's draw rule
        L = int(rng.integers(64, 4097))
        L = min(L, 32768 - tot)
        lens.append(L); tot += L
    cases.append(lens)
    for lens in cases:
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        for bt in (16, 64):
            idx, off = chunk_tables(cu, bt)
            ridx, roff = VI.chunk_tables_closed(cu, bt)
            assert idx.dtype == np.int32 and off.dtype == np.int32
            assert np.array_equal(idx, ridx) and np.array_equal(off, roff)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; --gpus N > 1 exits with a message instead of a number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_fallback_without_the_library_or_a_gpu(monkeypatch):
    """The ops have no CPU or eager path: host tensors are refused by name, and a missing library is an error at the
    first call, not a slower result."""
    import torch
    from nha_amd import chunk_nha, fused_recurrent_nha_decode
    x = torch.zeros(1, 8, 2, 64)
    g = torch.zeros(1, 8, 2, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        chunk_nha(x, x, x, x, x, g, g)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fused_recurrent_nha_decode(q=x[:, :1], k=x[:, :1], v=x[:, :1], g=g[:, :1], sw_k=x, sw_v=x, sq=x[:, :1])
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "nha_amd", "no_such_library.so"))
    with pytest.raises(RuntimeError, match="no CPU or eager fallback"):
        _lib.load()
