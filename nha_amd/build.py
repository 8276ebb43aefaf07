"""Build libnha_hip.so (gfx950) in-tree with hipcc.  `python -m nha_amd.build` or build_library()."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libnha_hip.so")
SOURCES = ["abi.hip", "decode.hip", "decode_mfma.hip", "prefill_simple.hip", "prefill_mfma.hip", "prefill_ring.hip", "prefill_ring256.hip", "prefill_bwd.hip", "prefill_bwd_mfma.hip", "prefill_bwd_ring.hip",
           "layer_fuse.hip", "hybrid_fuse.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffast-math" if False else "-fno-fast-math",
    # hipcc -O3 may otherwise emit packed-fp32 VALU forms from ordinary float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
]


# the MFMA kernels never produce NaN on purpose; without this flag every fmaxf operand is
# canonicalised by an extra VALU instruction in the softmax inner loop
EXTRA = {"prefill_mfma.hip": ["-fno-honor-nans"], "prefill_ring.hip": ["-fno-honor-nans"], "prefill_ring256.hip": ["-fno-honor-nans"], "decode_mfma.hip": ["-fno-honor-nans"],
         "prefill_bwd_mfma.hip": ["-fno-honor-nans"], "prefill_bwd_ring.hip": ["-fno-honor-nans"]}


STAMP = os.path.join(HERE, "build", "sources.sha256")


def sources_digest() -> str:
    """sha256 over the library's sources (csrc/ and the C header), in name order.  The build writes it beside the
    objects after a successful link; a test compares, so a library older than its sources does not pass for current."""
    import hashlib
    h = hashlib.sha256()
    files = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h")))
    inc = os.path.join(os.path.dirname(HERE), "include")
    files += sorted(os.path.join(inc, f) for f in os.listdir(inc) if f.endswith(".h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def build_library(verbose: bool = False, jobs: int = 4) -> str:
    digest = sources_digest()
    if os.path.exists(STAMP):
        os.remove(STAMP)
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
        cmd = [HIPCC, *FLAGS, *EXTRA.get(src, []), *os.environ.get("NHA_EXTRA_FLAGS", "").split(),
               "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("link failed:\n" + out.stdout)
    with open(STAMP, "w") as fh:
        fh.write(digest + "\n")
    return LIB


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        real = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if real and os.environ.get("NHA_BUILD_VERBOSE"):
            print(real)


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
