"""Build recipe for libksa_hip.so (hipcc, gfx950 only)."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libksa_hip.so")
SOURCES = ["ksa_api.hip", "ksa_index.hip", "ksa_prefill.hip", "ksa_decode.hip", "ksa_cache.hip",
           "ksa_pre.hip", "ksa_elementwise.hip", "ksa_gemm_rows.hip",
           "ksa_probe.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # scores never hold NaN unless the inputs do; without this every fmax is preceded by a
    # canonicalising v_max
    "-fno-honor-nans",
]


def build(verbose: bool = False, extra_flags=(), out: str = LIB) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, *extra_flags, "-I", CSRC, "-o", out] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is expected
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return out


if __name__ == "__main__":
    print(build(verbose=True))
