"""Build recipe for libksa_hip.so (hipcc, gfx950 only)."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libksa_hip.so")
# (the slowest units first: they run next to the others)
SOURCES = ["ksa_prefill_d256_bf16_regular.hip", "ksa_prefill_d256_bf16_general.hip", "ksa_prefill_d256_f16_regular.hip",
           "ksa_prefill_d256_f16_general.hip", "ksa_prefill.hip", "ksa_api.hip", "ksa_index.hip", "ksa_decode.hip", "ksa_decode_weights.hip", "ksa_cache.hip",
           "ksa_pre.hip", "ksa_elementwise.hip", "ksa_gemm_rows.hip", "ksa_mlp_rows.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # scores never hold NaN unless the inputs do; without this every fmax is preceded by a
    # canonicalising v_max
    "-fno-honor-nans",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is expected
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, extra_flags=(), out: str = LIB, csrc: str = CSRC, jobs: int = 8) -> str:
    """Compiles every source of `csrc` (one hipcc process each, `jobs` at a time) and links them
    into `out`.  Objects go to a `build/` folder next to `out`, named after it."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(os.path.dirname(os.path.abspath(out)), "build",
                          os.path.splitext(os.path.basename(out))[0])
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    cmds = [[hipcc, *FLAGS, *extra_flags, "-I", csrc, "-c", os.path.join(csrc, s), "-o", o]
            for s, o in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs], verbose)
    return out


if __name__ == "__main__":
    print(build(verbose=True))
