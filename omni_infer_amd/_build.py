"""Compile the gfx950 HIP sources of this package into libomni_moe_hip.so (in-tree)."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libomni_moe_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["route.hip", "quant.hip", "norm.hip", "permute.hip", "gemm.hip", "combine.hip", "placement.hip", "diag.hip"]

# -ffp-contract=off: every fp32 operation of the kernels rounds once (the parity contract).
# The packed-fp32 feature is switched off for the device pass; the host pass does not know it
# and says so, which is harmless.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]
NOISE = "is not a recognized feature for this target"


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC)")


def _run(cmd, verbose):
    if verbose:
        print("[omni_infer_amd] " + " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = True) -> str:
    """Always compiles (every source to an object of its own, side by side, then one link); returns
    the path of the shared library."""
    hipcc = hipcc_path()
    with tempfile.TemporaryDirectory(prefix="omni_moe_build_") as tmp:
        objs = [os.path.join(tmp, s.replace(".hip", ".o")) for s in SOURCES]
        jobs = [[hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objs)]
        with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            list(pool.map(lambda c: _run(c, verbose), jobs))
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH + ".tmp", *objs], verbose)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
