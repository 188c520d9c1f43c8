"""Compile the gfx950 HIP sources of this package into libomni_moe_hip.so (in-tree)."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libomni_moe_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["route.hip", "quant.hip", "norm.hip", "permute.hip", "gemm.hip", "combine.hip", "placement.hip", "diag.hip"]

# -ffp-contract=off: every fp32 operation of the kernels rounds once (the parity contract).
# The packed-fp32 feature is switched off for the device pass; the host pass does not know it
# and says so, which is harmless.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC)")


def build(verbose: bool = True) -> str:
    """Always compiles; returns the path of the shared library."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", LIB_PATH + ".tmp", *[os.path.join(CSRC, s) for s in SOURCES]]
    if verbose:
        print("[omni_infer_amd] " + " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
