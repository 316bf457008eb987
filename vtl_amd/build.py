"""Builds libvtlhip.so (gfx950) with hipcc.  Run as `python -m vtl_amd.build`."""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libvtlhip.so")
SOURCES = ["runtime.hip", "quant.hip", "gemm_i8.hip", "matmul_f64acc.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # the f32 epilogue and the quantizer are specified as separately rounded
    # operations: no fused multiply-add contraction
    "-ffp-contract=off",
    # no packed-f32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def build_lib(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile every HIP source into vtl_amd/libvtlhip.so."""
    cmd = [hipcc(), *HIPCC_FLAGS, *(extra_flags or []),
           "-I", os.path.join(REPO_ROOT, "include"), "-I", CSRC,
           *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; drop that line
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    print(build_lib(verbose=True, extra_flags=sys.argv[1:]))
