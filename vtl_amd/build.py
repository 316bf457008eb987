"""Builds libvtlhip.so (gfx950) with hipcc.  Run as `python -m vtl_amd.build`."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libvtlhip.so")
OBJ_DIR = os.path.join(PKG_DIR, "_build")
# bench.py's measurement aid (an MFMA-only loop): a library of its own, no part of the product
BENCH_PROBE_PATH = os.path.join(PKG_DIR, "libvtlbenchprobe.so")
SOURCES = ["runtime.hip", "quant.hip", "gemm_i8.hip", "matmul_f64acc.hip", "tensor_ops.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # the f32 epilogue and the quantizer are specified as separately rounded
    # operations: no fused multiply-add contraction
    "-ffp-contract=off",
    # no packed-f32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]

# Flags of single sources.  The f64 MFMA accumulators of the matmul kernel fit
# the architectural VGPRs; asking for the VGPR form of MFMA keeps the compiler
# from shuttling them to and from the accumulation registers every k-step.
SOURCE_FLAGS = {
    "matmul_f64acc.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so; drop that line
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out, flush=True)


def build_lib(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile every HIP source (one object each, side by side) and link
    vtl_amd/libvtlhip.so."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    includes = ["-I", os.path.join(REPO_ROOT, "include"), "-I", CSRC]
    objects = [os.path.join(OBJ_DIR, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(i: int) -> None:
        src = SOURCES[i]
        _run([hipcc(), *HIPCC_FLAGS, *SOURCE_FLAGS.get(src, []), *(extra_flags or []), *includes,
              "-c", os.path.join(CSRC, src), "-o", objects[i]], verbose)

    def compile_probe() -> None:
        _run([hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
              os.path.join(CSRC, "bench_probe.hip"), "-o", BENCH_PROBE_PATH], verbose)

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES) + 1)) as pool:
        probe = pool.submit(compile_probe)
        list(pool.map(compile_one, range(len(SOURCES))))
        probe.result()
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", LIB_PATH], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_lib(verbose=True, extra_flags=sys.argv[1:]))
