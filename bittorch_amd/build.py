"""Builds ``_hip/libbittorch_hip.so`` (the C-ABI HIP library) with hipcc for gfx950.

Usage: ``python -m bittorch_amd.build``.  The library has no torch dependency;
hipcc cross-compiles it on a machine without a GPU.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
OUT_DIR = os.path.join(_HERE, "_hip")
LIB_PATH = os.path.join(OUT_DIR, "libbittorch_hip.so")

SOURCES = ["capi.hip", "quantize_pack.hip", "stream_gemm.hip", "gemv_planes.hip", "gemv_i8_group.hip", "gemm_i8.hip", "gemm_f16.hip", "act_quant.hip", "row_ops.hip", "misc_kernels.hip"]

# packed fp32 VALU forms are disabled on purpose (they have produced wrong
# results on this hardware generation's boxes); the host pass warns that it
# does not know the feature, which is harmless.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    # every float multiply and add rounds on its own (the epilogues restate the
    # reference's operation order; a fused multiply-add would change the last bit)
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# per-source extra flags
EXTRA_FLAGS = {
    # the iterative ILP scheduler keeps the MFMA accumulators in place across the
    # software-pipelined main loop (the default strategy permutes them every iteration)
    "gemm_i8.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp"],
    "gemm_f16.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp"],
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def build(verbose: bool = False, extra_flags=()) -> str:
    """Compile every kernel source and link the shared library; returns its path."""
    os.makedirs(OUT_DIR, exist_ok=True)
    hipcc = _hipcc()
    objs = []

    def compile_one(src: str) -> str:
        obj = os.path.join(OUT_DIR, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), *extra_flags, "-c",
               os.path.join(CSRC, src), "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
        if verbose and res.stderr.strip():
            print(res.stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc link failed:\n{res.stdout}\n{res.stderr}")
    return LIB_PATH


def build_bench_probe() -> str:
    """The benchmark's own measurement aid (``bench_mfma_probe.hip`` at the repository root): a separate
    shared object that only ``bench.py`` loads."""
    root = os.path.dirname(_HERE)
    src, out = os.path.join(root, "bench_mfma_probe.hip"), os.path.join(root, "bench_mfma_probe.so")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", src, "-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on bench_mfma_probe.hip:\n{res.stdout}\n{res.stderr}")
    return out


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_bench_probe())
