"""Builds libdeepj_hip.so for gfx950 with hipcc (run on the CPU: hipcc cross-compiles).

    python -m deepj_amd.build            # rebuild everything
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libdeepj_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops off: v_pk_*_f32 forms are not used by this library's kernels.
# kernarg preload: a kernel's leading scalar arguments (pointers, sizes; as many as fit in 14 registers) reach a
# wavefront in registers at launch instead of through a load from the argument buffer that every other load of the
# kernel would have to wait for.  The latency-bound decode kernels take their operands as separate arguments,
# the first-needed ones in front, for this reason.
COMMON = ["-x", "hip", f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-kernarg-preload-count=16"]

# Kernels whose results are compared element by element with the CPU backend keep
# a*b+c unfused (the CPU never fuses); the contraction kernels use fma on purpose.
SOURCES = {
    "runtime.cpp": [],
    "kernels_elementwise.hip": ["-ffp-contract=off"],
    "kernels_reduce.hip": ["-ffp-contract=off"],
    # matrix-core accumulators in ordinary vector registers: the kernels rescale or mask them with vector
    # instructions after every few products, and each trip through the accumulator file costs a move per value
    "kernels_matmul.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "kernels_q8.hip": [],
    "kernels_attn.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "kernels_decode.hip": [],
    "runner.cpp": [],
    "host_random.cpp": [],
}


def _compile(item):
    src, extra = item
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *COMMON, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    return obj, out


def build(verbose: bool = False) -> str:
    os.makedirs(OBJ, exist_ok=True)
    present = {s: e for s, e in SOURCES.items() if os.path.exists(os.path.join(CSRC, s))}
    with ThreadPoolExecutor(max_workers=min(8, len(present))) as ex:
        results = list(ex.map(_compile, present.items()))
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    objs = [o for o, _ in results]
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB, *objs, "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
