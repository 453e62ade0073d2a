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
BASE = ["-x", "hip", f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
PRELOAD = ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
COMMON = BASE + PRELOAD
# A second build of the same sources without kernarg preload, for runs under a hardware-counter profiler (the
# counter-collecting rocprofv3 crashed on the host at the first dispatch of a kernel with preloaded arguments; the
# bytes a kernel moves do not depend on how its arguments arrive).  DEEPJ_HIP_LIBRARY selects it at run time.
LIB_NO_PRELOAD = os.path.join(HERE, "libdeepj_hip_nopreload.so")

# Kernels whose results are compared element by element with the CPU backend keep
# a*b+c unfused (the CPU never fuses); the contraction kernels use fma on purpose.
SOURCES = {
    "runtime.cpp": [],
    "kernels_elementwise.hip": ["-ffp-contract=off"],
    "kernels_reduce.hip": ["-ffp-contract=off"],
    # matrix-core accumulators in ordinary vector registers: the kernels rescale or mask them with vector
    # instructions after every few products, and each trip through the accumulator file costs a move per value
    "kernels_matmul.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "kernels_gemm_f16.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "kernels_q8.hip": [],
    "kernels_attn.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "runner.cpp": [],
    "host_random.cpp": [],
}


PACKED_FLAG = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# hipcc hands -Xclang options to the host (x86-64) pass as well, which does not know the AMDGPU feature and says so,
# once per use; only that exact line is dropped from the compiler output.  That the DEVICE pass honours the flag is
# checked by verify_packed_fp32_off() on every build.
_HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"

_PROBE = """#include <hip/hip_runtime.h>
__global__ void probe(const float2 *a, const float2 *b, float2 *o, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) { float2 x = a[i], y = b[i]; o[i] = make_float2(x.x * y.x + 1.0f, x.y * y.y + 1.0f); }
}
"""


def verify_packed_fp32_off() -> None:
    """Compiles a float2 kernel for gfx950 (device pass only, to assembly) with the library's flags and fails when
    a packed fp32 instruction (v_pk_add/mul/fma_f32) is in it; without the flag the same kernel must contain one,
    which shows that the probe can tell the difference."""
    import re
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "probe.hip")
        with open(src, "w") as f:
            f.write(_PROBE)

        def packed(flags):
            out = os.path.join(tmp, "probe.s")
            r = subprocess.run([HIPCC, "-x", "hip", f"--offload-arch={ARCH}", "-O3", "--cuda-device-only", "-S", *flags,
                                src, "-o", out], capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError("hipcc failed on the packed-fp32 probe:\n" + r.stdout + r.stderr)
            return len(re.findall(r"\bv_pk_(?:add|mul|fma)_f32\b", open(out).read()))

        if packed([]) == 0:
            raise RuntimeError("packed-fp32 probe: the kernel compiles without v_pk_*_f32 even with the feature on; "
                               "the probe no longer shows whether the flag works")
        if packed(PACKED_FLAG) != 0:
            raise RuntimeError("-packed-fp32-ops is not honoured by the device pass: v_pk_*_f32 in the probe kernel")


def _compile(item):
    src, extra, common, obj_dir = item
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *common, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if l.strip() != _HOST_PASS_NOTE)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    return obj, out


def build(verbose: bool = False, kernarg_preload: bool = True) -> str:
    obj_dir = OBJ if kernarg_preload else OBJ + "_nopreload"
    lib = LIB if kernarg_preload else LIB_NO_PRELOAD
    common = COMMON if kernarg_preload else BASE
    os.makedirs(obj_dir, exist_ok=True)
    verify_packed_fp32_off()
    present = [(s, e, common, obj_dir) for s, e in SOURCES.items() if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(present))) as ex:
        results = list(ex.map(_compile, present))
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    objs = [o for o, _ in results]
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", lib, *objs, "-lpthread"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return lib


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, kernarg_preload="--no-kernarg-preload" not in sys.argv))
