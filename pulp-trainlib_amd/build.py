"""Build libptl_hip.so (HIP kernels for gfx950 + the C entry points) in-tree.

Usage: python pulp-trainlib_amd/build.py [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libptl_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
CLANG = os.environ.get("PTL_CC", "/opt/rocm/lib/llvm/bin/clang")

HIP_SOURCES = ["ptl_runtime.hip", "ptl_gemm.hip", "ptl_gemm_async_sel.hip", "ptl_gemm_plain_f16.hip", "ptl_gemm_plain_f32.hip", "ptl_gemm_async_f16_c0.hip", "ptl_gemm_async_f16_c1.hip", "ptl_gemm_async_f16_c2.hip", "ptl_gemm_async_f16_c3.hip", "ptl_gemm_async_f32_c0.hip", "ptl_gemm_async_f32_c1.hip", "ptl_gemm_async_f32_c2.hip", "ptl_gemm_async_f32_c3.hip", "ptl_layers.hip", "ptl_conv_tile.hip", "ptl_conv_wg.hip", "ptl_conv_taps.hip", "ptl_conv_halo.hip", "ptl_conv_small.hip", "ptl_tensor_ops.hip", "ptl_mhsa.hip", "ptl_glue.hip", "ptl_probe.hip"]
C_SOURCES = ["pulp_entry.c"]

# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU ops.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-I", CSRC]
C_FLAGS = ["-O2", "-fPIC", "-std=gnu99", "-Wall", "-I", os.path.join(ROOT, "include"), "-I", CSRC]


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), res.stdout))
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if out.strip():
        print(out)


def build(force=True):
    """Compile every source and link the shared library. Always recompiles when force is True."""
    os.makedirs(OBJ, exist_ok=True)
    jobs = []
    objs = []
    for src in HIP_SOURCES:
        o = os.path.join(OBJ, src + ".o")
        objs.append(o)
        jobs.append([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", o])
    for src in C_SOURCES:
        o = os.path.join(OBJ, src + ".o")
        objs.append(o)
        jobs.append([CLANG] + C_FLAGS + ["-c", os.path.join(CSRC, src), "-o", o])
    if not force:
        deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [
            os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include"))]
        newest = max(os.path.getmtime(d) for d in deps)
        if os.path.exists(LIB) and os.path.getmtime(LIB) >= newest:
            return LIB
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        list(ex.map(_run, jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(force=True))
