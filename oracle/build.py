"""Build the CPU oracle (test infrastructure) as oracle/libptl_oracle.so.

ROCm's clang is used because gcc 11 has no _Float16 on x86-64.  The reference
library itself is NOT built: its sources include the PULP-SDK header pmsis.h,
which this image does not have, so there is no oracle/_ref.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB = os.path.join(HERE, "libptl_oracle.so")
CLANG = os.environ.get("PTL_CC", "/opt/rocm/lib/llvm/bin/clang")

# x86-64-v3 (AVX2/FMA/F16C) runs on this container and on the GPU host alike;
# contraction is off so fp32 sums are the plain multiply-then-add sequence.
FLAGS = ["-O3", "-fPIC", "-shared", "-std=gnu99", "-march=x86-64-v3", "-ffp-contract=off", "-fopenmp", "-Wall",
         "-Wno-unused-function", "-I", os.path.join(ROOT, "include")]


def build():
    cmd = [CLANG] + FLAGS + [os.path.join(HERE, "ptl_oracle.c"), os.path.join(HERE, "ptl_oracle_mhsa.c"), os.path.join(HERE, "ptl_oracle_glue.c"), "-o", LIB,
                             "-Wl,-rpath,/opt/rocm/lib/llvm/lib", "-lm"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + res.stdout)
    if res.stdout.strip():
        print(res.stdout)
    return LIB


if __name__ == "__main__":
    print(build())
