"""Build recipe of the CPU checker (test infrastructure, not part of the product).

    python oracle/build.py            # oracle/_build/liboracle.so and liboracle_omp.so

The reference rasterizer itself cannot be compiled here (it needs CUDA and the absent saiga submodule), so
there is no oracle/_ref build; the checker is the restatement in adop_oracle.cpp.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "adop_oracle.cpp")
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "liboracle.so")
LIB_OMP = os.path.join(OUT_DIR, "liboracle_omp.so")

# -ffp-contract=off: no fused multiply-add, every operation rounds on its own (the operation order is the
# specification the HIP kernels are held to, bit for bit, for depth and index).
COMMON = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-ffp-contract=off", "-fno-fast-math", "-Wall", "-Wno-unknown-pragmas"]


def build(force=True):
    os.makedirs(OUT_DIR, exist_ok=True)
    for lib, extra in ((LIB, []), (LIB_OMP, ["-fopenmp"])):
        if not force and os.path.exists(lib) and os.path.getmtime(lib) >= os.path.getmtime(SRC):
            continue
        subprocess.check_call(COMMON + extra + [SRC, "-o", lib])
    return LIB, LIB_OMP


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
