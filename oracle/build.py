"""Build recipe of the CPU checker (test infrastructure, not part of the product).

    python oracle/build.py            # oracle/_build/liboracle.so and liboracle_omp.so
    python oracle/build.py --sanitize # oracle/_build/liboracle_san.so (g++ -fsanitize=address,undefined)

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


LIB_SAN = os.path.join(OUT_DIR, "liboracle_san.so")
# AddressSanitizer + UndefinedBehaviorSanitizer build (CPU only): any report aborts the process
SANITIZE = ["-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined,float-cast-overflow",
            "-fno-sanitize-recover=all"]


def build_sanitized(force=True):
    """oracle/_build/liboracle_san.so: the checker under ASan / UBSan.  A Python process loads it only with the ASan
    runtime preloaded (``sanitizer_env()``); ``ADOP_ORACLE_SANITIZE=1`` makes ``oracle.lib()`` pick this build."""
    os.makedirs(OUT_DIR, exist_ok=True)
    if force or not os.path.exists(LIB_SAN) or os.path.getmtime(LIB_SAN) < os.path.getmtime(SRC):
        subprocess.check_call([c for c in COMMON if c != "-O2"] + SANITIZE + [SRC, "-o", LIB_SAN])
    return LIB_SAN


def sanitizer_env(env=None):
    """Environment of a child process that runs the sanitized checker: the ASan runtime goes first in LD_PRELOAD
    (whatever is there stays), leak reports are off (the interpreter itself leaks)."""
    env = dict(os.environ if env is None else env)
    asan = subprocess.check_output(["g++", "-print-file-name=libasan.so"]).decode().strip()
    env["LD_PRELOAD"] = asan + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    env["ADOP_ORACLE_SANITIZE"] = "1"
    return env


def build(force=True):
    os.makedirs(OUT_DIR, exist_ok=True)
    for lib, extra in ((LIB, []), (LIB_OMP, ["-fopenmp"])):
        if not force and os.path.exists(lib) and os.path.getmtime(lib) >= os.path.getmtime(SRC):
            continue
        subprocess.check_call(COMMON + extra + [SRC, "-o", lib])
    return LIB, LIB_OMP


if __name__ == "__main__":
    if "--sanitize" in sys.argv:
        print(build_sanitized(force="--if-stale" not in sys.argv))
    else:
        print(build(force="--if-stale" not in sys.argv))
