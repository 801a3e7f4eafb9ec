"""CPU sanitizer runs (AddressSanitizer + UndefinedBehaviorSanitizer; the GPU code itself cannot be sanitized on this
pool): the checker's pinning tests, its golden fixtures and the hostile-input scenes on an ASan / UBSan build of
oracle/adop_oracle.cpp, and the host side of the C-ABI (argument checks, workspace arithmetic) compiled with the host
sanitizers and driven with extreme sizes by tests/host_checks_driver.cpp.  Everything runs in child processes: the
ASan runtime has to be the first library of a process."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "adop_amd", "csrc")

pytestmark = pytest.mark.sanitize


def _run(cmd, env=None, cwd=ROOT, timeout=900):
    return subprocess.run(cmd, env=env, cwd=cwd, capture_output=True, text=True, timeout=timeout)


def test_the_sanitizer_set_up_catches_a_heap_overflow(tmp_path):
    """The mechanism itself: a library built with the flags of the sanitized checker, loaded into a child process with
    the same environment, is stopped at a one-byte heap overflow (a run that could not fail would show nothing)."""
    from oracle import build

    src = tmp_path / "overflow.c"
    src.write_text("#include <stdlib.h>\nint poke(int n) { char* p = (char*)malloc(8); p[n] = 1; int r = p[n]; free(p); return r; }\n")
    lib = tmp_path / "liboverflow.so"
    subprocess.check_call(["gcc", "-shared", "-fPIC"] + build.SANITIZE + [str(src), "-o", str(lib)])
    code = f"import ctypes, sys; L = ctypes.CDLL({str(lib)!r}); L.poke(int(sys.argv[1])); print('survived')"
    ok = _run([sys.executable, "-c", code, "7"], env=build.sanitizer_env())
    assert ok.returncode == 0 and "survived" in ok.stdout, ok.stderr[-2000:]
    bad = _run([sys.executable, "-c", code, "8"], env=build.sanitizer_env())
    # (UBSan's object-size check or ASan's red zone, whichever sees it first)
    assert bad.returncode != 0 and "survived" not in bad.stdout
    assert "AddressSanitizer" in bad.stderr or "runtime error" in bad.stderr


def test_checker_pins_fixtures_and_hostile_inputs_under_asan_ubsan():
    from oracle import build

    lib = build.build_sanitized(force=True)
    env = build.sanitizer_env()
    which = _run([sys.executable, "-c", "import oracle; print(oracle.lib()._name)"], env=env)
    assert which.returncode == 0 and which.stdout.strip() == lib, which.stderr[-2000:]
    r = _run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "not gpu", "-p", "no:cacheprovider",
              "tests/test_oracle_math.py", "tests/test_oracle_render.py", "tests/test_golden.py",
              "tests/test_hostile_inputs.py"], env=env)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])
    assert " passed" in r.stdout and "failed" not in r.stdout
    assert "AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr


def test_host_side_of_the_c_abi_under_asan_ubsan(tmp_path):
    """adop_raster.hip (argument checks, workspace layout, launch sequences) compiled with -fsanitize=address,undefined
    for the host, linked with the device objects of the library into tests/host_checks_driver.cpp's program, which
    asks for workspace sizes at the largest sizes the interface takes (2^30 points, 64 views of 2200 x 1500 x 5 levels,
    INT_MAX everywhere) and walks the rejections.  Nothing in it launches a kernel."""
    objs = ["forward_kernels.o", "binned_kernels.o", "tile_kernels.o", "backward_kernels.o", "env_kernels.o",
            "preprocess_kernels.o"]
    if not all(os.path.exists(os.path.join(CSRC, o)) for o in objs):
        subprocess.check_call(["make", "-j4", "-C", CSRC, "libadop_raster.so"])
    hipcc = "/opt/rocm/bin/hipcc"
    san_o = str(tmp_path / "adop_raster_san.o")
    flags = ["--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
             "-fhip-fp32-correctly-rounded-divide-sqrt", "-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops"]
    host_san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
                "-fno-sanitize-recover=all"]
    r = _run([hipcc] + flags + host_san + ["-c", "adop_raster.hip", "-o", san_o], cwd=CSRC)
    assert r.returncode == 0, r.stderr[-3000:]
    drv_o = str(tmp_path / "driver.o")
    r = _run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-c",
              os.path.join(ROOT, "tests", "host_checks_driver.cpp"), "-o", drv_o])
    assert r.returncode == 0, r.stderr[-3000:]
    exe = str(tmp_path / "host_checks")
    r = _run([hipcc, "--offload-arch=gfx950", "-fsanitize=address,undefined", "-fno-gpu-sanitize", drv_o, san_o] + objs +
             ["-o", exe], cwd=CSRC)
    assert r.returncode == 0, r.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=1", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    r = _run([exe], env=env)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])
    assert "0 failure(s)" in r.stdout and "FAIL" not in r.stdout
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr
    assert r.stdout.count("ok   ") >= 50
