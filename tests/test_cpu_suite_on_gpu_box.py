"""The CPU pinning tests (closed forms, finite differences, brute force: the only guard of the arithmetic that checker
and kernels share line for line) are not marked `gpu`; this test runs them on the GPU box as well, in a child process
that touches no GPU, so that a run of the GPU tests alone also vouches for the checker it compares with."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.gpu
def test_cpu_pins_pass_on_this_box():
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", ROCR_VISIBLE_DEVICES="")
    r = subprocess.run([sys.executable, "-m", "pytest", "tests", "-q", "-x", "-m", "not gpu and not sanitize", "-p",
                        "no:cacheprovider"], cwd=ROOT, env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-2000:])
    tail = r.stdout.strip().splitlines()[-1]
    print("[cpu suite]", tail, flush=True)
    assert " passed" in tail and "failed" not in tail
