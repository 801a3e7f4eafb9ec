"""Parity at the largest clouds the library takes, against the CPU checker: 2^28 - 1024 points through both forward
paths (the tile path's limit: point ids have 28 bits in a bin entry), 2^28 + 1024 (the library's choice must fall
back to the direct path) and 2^30 points (the limit of a call), forward and backward with all gradients.  The scenes
take minutes to generate and 10 to 100 GB of host memory, so the cases run only when ADOP_TEST_POINT_LIMITS=1; a line
is printed every 30 s while they work."""
import os
import threading
import time

import pytest

from helpers import announce, check_backward, check_forward, download_forward, run_hip_forward

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("ADOP_TEST_POINT_LIMITS") != "1",
                                 reason="takes several minutes and 100 GB of host memory: set ADOP_TEST_POINT_LIMITS=1")]


@pytest.fixture
def heartbeat():
    stop = threading.Event()

    def beat():
        while not stop.wait(30):
            print(time.strftime("%H:%M:%S"), "... working", flush=True)

    t = threading.Thread(target=beat, daemon=True)
    t.start()
    yield
    stop.set()


@pytest.mark.parametrize("n,paths", [((1 << 28) - 1024, (2, 1)), ((1 << 28) + 1024, (0,)), (1 << 30, (0,))],
                         ids=["tile_path_limit", "past_the_tile_path_limit", "call_limit"])
def test_largest_clouds(oracle_mod, heartbeat, n, paths):
    import torch
    from adop_amd import render, scenes

    announce(f"{n} points in 3840 x 2160, 5 levels, fp16 descriptors: generate")
    hs = scenes.config4(n=n, w=3840, h=2160, levels=5, frames=1, point_order="generated")
    hs.dropout = None
    hs.params.ghost_gradients = 0  # spatial gradients of the rendered points
    announce("checker forward")
    ref = oracle_mod.forward(hs, omp=True)  # (the OpenMP build: held to the serial one by tests/test_oracle_omp.py)
    assert int(ref.stats.visible[0]) > 0.8 * n
    for path in paths:
        announce(f"{n} points, forward_path={path}: forward")
        scene, info, ctx, images, masks = run_hip_forward(hs, collect_stats=True, forward_path=path)
        check_forward(hs, ref, ctx, images, masks, info, stats=True)
        if path == 1:
            continue
        announce("backward")
        gout = scenes.upstream_grads(hs, 5)
        grads = render.BlendPointCloudBackward(ctx, info, [torch.from_numpy(g).cuda() for g in gout], (True, True, True))
        torch.cuda.synchronize()
        announce("checker backward")
        refb = oracle_mod.backward(hs, download_forward(hs, info, images, masks), gout, True, True, True, omp=True)
        check_backward(hs, refb, grads, info, stats=True)
        del grads, gout, refb, scene, info, ctx, images, masks
        torch.cuda.empty_cache()
