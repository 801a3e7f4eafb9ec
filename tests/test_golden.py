"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py): the CPU checker must still
reproduce them (CPU test), and the HIP path must match them (GPU test)."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402

NAMES = sorted(make_golden.golden_scenes())


def load(name):
    return np.load(os.path.join(HERE, "golden", name + ".npz"))


@pytest.mark.parametrize("name", NAMES)
def test_checker_reproduces_fixture(oracle_mod, name):
    hs = make_golden.golden_scenes()[name]
    got = make_golden.run(hs)
    want = load(name)
    assert sorted(got) == sorted(want.files)
    for k in want.files:
        assert np.array_equal(got[k], want[k], equal_nan=True), k  # same machine code, same bits


@pytest.mark.gpu
@pytest.mark.parametrize("path", [1, 2], ids=["direct", "tiles"])
@pytest.mark.parametrize("name", NAMES)
def test_hip_path_matches_fixture(name, path):
    import torch
    from adop_amd import render, scenes
    from helpers import announce, assert_close, assert_norm_close, run_hip_forward

    announce(f"golden {name} forward_path={path}")
    hs = make_golden.golden_scenes()[name]
    want = load(name)
    scene, info, ctx, images, masks = run_hip_forward(hs, forward_path=path)
    for l in range(hs.num_layers):
        L = info.cache.layers_cuda[l]
        assert np.array_equal(L.depth_index_tensor.cpu().numpy().view(np.uint64), want[f"depth_index_{l}"])
        assert np.array_equal(L.weight.cpu().numpy(), want[f"weight_{l}"])
        assert_close(images[l].cpu().numpy(), want[f"out_{l}"], 1e-5, 1e-7, f"out {l}")
    gout = [torch.from_numpy(g).cuda() for g in scenes.upstream_grads(hs, 77)]
    g_tex, g_bg, g_pts, g_pose, g_intr = render.BlendPointCloudBackward(ctx, info, gout)
    torch.cuda.synchronize()
    assert_close(g_tex.cpu().numpy(), want["grad_texture"], 1e-4, 1e-6, "grad_texture")
    assert_close(g_bg.cpu().numpy(), want["grad_background"], 1e-4, 1e-5, "grad_background")
    assert np.array_equal(info.cache.output_gradient_point_count.cpu().numpy(), want["grad_points_count"])
    # the fixture's backward ran on the checker's own forward image: tensor-level bound (see test_parity_gpu)
    assert_norm_close(g_pts.cpu().numpy(), want["grad_points"], 1e-4, "grad_points")
    assert_norm_close(g_pose.cpu().numpy(), want["grad_pose"], 1e-4, "grad_pose")
    assert_norm_close(g_intr.cpu().numpy(), want["grad_intrinsics"], 1e-4, "grad_intrinsics")
