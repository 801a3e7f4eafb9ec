"""The OpenMP build of the CPU checker against the serial build.

The OpenMP build is what the GPU parity tests at the full BASELINE sizes and the benchmark's cpu_baseline leg run (the
serial build would take minutes there).  Its depth prepass is different code (compare-and-swap minima without the
early depth test) and its sums are atomic additions in whatever order the threads arrive, so it is held here to the
serial build, which tests/test_oracle_math.py and tests/test_oracle_render.py pin: packed depth|index, depth, weight,
mask and the counters bit for bit; the blended descriptors within 1e-5 relative; the gradients within 1e-4 relative /
1e-6 absolute (the orders of the float additions differ).
"""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402
from helpers import assert_close  # noqa: E402


def big_scene():
    """240 k points of the config-3 scene with distortion, a crop window, the LOD radius test, a dropout mask and two
    views of one frame: every branch of the three loops runs with many threads on the same pixels."""
    from adop_amd import scenes

    hs = scenes.config3(n=240_000, w=320, h=180, levels=4, channels=4, seed=5)
    hs.intrinsics[0, 5:] = [0.05, -0.02, 0.003, 0.01, 0.002, -0.001, 0.001, -0.0015]
    hs.position[:, 3] = scenes.rng(9).uniform(0.001, 0.02, hs.num_points).astype(np.float32)
    hs.params.drop_out_points_by_radius = 1
    hs.params.output_background_mask = 1
    hs.views = [scenes.make_view(320, 180), scenes.make_view(320, 180, crop=(1.5, 1.5, -90.0, -40.0, 0.0))]
    hs.dropout = scenes.bernoulli_mask(3, 2, hs.num_points, 0.25)
    return hs


def scenes_under_test():
    out = dict(make_golden.golden_scenes())
    out["config3_240k_320x180_two_views"] = big_scene()
    return out


@pytest.mark.parametrize("name", sorted(scenes_under_test()))
def test_openmp_build_equals_serial_build(oracle_mod, name):
    import ctypes

    from adop_amd import scenes

    oracle = oracle_mod
    lib = oracle.lib(True)
    if lib.oracle_num_threads() < 4:  # e.g. OMP_NUM_THREADS=1 in the environment: the comparison needs real threads
        ctypes.CDLL("libgomp.so.1").omp_set_num_threads(8)
    assert lib.oracle_num_threads() >= 4, "the OpenMP build must run on several threads here"
    hs = scenes_under_test()[name]
    a = oracle.forward(hs)
    b = oracle.forward(hs, omp=True)
    for l in range(hs.num_layers):
        assert np.array_equal(a.depth_index[l], b.depth_index[l]), (l, "packed depth|index")
        assert np.array_equal(a.depth[l].view(np.uint32), b.depth[l].view(np.uint32)), (l, "depth")
        assert np.array_equal(a.weight[l], b.weight[l]), (l, "weight")
        assert np.array_equal(a.mask[l], b.mask[l]), (l, "mask")
        assert_close(b.out[l], a.out[l], 1e-5, 1e-7, f"out {l}")
        assert a.stats.visible[l] == b.stats.visible[l] and a.stats.accepted[l] == b.stats.accepted[l]
    gout = scenes.upstream_grads(hs, 77)
    # both backward passes on the serial forward state, as the reference's backward runs on its saved variables
    ga = oracle.backward(hs, a, gout)
    gb = oracle.backward(hs, a, gout, omp=True)
    assert_close(gb.grad_texture, ga.grad_texture, 1e-4, 1e-6, "grad_texture")
    assert_close(gb.grad_background, ga.grad_background, 1e-4, 1e-6, "grad_background")
    assert np.array_equal(ga.grad_points_count, gb.grad_points_count)
    assert np.array_equal(ga.grad_points, gb.grad_points), "one owner per point: no reordering"
    assert np.array_equal(ga.grad_pose_count, gb.grad_pose_count)
    assert np.array_equal(ga.grad_intrinsics_count, gb.grad_intrinsics_count)
    assert_close(gb.grad_pose, ga.grad_pose, 1e-4, 1e-6, "grad_pose")  # f64 partial sums per thread
    assert_close(gb.grad_intrinsics, ga.grad_intrinsics, 1e-4, 1e-6, "grad_intrinsics")
    for l in range(hs.num_layers):
        assert ga.stats.spatial[l] == gb.stats.spatial[l]
