"""Random sweep over the preprocessing kernels: every seed draws a cloud (size, shape, exact duplicates, stray points,
degenerate axes), a neighbour rank and radii, and the device results are compared with the CPU checker: neighbour
distances and Morton codes bit for bit, the close-point filter equal to the sequential sweep."""
import os

import numpy as np
import pytest

from helpers import announce

pytestmark = pytest.mark.gpu


def random_cloud(seed):
    g = np.random.default_rng(9000 + seed)
    n = int(g.choice([9, 10, 33, 64, 65, 300, 1000, 2049, 4000, 7000]))
    kind = str(g.choice(["uniform", "gauss", "plane", "line", "clusters", "shell"]))
    if kind == "uniform":
        xyz = g.random((n, 3)) * g.choice([1.0, 1e-3, 1e3])
    elif kind == "gauss":
        xyz = g.standard_normal((n, 3)) * [1.0, 0.3, 2.0]
    elif kind == "plane":
        xyz = g.random((n, 3)) * [1.0, 1.0, 0.0] + [0.0, 0.0, 0.5]  # one axis without extent
    elif kind == "line":
        xyz = np.outer(g.random(n), [1.0, 2.0, -1.0])
    elif kind == "clusters":
        xyz = g.standard_normal((n, 3)) * 0.01 + g.integers(0, 4, (n, 1)) * [3.0, 0.0, 1.0]
    else:
        d = g.standard_normal((n, 3))
        xyz = d / np.linalg.norm(d, axis=1, keepdims=True)
    xyz = xyz.astype(np.float32)
    what = f"{kind} n={n}"
    if g.random() < 0.4:  # exact duplicates
        m = max(1, n // 10)
        xyz[g.choice(n, m, replace=False)] = xyz[g.choice(n, m)]
        what += " +duplicates"
    if g.random() < 0.4:  # stray points far outside
        m = int(g.integers(1, 4))
        xyz[g.choice(n, m, replace=False)] = (g.standard_normal((m, 3)) * 1e4).astype(np.float32)
        what += f" +{m} strays"
    p = np.zeros((n, 4), np.float32)
    p[:, :3] = xyz
    rank = int(g.integers(1, 9))
    return g, p, rank, what


# (ADOP_PREPROCESS_SWEEP_SEEDS="first:count" draws other clouds than the 60 of a default run)
_first, _count = (int(x) for x in os.environ.get("ADOP_PREPROCESS_SWEEP_SEEDS", "0:60").split(":"))


@pytest.mark.parametrize("seed", range(_first, _first + _count))
def test_random_cloud(seed):
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess

    g, p, rank, what = random_cloud(seed)
    announce(f"seed {seed}: {what} rank={rank}")
    dev = torch.from_numpy(p).cuda()
    want = op.knn_distance(p, rank)
    got = preprocess.KNearestNeighbourDistance(dev, rank).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (what, rank, np.abs(got - want).max())
    codes = preprocess.MortonCodes(dev).cpu().numpy().view(np.uint64)
    assert np.array_equal(codes, op.morton_codes(p)), what
    # close points: radii around the typical neighbour distance, some of them zero
    scale = float(np.median(want)) if np.median(want) > 0 else 1.0
    radius = (g.uniform(0.0, 3.0, len(p)) * scale).astype(np.float32)
    radius[g.random(len(p)) < 0.1] = 0.0
    cam = torch.from_numpy((1.0 / np.maximum(radius, np.float32(1e-30))).astype(np.float32)).cuda()
    used = (1.0 / cam).float().cpu().numpy()
    keep = preprocess.RemoveClosePoints(dev, cam, dis_th=1.0).cpu().numpy()
    assert np.array_equal(keep, op.remove_close_points(p, used)), what


@pytest.mark.parametrize("seed", range(20))
def test_random_cameras(seed):
    """Camera distance for random rigs: 1-70 frames at random places around and inside the cloud, 1-3 camera models
    with random intrinsics and distortion, random image sizes."""
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess, scene_io, scenes

    g = np.random.default_rng(500 + seed)
    n = int(g.choice([1, 100, 5000, 20000]))
    frames = int(g.choice([1, 2, 31, 32, 33, 70]))
    cams = int(g.integers(1, 4))
    p = np.zeros((n, 4), np.float32)
    p[:, :3] = g.standard_normal((n, 3)) * g.choice([0.3, 1.0, 3.0])
    views = np.stack([scenes.look_at_view(g.standard_normal(3) * g.choice([0.5, 2.0, 4.0]), g.standard_normal(3) * 0.3)
                      for _ in range(frames)])
    poses = np.stack([scene_io.invert_pose(v[:7]) for v in views])
    K = np.stack([scenes.pinhole_row(g.uniform(100, 400), g.uniform(100, 400), g.uniform(100, 200), g.uniform(80, 150),
                                     g.uniform(-0.5, 0.5), g.uniform(-1, 1, 8) * [0.1, 0.05, 0.01, 0.05, 0.02, 0.005, 0.003, 0.003])
                  for _ in range(cams)])
    fr = [(int(g.integers(64, 400)), int(g.integers(64, 300)), f, int(g.integers(0, cams))) for f in range(frames)]
    announce(f"seed {seed}: camera distance n={n} frames={frames} cameras={cams}")
    want = op.point_distance_to_camera(p, poses, K, fr)
    got = preprocess.PointDistanceToCamera(torch.from_numpy(p).cuda(), torch.from_numpy(views).cuda(),
                                           torch.from_numpy(K).cuda(),
                                           [scenes.make_view(w, h, image_index=f, camera_index=c) for w, h, f, c in fr])
    got = got.cpu().numpy()
    # a point whose projection lies within rounding of the image border may be seen by one side only: such points
    # flip between a camera's distance and the next candidate; all others agree to 1e-5
    close = np.abs(got - want) <= 1e-5 * np.abs(want)
    assert close.mean() >= 0.999, (close.mean(), n)
