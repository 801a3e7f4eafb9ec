"""The preprocessing kernels (adop_knn_distance, adop_morton_codes) and the Python mirror of SceneData's initial
processing against the CPU checker: distances and codes bit-exact."""
import numpy as np
import pytest

from helpers import announce

pytestmark = pytest.mark.gpu


def _clouds():
    g = np.random.default_rng(11)
    n = 8000
    uniform = g.random((n, 4)).astype(np.float32)
    plane = g.random((n, 4)).astype(np.float32)
    plane[:, 2] = 0.25 + 1e-3 * plane[:, 2]
    slab = (g.random((n, 4)) * [100.0, 1.0, 0.01, 1.0] - [50.0, 0.0, 0.0, 0.0]).astype(np.float32)
    clustered = (g.standard_normal((n, 4)) * 0.01 + g.integers(0, 5, (n, 1))).astype(np.float32)
    dup = uniform.copy()
    dup[1000:1400] = dup[:400]
    tiny = g.random((9, 4)).astype(np.float32)
    same = np.ones((100, 4), np.float32)
    return {"uniform": uniform, "plane": plane, "slab": slab, "clustered": clustered, "duplicates": dup, "tiny": tiny,
            "coincident": same}


@pytest.mark.parametrize("name", ["uniform", "plane", "slab", "clustered", "duplicates", "tiny", "coincident"])
def test_knn_distance_bit_exact(name):
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess

    p = _clouds()[name]
    for rank in ((1, 4, 8) if name in ("uniform", "tiny", "coincident") else (4,)):
        announce(f"knn distance, cloud={name} N={len(p)} rank={rank}")
        want = op.knn_distance(p, rank)
        got = preprocess.KNearestNeighbourDistance(torch.from_numpy(p).cuda(), rank).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (name, rank, np.abs(got - want).max())


def test_knn_distance_rejects_bad_arguments():
    import torch
    from adop_amd import preprocess

    p = torch.rand(4, 4, device="cuda")
    with pytest.raises(RuntimeError):
        preprocess.KNearestNeighbourDistance(p, 4)  # needs more than `rank` points
    with pytest.raises(RuntimeError):
        preprocess.KNearestNeighbourDistance(torch.rand(100, 4, device="cuda"), 9)


def test_morton_codes_bit_exact():
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess

    for name, p in _clouds().items():
        announce(f"morton codes, cloud={name}")
        want = op.morton_codes(p)
        got = preprocess.MortonCodes(torch.from_numpy(p).cuda()).cpu().numpy().view(np.uint64)
        assert np.array_equal(got, want), name


def test_preprocess_point_cloud():
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess

    announce("PreprocessPointCloud: 12 288 points + 77 (a last partial block)")
    g = np.random.default_rng(5)
    p = g.random((12365, 4)).astype(np.float32)
    p[:, 3] = 0
    nrm = np.arange(12365, dtype=np.int32)
    pos, normal, data, order = preprocess.PreprocessPointCloud(torch.from_numpy(p).cuda(), torch.from_numpy(nrm).cuda(),
                                                               seed=3)
    pos, normal, data, order = pos.cpu().numpy(), normal.cpu().numpy(), data.cpu().numpy(), order.cpu().numpy()
    assert sorted(order.tolist()) == list(range(12365))  # a permutation ...
    assert np.array_equal(pos[:, :3], p[order, :3]) and np.array_equal(normal, nrm[order])  # ... applied to everything
    assert np.array_equal(data[:, 0].view(np.uint32), op.knn_distance(pos, 4).view(np.uint32))
    assert np.all(data[:, 2] >= 1.0) and np.array_equal(data[:, 3], data[:, 0] * data[:, 2])
    assert np.array_equal(pos[:, 3], data[:, 3])  # the rasterizer's LOD radius
    nb = 12365 // 256
    r = pos[: nb * 256, 3].reshape(nb, 256)
    assert np.all(np.diff(r, axis=1) >= 0)  # every block ascends in radius
    # the blocks are Morton blocks: the points of a block are 256 consecutive points of the Morton order
    codes = op.morton_codes(p)
    ranks = np.empty(12365, np.int64)
    ranks[np.argsort(codes, kind="stable")] = np.arange(12365)
    blk = ranks[order[: nb * 256]].reshape(nb, 256)
    assert np.all(blk.max(1) - blk.min(1) == 255)
    assert len(set((blk.min(1) // 256).tolist())) == nb and not np.all(np.diff(blk.min(1)) > 0)  # shuffled


def test_knn_distance_two_million_points_against_kdtree_sample():
    import torch
    from scipy.spatial import cKDTree
    from adop_amd import preprocess

    announce("knn distance, 2 M points (surface-like: points on random patches), sample of 3 000 against scipy")
    g = np.random.default_rng(9)
    n = 2_000_000
    c = g.uniform(-3, 3, (400, 3))
    a = g.standard_normal((400, 3))
    a /= np.linalg.norm(a, axis=1, keepdims=True)
    b = np.cross(a, g.standard_normal((400, 3)))
    b /= np.linalg.norm(b, axis=1, keepdims=True)
    pid = g.integers(0, 400, n)
    xyz = (c[pid] + g.uniform(-0.3, 0.3, (n, 1)) * a[pid] + g.uniform(-0.3, 0.3, (n, 1)) * b[pid]).astype(np.float32)
    p = np.concatenate([xyz, np.zeros((n, 1), np.float32)], 1)
    got = preprocess.KNearestNeighbourDistance(torch.from_numpy(p).cuda(), 4).cpu().numpy()
    tree = cKDTree(xyz.astype(np.float64))
    sample = g.integers(0, n, 3000)
    want = tree.query(xyz[sample].astype(np.float64), k=5)[0][:, 4]
    assert np.allclose(got[sample], want, rtol=2e-6, atol=1e-9)


def _orbit_scene(n, frames, seed):
    """A Gaussian cloud and `frames` cameras on a sphere looking at it, two camera models (one with distortion)."""
    from adop_amd import scene_io, scenes

    g = np.random.default_rng(seed)
    p = np.zeros((n, 4), np.float32)
    p[:, :3] = g.standard_normal((n, 3)) * 0.7
    views = np.stack([scenes.look_at_view(g.uniform(1.5, 3.0) * d / np.linalg.norm(d)) for d in g.standard_normal((frames, 3))])
    poses = np.stack([scene_io.invert_pose(v[:7]) for v in views])  # camera -> world, as in poses.txt
    K = np.stack([scenes.pinhole_row(300, 300, 160, 120), scenes.pinhole_row(250, 260, 150, 110, 0.5,
                 [0.1, -0.05, 0.01, 0.02, 0.0, 0.0, 0.002, -0.001])])
    fr = [(320, 240, f, f % 2) for f in range(frames)]
    return p, views, poses, K, fr


def test_point_distance_to_camera():
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess, scenes

    p, views, poses, K, fr = _orbit_scene(20000, 37, 1)  # more frames than one chunk of view constants
    announce("camera distance: N=20000, 37 frames, 2 cameras")
    want = op.point_distance_to_camera(p, poses, K, fr)
    got = preprocess.PointDistanceToCamera(torch.from_numpy(p).cuda(), torch.from_numpy(views).cuda(),
                                           torch.from_numpy(K).cuda(),
                                           [scenes.make_view(w, h, image_index=f, camera_index=c) for w, h, f, c in fr])
    got = got.cpu().numpy()
    seen = want < 1.0e4
    assert seen.mean() > 0.5 and np.array_equal(seen, got < 1.0e4)
    # the reference measures |p - c| in world space, the kernel |V p| in camera space: equal to fp32 rounding
    np.testing.assert_allclose(got, want, rtol=1e-5)
    one = preprocess.PointDistanceToCamera(torch.from_numpy(p).cuda(), torch.from_numpy(views).cuda(),
                                           torch.from_numpy(K).cuda(), [scenes.make_view(320, 240, image_index=3)])
    want1 = op.point_distance_to_camera(p, poses, K, [(320, 240, 3, 0)])
    assert 0.05 < (want1 < 1.0e4).mean() < 0.95  # one camera leaves points unseen: they keep the start value
    np.testing.assert_allclose(one.cpu().numpy(), want1, rtol=1e-5)
    with pytest.raises(RuntimeError):
        preprocess.PointDistanceToCamera(torch.from_numpy(p).cuda(), torch.from_numpy(views).cuda(),
                                         torch.from_numpy(K).cuda(), [scenes.make_view(320, 240, image_index=37)])


@pytest.mark.parametrize("name", ["uniform", "plane", "duplicates", "coincident", "line"])
def test_remove_close_points_equals_the_sequential_sweep(name):
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess

    g = np.random.default_rng(21)
    if name == "line":
        # every point within reach of its predecessor: one chain of dependencies through the whole cloud
        p = np.zeros((700, 4), np.float32)
        p[:, 0] = np.arange(700) * 0.01
        radius = np.full(700, 0.015, np.float32)
    else:
        p = _clouds()[name][:6000]
        radius = g.uniform(0.0, 0.06, len(p)).astype(np.float32)
    announce(f"close points, cloud={name} N={len(p)}")
    want = op.remove_close_points(p, radius)
    # RemoveClosePoints takes dis_th / camera distance as the radius: camera distance 1 / radius, dis_th 1
    cam = torch.from_numpy(1.0 / np.maximum(radius, 1e-30)).cuda()
    got = preprocess.RemoveClosePoints(torch.from_numpy(p).cuda(), cam, dis_th=1.0).cpu().numpy()
    radius_used = (1.0 / cam).float().cpu().numpy()
    if not np.array_equal(radius_used, radius):
        want = op.remove_close_points(p, radius_used)
    assert np.array_equal(got, want), (name, int((got != want).sum()))
    if name == "line":
        assert np.array_equal(want, np.arange(700) % 2 == 0)
    if name == "coincident":
        assert want.sum() == 1


def test_remove_lonely_points():
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess

    g = np.random.default_rng(4)
    p = np.zeros((9000, 4), np.float32)
    p[:8900, :3] = g.random((8900, 3)) * 0.5
    p[8900:, :3] = g.random((100, 3)) * 4 + 1  # stragglers
    cam = g.uniform(1.0, 3.0, 9000).astype(np.float32)
    announce("lonely points: N=9000")
    keep = preprocess.RemoveLonelyPoints(torch.from_numpy(p).cuda(), torch.from_numpy(cam).cuda(), 5, 0.02).cpu().numpy()
    want = ~(op.knn_distance(p, 5) / cam > np.float32(0.02))
    assert np.array_equal(keep, want) and keep[:8900].mean() > 0.5 and keep[8900:].mean() < 0.1


def test_filter_point_cloud_composes_the_filters():
    import torch
    import oracle.preprocess as op
    from adop_amd import preprocess, scenes

    p, views, poses, K, fr = _orbit_scene(6000, 5, 8)
    p[3000:3300] = p[:300] + np.float32(1e-6)  # near-duplicates for the close-point filter
    announce("FilterPointCloud: N=6000, 5 frames")
    got = preprocess.FilterPointCloud(torch.from_numpy(p).cuda(), torch.from_numpy(views).cuda(), torch.from_numpy(K).cuda(),
                                      [scenes.make_view(w, h, image_index=f, camera_index=c) for w, h, f, c in fr],
                                      lonely=(5, 0.1)).cpu().numpy()
    cam = preprocess.PointDistanceToCamera(torch.from_numpy(p).cuda(), torch.from_numpy(views).cuda(),
                                           torch.from_numpy(K).cuda(),
                                           [scenes.make_view(w, h, image_index=f, camera_index=c) for w, h, f, c in fr]).cpu().numpy()
    ids = np.arange(6000)
    keep = ~(op.knn_distance(p, 5) / cam > np.float32(0.1))
    q, cam2, ids = p[keep], cam[keep], ids[keep]
    keep2 = op.remove_close_points(q, (np.float32(0.00005) / cam2).astype(np.float32))
    assert np.array_equal(got, ids[keep2])
    assert 0 < (~keep).sum() < 3000 and 200 < (~keep2).sum() <= 320


def test_knn_distance_with_far_outliers():
    """Reconstructed clouds carry stray points far outside the scene.  The search grid is laid over the bulk of the
    cloud (percentiles of a sample), the strays go to its boundary cells, and the result stays exact (and fast)."""
    import time
    import torch
    from scipy.spatial import cKDTree
    from adop_amd import preprocess

    g = np.random.default_rng(31)
    n = 1_000_000
    p = np.zeros((n, 4), np.float32)
    p[:, :3] = g.random((n, 3))
    stray = g.choice(n, 40, replace=False)
    p[stray, :3] = g.standard_normal((40, 3)) * [3000.0, 100.0, 1.0e4]
    announce("knn distance, 1 M points in the unit cube + 40 strays up to 1e4 away")
    dev = torch.from_numpy(p).cuda()
    preprocess.KNearestNeighbourDistance(dev, 4)  # first call: library load
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    got = preprocess.KNearestNeighbourDistance(dev, 4).cpu().numpy()
    seconds = time.perf_counter() - t0
    tree = cKDTree(p[:, :3].astype(np.float64))
    check = np.concatenate([stray, g.integers(0, n, 3000)])
    want = tree.query(p[check, :3].astype(np.float64), k=5)[0][:, 4]
    assert np.allclose(got[check], want, rtol=2e-6, atol=1e-9)
    print("seconds", seconds)
    assert seconds < 1.0, seconds  # (~0.01 s; with the grid over the bounding box, all in one cell: 2.6 s)
