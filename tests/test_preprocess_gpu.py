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
