"""Pins of the preprocessing checker (oracle/preprocess.py): the brute-force neighbour search against scipy's kd-tree,
the Morton key against hand-computed codes and the properties a Morton key must have, the block sort against sorted()."""
import numpy as np
import pytest

import oracle.preprocess as op


def _clouds():
    g = np.random.default_rng(1)
    uniform = g.random((2500, 4)).astype(np.float32)
    plane = g.random((2500, 4)).astype(np.float32)
    plane[:, 2] = 0.25 + 1e-3 * plane[:, 2]
    clustered = (g.standard_normal((2500, 4)) * 0.01 + g.integers(0, 5, (2500, 1))).astype(np.float32)
    dup = uniform.copy()
    dup[100:140] = dup[:40]  # exact duplicates: distance 0 neighbours
    return {"uniform": uniform, "plane": plane, "clustered": clustered, "duplicates": dup}


@pytest.mark.parametrize("name", ["uniform", "plane", "clustered", "duplicates"])
@pytest.mark.parametrize("rank", [1, 4, 8])
def test_knn_distance_matches_kdtree(name, rank):
    from scipy.spatial import cKDTree

    p = _clouds()[name]
    got = op.knn_distance(p, rank)
    xyz = p[:, :3].astype(np.float64)
    want = cKDTree(xyz).query(xyz, k=rank + 1)[0][:, rank]  # the point itself is the first hit, as in the reference
    assert np.allclose(got, want, rtol=2e-6, atol=1e-9)


def test_knn_distance_closed_forms():
    # a regular lattice with spacing 1: 6 neighbours at 1, 12 at sqrt(2), 8 at sqrt(3); interior points only
    g = np.stack(np.meshgrid(*[np.arange(7)] * 3, indexing="ij"), -1).reshape(-1, 3).astype(np.float32)
    p = np.concatenate([g, np.zeros((len(g), 1), np.float32)], 1)
    inner = np.all((g >= 2) & (g <= 4), axis=1)
    assert np.all(op.knn_distance(p, 1)[inner] == 1.0)
    assert np.all(op.knn_distance(p, 6)[inner] == 1.0)
    assert np.all(op.knn_distance(p, 7)[inner] == np.float32(np.sqrt(np.float32(2))))
    # four points on a line at 0, 1, 3, 7: ranks 1..3 of the point at 0
    line = np.zeros((4, 4), np.float32)
    line[:, 0] = [0, 1, 3, 7]
    assert [float(op.knn_distance(line, r)[0]) for r in (1, 2, 3)] == [1.0, 3.0, 7.0]


def test_morton_codes_known_answers_and_properties():
    m = 2097151  # 2^21 - 1 steps per axis
    p = np.zeros((6, 4), np.float32)
    p[1, :3] = m  # the far corner makes the quantisation step exactly 1
    p[2, 0] = 1
    p[3, 1] = 1
    p[4, 2] = 1
    p[5, :3] = [5, 3, 6]  # x=101b y=011b z=110b -> bits (z y x) per level, from the top: 101 110 011 = 0b101110011
    c = op.morton_codes(p)
    assert int(c[0]) == 0 and int(c[1]) == (1 << 63) - 1
    assert [int(c[2]), int(c[3]), int(c[4])] == [1, 2, 4]
    assert int(c[5]) == 0b101110011
    # moving along one axis never decreases the code's bits of that axis: the code is monotone along every axis
    g = np.random.default_rng(2)
    q = g.random((500, 4)).astype(np.float32)
    q[0, :3], q[1, :3] = 0, 1
    for ax in range(3):
        line = np.repeat(q[2:3], 400, 0)
        line[:, ax] = np.sort(g.random(400).astype(np.float32))
        line = np.concatenate([q[:2], line])
        cc = op.morton_codes(line)[2:]
        assert np.all(np.diff(cc.astype(np.float64)) >= 0)
    # two points of one octant of the box share the top three bits
    c = op.morton_codes(q)
    oct_ = (q[:, 0] >= 0.5).astype(np.uint64) | ((q[:, 1] >= 0.5).astype(np.uint64) << np.uint64(1)) | \
           ((q[:, 2] >= 0.5).astype(np.uint64) << np.uint64(2))
    inside = np.all(np.abs(q[:, :3] - 0.5) > 1e-3, axis=1)
    assert np.all((c >> np.uint64(60))[inside] == oct_[inside])


def test_sort_blocks():
    g = np.random.default_rng(3)
    r = g.random(1000).astype(np.float32)
    r[10] = r[20]  # a tie keeps its order
    order = op.sort_blocks(r, 256)
    assert sorted(order.tolist()) == list(range(1000))
    for b in range(3):
        blk = order[b * 256:(b + 1) * 256]
        assert np.all((blk >= b * 256) & (blk < (b + 1) * 256))
        assert blk.tolist() == sorted(range(b * 256, (b + 1) * 256), key=lambda i: (r[i], i))
    assert order[768:].tolist() == list(range(768, 1000))  # the last, shorter block is left alone
