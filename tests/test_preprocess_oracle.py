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


SENTINEL = np.sqrt(np.float32(105235545.0))


def test_camera_distance_hand_computed_cases():
    identity = [0, 0, 0, 1, 0, 0, 0]
    K = np.zeros((2, 13), np.float32)
    K[0, :5] = [100, 100, 50, 40, 0]  # 100 x 80 image, centre (50, 40)
    K[1, :5] = [100, 100, 50, 40, 0]
    K[1, 5] = 5.0  # k1: x' = x (1 + 5 r^2)
    pts = np.float32([[0, 0, 5, 0],        # on the axis: 5
                      [0, 0, -5, 0],       # behind the camera
                      [3, 0, 5, 0],        # x/z = 0.6 -> pixel 110: outside
                      [2.4, 0, 5, 0],      # x/z = 0.48 -> pixel 98: inside, distance sqrt(2.4^2 + 25)
                      [1.5, 0, 5, 0],      # x/z = 0.3 -> 80 undistorted; 0.3 (1 + 0.45) = 0.435 -> 93.5 with k1
                      [2.0, 0, 5, 0]])     # x/z = 0.4 -> 90 undistorted; 0.4 (1 + 0.8) = 0.72 -> 122 with k1: outside
    d0 = op.point_distance_to_camera(pts, [identity], K, [(100, 80, 0, 0)])
    want0 = np.float32([5, SENTINEL, SENTINEL, np.sqrt(2.4 ** 2 + 25), np.sqrt(1.5 ** 2 + 25), np.sqrt(29.0)])
    np.testing.assert_allclose(d0, want0, rtol=1e-6)
    d1 = op.point_distance_to_camera(pts, [identity], K, [(100, 80, 0, 1)])
    assert d1[4] == d0[4] and d1[5] == SENTINEL and d1[3] == SENTINEL
    # a second camera at (10, 0, 5) looking down -x sees the points from the side: the nearer camera wins
    s = np.sqrt(0.5)
    side = [0, -s, 0, s, 10, 0, 5]  # camera -> world: the camera's +z is the world's -x
    both = op.point_distance_to_camera(pts, [identity, side], K, [(100, 80, 0, 0), (100, 80, 1, 0)])
    alone = op.point_distance_to_camera(pts, [identity, side], K, [(100, 80, 1, 0)])
    np.testing.assert_allclose(alone[0], 10, rtol=1e-6)  # (0,0,5) is 10 away on the axis
    assert alone[1] == SENTINEL  # (0,0,-5): 10 in front, 10 to the side: tangent 1 -> 100 pixels off the centre
    np.testing.assert_allclose(both[0], 5, rtol=1e-6)
    np.testing.assert_allclose(both[2], min(7.0, SENTINEL), rtol=1e-6)  # (3,0,5): unseen by the first, 7 from the second


@pytest.mark.parametrize("name", ["uniform", "plane", "duplicates"])
def test_close_point_sweep_has_the_defining_properties(name):
    from scipy.spatial import cKDTree

    g = np.random.default_rng(2)
    p = _clouds()[name]
    radius = g.uniform(0.0, 0.08, len(p)).astype(np.float32)
    keep = op.remove_close_points(p, radius)
    assert 0.2 < keep.mean() < 0.95
    xyz = p[:, :3].astype(np.float64)
    tree = cKDTree(xyz)
    for i in range(len(p)):
        near = [j for j in tree.query_ball_point(xyz[i], float(radius[i]) * (1 + 1e-6) + 1e-12) if j < i and keep[j]]
        # leave pairs at the radius to within rounding to the fp32 sweep
        sure = [j for j in near if np.linalg.norm(xyz[i] - xyz[j]) < float(radius[i]) * (1 - 1e-6)]
        if keep[i]:
            assert not sure, i  # no kept point has an earlier kept point within its radius
        else:
            assert near, i  # every erased point has one
