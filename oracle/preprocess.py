"""CPU checker of the point-cloud preprocessing (test infrastructure only: imported by tests/, never by adop_amd/).

Restates, in numpy, what SceneData::ComputeRadius asks of its kd-tree (data/SceneData.cpp:441-463: the n + 1 nearest
points of every point, itself included, and the distance to the last of them) as a brute-force search with the same
fp32 arithmetic as the HIP kernel, and the Morton key of PointCloud::ReorderMorton64 (SceneData.cpp:101; saiga's own
source is not part of the reference tree, so the quantisation - 21 bits per axis of the position inside the bounding
box, x in the lowest bit - is defined here, not verified against saiga: parity unpinned for the key itself; the
properties a Morton key must have are pinned by tests/test_preprocess_oracle.py).  The distance search is pinned
against scipy.spatial.cKDTree.

Also restated: SceneData::PointDistanceToCamera (SceneData.cpp:645-669, with FrameData::Project3 :26-34), pinned by
hand-computed cases (in view, behind the camera, outside the image, pushed outside by the distortion, two cameras),
and the sweep of SceneData::RemoveClosePoints (:598-642), pinned by the two properties that determine its result
(every erased point has an earlier kept point within its radius, no kept point has one), checked with a kd-tree.
saiga's KDTree::RadiusSearch is not part of the reference tree: whether a point at exactly the radius counts is
defined here (it does not: d2 < r2): parity unpinned for that boundary.
"""
import numpy as np


def knn_distance(position, rank=4, chunk=512):
    """[N] f32: distance to the rank-th nearest other point, sqrt((dx*dx + dy*dy) + dz*dz) in fp32."""
    xyz = np.ascontiguousarray(position[:, :3], dtype=np.float32)
    n = len(xyz)
    assert n > rank
    out = np.empty(n, np.float32)
    for s in range(0, n, chunk):
        q = xyz[s:s + chunk]
        d = q[:, None, :] - xyz[None, :, :]
        d2 = (d[..., 0] * d[..., 0] + d[..., 1] * d[..., 1]) + d[..., 2] * d[..., 2]
        out[s:s + chunk] = np.sqrt(np.partition(d2, rank, axis=1)[:, rank])  # index 0 is the point itself
    return out


def _spread21(v):
    v = v.astype(np.uint64) & np.uint64(0x1FFFFF)
    v = (v | (v << np.uint64(32))) & np.uint64(0x1F00000000FFFF)
    v = (v | (v << np.uint64(16))) & np.uint64(0x1F0000FF0000FF)
    v = (v | (v << np.uint64(8))) & np.uint64(0x100F00F00F00F00F)
    v = (v | (v << np.uint64(4))) & np.uint64(0x10C30C30C30C30C3)
    v = (v | (v << np.uint64(2))) & np.uint64(0x1249249249249249)
    return v


def morton_codes(position):
    """[N] u64: 21 bits per axis, fp32 arithmetic: q = clamp((p - min) * (2097151 / (max - min)), 0, 2097151)."""
    xyz = np.ascontiguousarray(position[:, :3], dtype=np.float32)
    mn, mx = xyz.min(0), xyz.max(0)
    ext = (mx - mn).astype(np.float32)
    scale = np.where(ext > 0, np.float32(2097151.0) / np.where(ext > 0, ext, 1).astype(np.float32), np.float32(0)).astype(np.float32)
    q = np.clip(((xyz - mn).astype(np.float32) * scale).astype(np.float32), np.float32(0), np.float32(2097151.0))
    q = q.astype(np.uint64)
    return _spread21(q[:, 0]) | (_spread21(q[:, 1]) << np.uint64(1)) | (_spread21(q[:, 2]) << np.uint64(2))


def sort_blocks(radius, block_size=256):
    """Permutation of SortBlocksByRadius (SceneData.cpp:671-684), ties in their original order."""
    n = len(radius)
    nb = n // block_size
    order = np.arange(n)
    for b in range(nb):
        sl = slice(b * block_size, (b + 1) * block_size)
        order[sl] = b * block_size + np.argsort(radius[sl], kind="stable")
    return order


def _quat_rotate(q, v):
    """Eigen's quaternion * vector in fp32: v + w*t + u x t with t = 2 (u x v)."""
    u = q[:3].astype(np.float32)
    w = np.float32(q[3])
    t = (np.float32(2) * np.cross(u[None, :], v)).astype(np.float32)
    return (v + w * t + np.cross(u[None, :], t)).astype(np.float32)


def _distort(x, y, d):
    """distortNormalizedPoint: OpenCV rational + tangential model (k1..k6, p1, p2), fp32."""
    k1, k2, k3, k4, k5, k6, p1, p2 = [np.float32(c) for c in d]
    one, two = np.float32(1), np.float32(2)
    x2, y2 = x * x, y * y
    r2 = x2 + y2
    xy2 = two * x * y
    r4 = r2 * r2
    r6 = r2 * r4
    rad = (one + k1 * r2 + k2 * r4 + k3 * r6) / (one + k4 * r2 + k5 * r4 + k6 * r6)
    return x * rad + (p1 * xy2 + p2 * (r2 + two * x2)), y * rad + (p1 * (r2 + two * y2) + p2 * xy2)


def point_distance_to_camera(position, poses, intrinsics, frames):
    """[N] f32, SceneData::PointDistanceToCamera (SceneData.cpp:645-669).  poses [F,7] f64 camera -> world
    (FrameData::pose), intrinsics [K,13] f32, frames: (w, h, pose index, camera index) per frame."""
    xyz = np.ascontiguousarray(position[:, :3], dtype=np.float32)
    best = np.full(len(xyz), np.float32(105235545.0), np.float32)
    with np.errstate(all="ignore"):
        for w, h, fi, ci in frames:
            pose = np.asarray(poses[fi], np.float64)
            q = pose[:4] / np.linalg.norm(pose[:4])
            qi = np.array([-q[0], -q[1], -q[2], q[3]])
            # t' = -(q^-1 * t) in f64, then the inverse pose is cast to float (:28)
            u = qi[:3]
            tt = 2.0 * np.cross(u, pose[4:7])
            ti = -(pose[4:7] + qi[3] * tt + np.cross(u, tt))
            p = _quat_rotate(qi.astype(np.float32), xyz) + ti.astype(np.float32)[None, :]
            z = p[:, 2]
            dx, dy = _distort(p[:, 0] / z, p[:, 1] / z, intrinsics[ci, 5:13])
            K = intrinsics[ci, :5].astype(np.float32)
            ix = (K[0] * dx + K[4] * dy) + K[2]
            iy = K[1] * dy + K[3]
            ok = (z > 0) & (ix >= 0) & (iy >= 0) & (ix < np.float32(w)) & (iy < np.float32(h))
            d = xyz - pose[4:7].astype(np.float32)[None, :]
            dis = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
            best = np.where(ok & (dis < best), dis, best).astype(np.float32)
    return np.sqrt(best)


def remove_close_points(position, radius):
    """[N] bool keep mask of the sweep of SceneData::RemoveClosePoints (SceneData.cpp:617-637): in index order a point
    is erased when a point kept before lies within its radius (d2 < r2, fp32, the kernel's summation order)."""
    xyz = np.ascontiguousarray(position[:, :3], dtype=np.float32)
    radius = np.asarray(radius, np.float32)
    keep = np.zeros(len(xyz), bool)
    for i in range(len(xyz)):
        d = xyz[i][None, :] - xyz[:i]
        d2 = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
        keep[i] = not np.any(keep[:i] & (d2 < radius[i] * radius[i]))
    return keep
