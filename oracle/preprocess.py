"""CPU checker of the point-cloud preprocessing (test infrastructure only: imported by tests/, never by adop_amd/).

Restates, in numpy, what SceneData::ComputeRadius asks of its kd-tree (data/SceneData.cpp:441-463: the n + 1 nearest
points of every point, itself included, and the distance to the last of them) as a brute-force search with the same
fp32 arithmetic as the HIP kernel, and the Morton key of PointCloud::ReorderMorton64 (SceneData.cpp:101; saiga's own
source is not part of the reference tree, so the quantisation - 21 bits per axis of the position inside the bounding
box, x in the lowest bit - is defined here, not verified against saiga: parity unpinned for the key itself; the
properties a Morton key must have are pinned by tests/test_preprocess_oracle.py).  The distance search is pinned
against scipy.spatial.cKDTree.
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
