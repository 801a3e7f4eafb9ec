"""Synthetic scenes for the rasterizer: the five benchmark configurations and small test scenes.

Everything is generated on the host with numpy's Philox generator from a fixed seed, so the CPU checker and
the HIP path see identical bits.  Tensor layouts follow the reference (see ``include/adop_raster.h``):
``position [N,4]`` (x,y,z,radius), ``normal [N]`` (10-bit packed), ``index [N]``, ``texture [C,N]``,
``poses_se3 [F,8]`` world->camera (qx,qy,qz,qw,tx,ty,tz,0), ``intrinsics [K,13]`` or ``[K,5+P]``.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import _capi


def rng(seed):
    return np.random.Generator(np.random.Philox(seed))


# ---------------------------------------------------------------------------------------------------
# small math helpers (host side, float64)
# ---------------------------------------------------------------------------------------------------

def pack_normals(n):
    """3 x 10-bit quantisation of unit normals, x in bits 0..9 (NeuralPointCloudCuda.cpp:31)."""
    n = np.asarray(n, dtype=np.float32)
    q = np.rint((n * np.float32(0.5) + np.float32(0.5)) * np.float32(1023.0)).astype(np.int64)
    q = np.clip(q, 0, 1023)
    return (q[:, 0] | (q[:, 1] << 10) | (q[:, 2] << 20)).astype(np.int32)


def rotation_to_quaternion(R):
    """3x3 rotation -> (x,y,z,w)."""
    t = np.trace(R)
    if t > 0:
        s = np.sqrt(t + 1.0) * 2
        w = 0.25 * s
        x = (R[2, 1] - R[1, 2]) / s
        y = (R[0, 2] - R[2, 0]) / s
        z = (R[1, 0] - R[0, 1]) / s
    elif R[0, 0] > R[1, 1] and R[0, 0] > R[2, 2]:
        s = np.sqrt(1.0 + R[0, 0] - R[1, 1] - R[2, 2]) * 2
        w = (R[2, 1] - R[1, 2]) / s
        x = 0.25 * s
        y = (R[0, 1] + R[1, 0]) / s
        z = (R[0, 2] + R[2, 0]) / s
    elif R[1, 1] > R[2, 2]:
        s = np.sqrt(1.0 + R[1, 1] - R[0, 0] - R[2, 2]) * 2
        w = (R[0, 2] - R[2, 0]) / s
        x = (R[0, 1] + R[1, 0]) / s
        y = 0.25 * s
        z = (R[1, 2] + R[2, 1]) / s
    else:
        s = np.sqrt(1.0 + R[2, 2] - R[0, 0] - R[1, 1]) * 2
        w = (R[1, 0] - R[0, 1]) / s
        x = (R[0, 2] + R[2, 0]) / s
        y = (R[1, 2] + R[2, 1]) / s
        z = 0.25 * s
    q = np.array([x, y, z, w], dtype=np.float64)
    return q / np.linalg.norm(q)


def quaternion_to_rotation(q):
    x, y, z, w = q
    return np.array(
        [
            [1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (x * z + y * w)],
            [2 * (x * y + z * w), 1 - 2 * (x * x + z * z), 2 * (y * z - x * w)],
            [2 * (x * z - y * w), 2 * (y * z + x * w), 1 - 2 * (x * x + y * y)],
        ],
        dtype=np.float64,
    )


def look_at_view(cam_pos, target=(0.0, 0.0, 0.0), world_up=(0.0, 1.0, 0.0)):
    """World->camera SE3 row (8 doubles) of a camera at ``cam_pos`` looking at ``target``.

    Camera frame is the vision convention (x right, y down, z forward).  The stored pose is the inverse of
    the camera->world pose (NeuralStructure.cpp:15-18).
    """
    c = np.asarray(cam_pos, dtype=np.float64)
    z = np.asarray(target, dtype=np.float64) - c
    z /= np.linalg.norm(z)
    down = -np.asarray(world_up, dtype=np.float64)
    x = np.cross(down, z)
    if np.linalg.norm(x) < 1e-9:
        x = np.array([1.0, 0.0, 0.0])
    x /= np.linalg.norm(x)
    y = np.cross(z, x)
    R_cw = np.stack([x, y, z], axis=1)  # camera->world
    R = R_cw.T
    t = -R @ c
    q = rotation_to_quaternion(R)
    return np.array([q[0], q[1], q[2], q[3], t[0], t[1], t[2], 0.0], dtype=np.float64)


def pinhole_row(fx, fy, cx, cy, s=0.0, dist=None):
    row = np.zeros(13, dtype=np.float32)
    row[:5] = [fx, fy, cx, cy, s]
    if dist is not None:
        row[5:] = dist
    return row


# ---------------------------------------------------------------------------------------------------
# host scene container
# ---------------------------------------------------------------------------------------------------

def default_params(**kw):
    """RenderParams defaults of the reference (Settings.h:22-52) with the LOD radius test off."""
    p = _capi.RenderParams()
    p.test_backward_mode = 0
    p.check_normal = 1
    p.ghost_gradients = 0
    p.drop_out_points_by_radius = 0
    p.depth_accept = 0.01
    p.drop_out_radius_threshold = 0.6
    p.dist_cutoff = 1.0e4
    p.distortion_gradient_factor = 0.005
    p.K_gradient_factor = 0.5
    p.output_background_mask = 0
    p.output_background_mask_value = 0.0
    p.normalize_mode = 0
    p.forward_path = 0
    for k, v in kw.items():
        if not hasattr(p, k):
            raise AttributeError(k)
        setattr(p, k, v)
    return p


def make_view(w, h, image_index=0, camera_index=0, model=_capi.CAMERA_PINHOLE_DISTORTION, crop=(1, 1, 0, 0, 0)):
    v = _capi.View()
    v.w, v.h = int(w), int(h)
    v.image_index, v.camera_index = int(image_index), int(camera_index)
    v.camera_model_type = int(model)
    v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy, v.crop_s = [float(c) for c in crop]
    return v


@dataclass
class HostScene:
    """All inputs of one render call as numpy arrays (host memory)."""

    position: np.ndarray  # [N,4] f32
    normal: Optional[np.ndarray]  # [N] i32
    index: np.ndarray  # [N] i32
    texture: np.ndarray  # [C,Ntex] f32 | f16
    background: np.ndarray  # [C] f32
    poses_se3: np.ndarray  # [F,8] f64
    intrinsics: np.ndarray  # [K,cols] f32
    views: List[_capi.View]
    params: _capi.RenderParams
    num_layers: int
    dropout: Optional[np.ndarray] = None  # [B,N] f32 in {0,1}
    env_texture: Optional[np.ndarray] = None  # [C,eh,ew] f32
    name: str = ""
    meta: dict = field(default_factory=dict)

    @property
    def num_points(self):
        return int(self.position.shape[0])

    @property
    def num_channels(self):
        return int(self.texture.shape[0])

    @property
    def batch(self):
        return len(self.views)

    def level_sizes(self):
        w, h = self.views[0].w, self.views[0].h
        out = []
        for _ in range(self.num_layers):
            out.append((w, h))
            w //= 2
            h //= 2
        return out


def bernoulli_mask(seed, B, N, p):
    return (rng(seed).random((B, N), dtype=np.float32) < np.float32(p)).astype(np.float32)


def _unit(v):
    return v / np.linalg.norm(v, axis=1, keepdims=True)


def morton_order(xyz, bits=10):
    """Indices that sort points along a 3-D Morton curve (the reference reorders its clouds this way,
    SceneData.cpp:101, before shuffling 256-point blocks)."""
    mn, mx = xyz.min(0), xyz.max(0)
    q = ((xyz - mn) / np.maximum(mx - mn, 1e-12) * ((1 << bits) - 1)).astype(np.uint64)

    def spread(v):
        v = v & np.uint64(0x3FF)
        v = (v | (v << np.uint64(16))) & np.uint64(0x30000FF)
        v = (v | (v << np.uint64(8))) & np.uint64(0x300F00F)
        v = (v | (v << np.uint64(4))) & np.uint64(0x30C30C3)
        v = (v | (v << np.uint64(2))) & np.uint64(0x9249249)
        return v

    code = spread(q[:, 0]) | (spread(q[:, 1]) << np.uint64(1)) | (spread(q[:, 2]) << np.uint64(2))
    return np.argsort(code, kind="stable")


def reference_point_order(xyz, seed, block=256):
    """Morton order followed by a shuffle of whole 256-point blocks (SceneData.cpp:101-102)."""
    order = morton_order(xyz)
    n = len(order)
    nb = (n + block - 1) // block
    perm = rng(seed).permutation(nb)
    idx = (perm[:, None] * block + np.arange(block)[None, :]).reshape(-1)
    idx = idx[idx < n]
    return order[idx]


def apply_point_order(xyz, nrm, seed, point_order):
    """``morton``: the reference's preprocessing order (Morton curve + shuffled 256-point blocks, which every ADOP
    cloud goes through, SceneData.cpp:101-102); ``random``: a random permutation; ``generated``: unchanged."""
    if point_order == "morton":
        order = reference_point_order(xyz, seed + 7)
    elif point_order == "random":
        order = rng(seed + 8).permutation(len(xyz))
    elif point_order == "generated":
        return xyz, nrm
    else:
        raise ValueError(point_order)
    return xyz[order], (None if nrm is None else nrm[order])


# ---------------------------------------------------------------------------------------------------
# the five benchmark configurations
# ---------------------------------------------------------------------------------------------------

def config1(n=100_000, w=256, h=256, levels=4, seed=0, point_order="generated"):
    """Forward only; points uniform in [-1,1]^3, pinhole 256x256, camera at (0,0,-3) looking +z."""
    g = rng(seed)
    xyz = g.uniform(-1.0, 1.0, (n, 3)).astype(np.float32)
    nrm = _unit(g.standard_normal((n, 3))).astype(np.float32)
    xyz, nrm = apply_point_order(xyz, nrm, seed, point_order)
    pos = np.concatenate([xyz, np.zeros((n, 1), np.float32)], axis=1)
    tex = g.random((4, n), dtype=np.float32)
    f = float(w)
    return HostScene(
        position=pos, normal=pack_normals(nrm), index=np.arange(n, dtype=np.int32), texture=tex,
        background=np.zeros(4, np.float32),
        poses_se3=look_at_view((0, 0, -3), (0, 0, 0), world_up=(0, -1, 0))[None, :],
        intrinsics=pinhole_row(f, f, w / 2, h / 2)[None, :],
        views=[make_view(w, h)], params=default_params(), num_layers=levels, name="config1",
        meta={"point_order": point_order},
    )


def config2(n=1_000_000, w=512, h=512, levels=4, batch=4, seed=0, ghost=True, point_order="morton"):
    """Forward+backward, batch of views on a radius-3 sphere; Gaussian cloud, outward normals."""
    g = rng(seed)
    xyz = (g.standard_normal((n, 3)) * 0.5).astype(np.float32)
    nrm = _unit(xyz.astype(np.float64) + 1e-12).astype(np.float32)
    xyz, nrm = apply_point_order(xyz, nrm, seed, point_order)
    pos = np.concatenate([xyz, np.zeros((n, 1), np.float32)], axis=1)
    tex = np.clip(0.5 + 0.2 * g.standard_normal((4, n)), 0.0, 1.0).astype(np.float32)
    dirs = _unit(g.standard_normal((batch, 3)))
    poses = np.stack([look_at_view(3.0 * d) for d in dirs])
    f = float(w)
    params = default_params(ghost_gradients=1 if ghost else 0)
    return HostScene(
        position=pos, normal=pack_normals(nrm), index=np.arange(n, dtype=np.int32), texture=tex,
        background=np.zeros(4, np.float32), poses_se3=poses,
        intrinsics=pinhole_row(f, f, w / 2, h / 2)[None, :],
        views=[make_view(w, h, image_index=b) for b in range(batch)], params=params, num_layers=levels,
        dropout=bernoulli_mask(seed + 1, batch, n, 0.25) if ghost else None, name="config2",
        meta={"point_order": point_order},
    )


def config3(n=10_000_000, w=1920, h=1080, levels=4, channels=8, seed=0, point_order="morton"):
    """Forward+backward with every gradient: 60% of the points on the unit sphere, 40% on the 4x4 plane
    y=-1; pinhole 1920x1080 fx=fy=1400; camera on the radius-3 sphere, 20 degrees above the horizon."""
    g = rng(seed)
    ns = int(round(n * 0.6))
    npl = n - ns
    sph = _unit(g.standard_normal((ns, 3)))
    pl = np.stack([g.uniform(-2, 2, npl), np.full(npl, -1.0), g.uniform(-2, 2, npl)], axis=1)
    xyz = np.concatenate([sph, pl]).astype(np.float32)
    nrm = np.concatenate([sph, np.tile(np.array([[0.0, 1.0, 0.0]]), (npl, 1))]).astype(np.float32)
    xyz, nrm = apply_point_order(xyz, nrm, seed, point_order)
    pos = np.concatenate([xyz, np.zeros((n, 1), np.float32)], axis=1)
    tex = g.random((channels, n), dtype=np.float32)
    el, az = np.deg2rad(20.0), np.deg2rad(30.0)
    cam = 3.0 * np.array([np.cos(el) * np.sin(az), np.sin(el), -np.cos(el) * np.cos(az)])
    scale = w / 1920.0
    params = default_params(ghost_gradients=1)
    return HostScene(
        position=pos, normal=pack_normals(nrm), index=np.arange(n, dtype=np.int32), texture=tex,
        background=np.zeros(channels, np.float32), poses_se3=look_at_view(cam)[None, :],
        intrinsics=pinhole_row(1400.0 * scale, 1400.0 * scale, w / 2, h / 2)[None, :],
        views=[make_view(w, h)], params=params, num_layers=levels,
        dropout=bernoulli_mask(seed + 1, 1, n, 0.25), name="config3", meta={"point_order": point_order},
    )


def orbit_pose(frame, radius=12.0, deg_per_frame=1.2):
    a = np.deg2rad(frame * deg_per_frame)
    return look_at_view((radius * np.sin(a), 0.0, -radius * np.cos(a)))


def training_batch(n=10_000_000, frames=4, per_frame=4, crop=512, seed=1, point_order="morton"):
    """A training batch as the reference forms it (configs/train_boat.ini:5-6, Dataset.cpp:107-227): `frames` frames
    x `per_frame` random crops of crop x crop (zoom 0.75 .. 1.5) of the config-3 scene, all gradients."""
    hs = config3(n=n, point_order=point_order)
    g = np.random.default_rng(seed)
    hs.poses_se3 = np.stack([orbit_pose(f, radius=3.0, deg_per_frame=20.0) for f in range(frames)])
    views = []
    for f in range(frames):
        for _ in range(per_frame):
            zoom = float(g.uniform(0.75, 1.5))
            # window of crop / zoom source pixels somewhere inside the 1920 x 1080 frame
            src = crop / zoom
            x0 = float(g.uniform(0, 1920 - src))
            y0 = float(g.uniform(0, 1080 - src))
            views.append(make_view(crop, crop, image_index=f, crop=(zoom, zoom, -x0 * zoom, -y0 * zoom, 0.0)))
    hs.views = views
    hs.dropout = bernoulli_mask(2, len(views), hs.num_points, 0.25)
    hs.name = "crops"
    return hs


def config4(n=100_000_000, w=1920, h=1080, levels=5, frames=300, seed=0, point_order="morton"):
    """Viewer path: uniform points in a 10^3 volume, fp16-stored descriptors, 300-frame orbit of radius 12."""
    g = rng(seed)
    pos = np.empty((n, 4), np.float32)
    chunk = 10_000_000
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        pos[s:e, :3] = g.uniform(-5.0, 5.0, (e - s, 3)).astype(np.float32)
    pos[:, 3] = 0
    if point_order != "generated":
        xyz, _ = apply_point_order(pos[:, :3], None, seed, point_order)
        pos[:, :3] = xyz
        del xyz
    tex = np.empty((4, n), np.float16)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        tex[:, s:e] = g.random((4, e - s), dtype=np.float32).astype(np.float16)
    poses = np.stack([orbit_pose(f) for f in range(frames)])
    params = default_params(check_normal=0)
    scale = w / 1920.0
    return HostScene(
        position=pos, normal=None, index=np.arange(n, dtype=np.int32), texture=tex,
        background=np.zeros(4, np.float32), poses_se3=poses,
        intrinsics=pinhole_row(1400.0 * scale, 1400.0 * scale, w / 2, h / 2)[None, :],
        views=[make_view(w, h)], params=params, num_layers=levels, name="config4",
        meta={"point_order": point_order},
    )


def ocam_row(w, h, seed=0, max_angle_deg=95.0):
    """(c,d,e,cx,cy) + 5th-order world2cam polynomial in theta = atan(-z/|xy|) (theta = -pi/2 on the axis):
    an equidistant fisheye that maps ``max_angle_deg`` off-axis to half the image width, plus small seeded
    higher-order terms."""
    g = rng(seed + 100)
    f = (w / 2.0) / np.deg2rad(max_angle_deg)
    poly = np.array([f * np.pi / 2, f, 0, 0, 0, 0], dtype=np.float64)
    poly[2:] = g.uniform(-1.0, 1.0, 4) * np.array([4.0, 2.0, 1.0, 0.5])
    return np.concatenate([[1.0, 0.0, 0.0, w / 2.0, h / 2.0], poly]).astype(np.float32)


def config5(n=20_000_000, w=2200, h=1500, levels=4, batch=8, patches=1000, seed=0, env_hw=(512, 1024),
            point_order="morton"):
    """Forward+backward, OCam fisheye, random planar patches, spherical environment map."""
    g = rng(seed)
    centers = g.uniform(-3.0, 3.0, (patches, 3))
    normals = _unit(g.standard_normal((patches, 3)))
    a = _unit(np.cross(normals, g.standard_normal((patches, 3))))
    b = np.cross(normals, a)
    pid = g.integers(0, patches, n)
    u = g.uniform(-0.25, 0.25, (n, 1))
    v = g.uniform(-0.25, 0.25, (n, 1))
    xyz = (centers[pid] + u * a[pid] + v * b[pid]).astype(np.float32)
    nrm = normals[pid].astype(np.float32)
    xyz, nrm = apply_point_order(xyz, nrm, seed, point_order)
    pos = np.concatenate([xyz, np.zeros((n, 1), np.float32)], axis=1)
    tex = g.random((4, n), dtype=np.float32)
    dirs = _unit(g.standard_normal((batch, 3)))
    poses = np.stack([look_at_view(5.0 * d) for d in dirs])
    params = default_params(dist_cutoff=float(np.deg2rad(95.0 - 90.0)), output_background_mask=1)
    env = g.random((4, env_hw[0], env_hw[1]), dtype=np.float32)
    return HostScene(
        position=pos, normal=pack_normals(nrm), index=np.arange(n, dtype=np.int32), texture=tex,
        background=np.zeros(4, np.float32), poses_se3=poses, intrinsics=ocam_row(w, h, seed)[None, :],
        views=[make_view(w, h, image_index=i, model=_capi.CAMERA_OCAM) for i in range(batch)],
        params=params, num_layers=levels, env_texture=env, name="config5", meta={"point_order": point_order},
    )


def upstream_grads(scene, seed=123):
    """Upstream per-pixel gradients ~ N(0,1), one [B,C,h_l,w_l] array per level."""
    g = rng(seed)
    return [
        g.standard_normal((scene.batch, scene.num_channels, h, w)).astype(np.float32)
        for (w, h) in scene.level_sizes()
    ]
