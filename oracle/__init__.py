"""CPU checker of the rasterizer (TEST INFRASTRUCTURE: only tests, the smoke check and the benchmark's
cpu_baseline leg may import this package; the product never does).

Thin ctypes/numpy front end of ``adop_oracle.cpp``.
"""
import ctypes as C
import os

import numpy as np

from adop_amd import _capi
from . import build as _build

_libs = {}


def lib(omp=False):
    key = bool(omp)
    if key not in _libs:
        path = _build.LIB_OMP if omp else _build.LIB
        if os.environ.get("ADOP_ORACLE_SANITIZE") == "1":
            # the ASan / UBSan build (tests/test_sanitizers.py runs the pinning tests on it in a child process)
            path = _build.build_sanitized(force=False)
        elif not os.path.exists(path):
            _build.build(force=False)
        L = C.CDLL(path)
        L.oracle_forward.restype = C.c_int
        L.oracle_forward.argtypes = [C.POINTER(_capi.Scene), C.POINTER(_capi.View), C.c_int,
                                     C.POINTER(_capi.RenderParams), C.POINTER(_capi.ForwardBuffers),
                                     C.POINTER(_capi.Stats)]
        L.oracle_backward.restype = C.c_int
        L.oracle_backward.argtypes = [C.POINTER(_capi.Scene), C.POINTER(_capi.View), C.c_int,
                                      C.POINTER(_capi.RenderParams), C.POINTER(_capi.ForwardBuffers),
                                      C.POINTER(_capi.BackwardBuffers), C.POINTER(_capi.Stats)]
        L.oracle_env_uv.restype = None
        L.oracle_env_uv.argtypes = [C.POINTER(_capi.Scene), C.POINTER(_capi.View), C.c_int, C.c_int, C.c_int,
                                    C.c_void_p]
        L.oracle_grid_sample.restype = None
        L.oracle_grid_sample.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int,
                                         C.c_void_p]
        L.oracle_apply_tangent.restype = None
        L.oracle_apply_tangent.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        for name in ("oracle_atanf", "oracle_acosf"):
            getattr(L, name).restype = C.c_float
            getattr(L, name).argtypes = [C.c_float]
        L.oracle_atan2f.restype = C.c_float
        L.oracle_atan2f.argtypes = [C.c_float, C.c_float]
        L.oracle_f2i_rn.restype = C.c_int
        L.oracle_f2i_rn.argtypes = [C.c_float]
        L.oracle_half_to_float.restype = C.c_float
        L.oracle_half_to_float.argtypes = [C.c_uint16]
        L.oracle_pack_normal.restype = C.c_int32
        L.oracle_pack_normal.argtypes = [C.c_float] * 3
        L.oracle_unpack_normal.restype = None
        L.oracle_unpack_normal.argtypes = [C.c_int32, C.c_void_p]
        L.oracle_pack_index.restype = C.c_uint64
        L.oracle_pack_index.argtypes = [C.c_float, C.c_uint32]
        L.oracle_project_pinhole.restype = None
        L.oracle_project_pinhole.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_float,
                                             C.c_void_p]
        L.oracle_project_ocam.restype = None
        L.oracle_project_ocam.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                          C.c_float, C.c_void_p]
        L.oracle_project_pinhole_backward.restype = None
        L.oracle_project_pinhole_backward.argtypes = [C.c_void_p] * 6 + [C.c_int, C.c_float, C.c_void_p]
        L.oracle_project_ocam_backward.restype = None
        L.oracle_project_ocam_backward.argtypes = [C.c_void_p] * 5 + [C.c_int, C.c_void_p, C.c_int, C.c_float,
                                                                      C.c_void_p]
        L.oracle_distort.restype = None
        L.oracle_distort.argtypes = [C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p]
        L.oracle_undistort.restype = None
        L.oracle_undistort.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        L.oracle_sincosf.restype = None
        L.oracle_sincosf.argtypes = [C.c_float, C.c_void_p]
        L.oracle_ocam_unproject.restype = None
        L.oracle_ocam_unproject.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        L.oracle_ocam_core.restype = None
        L.oracle_ocam_core.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_void_p]
        L.oracle_num_threads.restype = C.c_int
        L.oracle_num_threads.argtypes = []
        _libs[key] = L
    return _libs[key]


def _p(a):
    return None if a is None else a.ctypes.data


def scene_struct(hs):
    """ctypes Scene over the numpy arrays of a HostScene (arrays must stay alive)."""
    for name in ("position", "index", "texture", "background", "poses_se3", "intrinsics"):
        a = getattr(hs, name)
        assert a.flags["C_CONTIGUOUS"], name
    s = _capi.Scene()
    s.position = _p(hs.position)
    s.normal = _p(hs.normal)
    s.index = _p(hs.index)
    s.num_points = hs.num_points
    s.texture = _p(hs.texture)
    s.texture_dtype = _capi.TEXTURE_F16 if hs.texture.dtype == np.float16 else _capi.TEXTURE_F32
    s.num_channels = hs.texture.shape[0]
    s.num_texels = hs.texture.shape[1]
    s.background_color = _p(hs.background)
    s.poses_se3 = _p(hs.poses_se3)
    s.num_poses = hs.poses_se3.shape[0]
    s.intrinsics = _p(hs.intrinsics)
    s.num_cameras = hs.intrinsics.shape[0]
    s.intrinsics_cols = hs.intrinsics.shape[1]
    return s


def views_array(hs):
    arr = (_capi.View * hs.batch)()
    for i, v in enumerate(hs.views):
        arr[i] = v
    return arr


class ForwardResult:
    """Per-level numpy outputs: depth_index (u64), depth, weight, out, mask."""

    def __init__(self, hs):
        B, Cn = hs.batch, hs.num_channels
        self.depth_index, self.depth, self.weight, self.out, self.mask = [], [], [], [], []
        for (w, h) in hs.level_sizes():
            self.depth_index.append(np.empty((B, 1, h, w), np.uint64))
            self.depth.append(np.empty((B, 1, h, w), np.float32))
            self.weight.append(np.empty((B, 1, h, w), np.float32))
            self.out.append(np.empty((B, Cn, h, w), np.float32))
            self.mask.append(np.zeros((B, 1, h, w), np.float32))
        self.stats = _capi.Stats()

    def struct(self, hs):
        fb = _capi.ForwardBuffers()
        fb.num_layers = hs.num_layers
        for l, (w, h) in enumerate(hs.level_sizes()):
            L = fb.layers[l]
            L.w, L.h = w, h
            L.depth_index = _p(self.depth_index[l])
            L.depth = _p(self.depth[l])
            L.weight = _p(self.weight[l])
            L.out = _p(self.out[l])
            L.mask = _p(self.mask[l])
        fb.dropout_points = _p(hs.dropout)
        return fb


def forward(hs, omp=False):
    res = ForwardResult(hs)
    s = scene_struct(hs)
    fb = res.struct(hs)
    rc = lib(omp).oracle_forward(C.byref(s), views_array(hs), hs.batch, C.byref(hs.params), C.byref(fb),
                                 C.byref(res.stats))
    if rc != 0:
        raise RuntimeError(f"oracle_forward returned {rc}")
    return res


class BackwardResult:
    def __init__(self, hs, points=True, pose=True, intrinsics=True):
        N = hs.num_points
        self.grad_texture = np.empty(hs.texture.shape, np.float32)
        self.grad_background = np.empty(hs.num_channels, np.float32)
        self.grad_points = np.empty((N, 4), np.float32) if points else None
        self.grad_points_count = np.empty(N, np.float32) if points else None
        F = hs.poses_se3.shape[0]
        self.grad_pose = np.empty((F, 6), np.float64) if pose else None
        self.grad_pose_count = np.empty(F, np.float32) if pose else None
        K = hs.intrinsics.shape[0]
        self.grad_intrinsics = np.empty(hs.intrinsics.shape, np.float32) if intrinsics else None
        self.grad_intrinsics_count = np.empty(K, np.float32) if intrinsics else None
        self.stats = _capi.Stats()

    def struct(self, grad_out):
        gb = _capi.BackwardBuffers()
        for l, g in enumerate(grad_out):
            assert g.flags["C_CONTIGUOUS"] and g.dtype == np.float32
            gb.grad_out[l] = _p(g)
        for name in ("grad_texture", "grad_background", "grad_points", "grad_points_count", "grad_pose",
                     "grad_pose_count", "grad_intrinsics", "grad_intrinsics_count"):
            setattr(gb, name, _p(getattr(self, name)))
        return gb


def backward(hs, fwd, grad_out, points=True, pose=True, intrinsics=True, omp=False):
    res = BackwardResult(hs, points, pose, intrinsics)
    s = scene_struct(hs)
    fb = fwd.struct(hs)
    gb = res.struct(grad_out)
    rc = lib(omp).oracle_backward(C.byref(s), views_array(hs), hs.batch, C.byref(hs.params), C.byref(fb),
                                    C.byref(gb), C.byref(res.stats))
    if rc != 0:
        raise RuntimeError(f"oracle_backward returned {rc}")
    return res


def env_uv(hs, b, level):
    w, h = hs.level_sizes()[level]
    uv = np.empty((h, w, 2), np.float32)
    s = scene_struct(hs)
    v = hs.views[b]
    lib().oracle_env_uv(C.byref(s), C.byref(v), level, w, h, _p(uv))
    return uv


def grid_sample(tex, uv):
    Cn, eh, ew = tex.shape
    h, w, _ = uv.shape
    out = np.empty((Cn, h, w), np.float32)
    tex = np.ascontiguousarray(tex, np.float32)
    uv = np.ascontiguousarray(uv, np.float32)
    lib().oracle_grid_sample(_p(tex), Cn, eh, ew, _p(uv), w, h, _p(out))
    return out


def apply_tangent(tangent, poses):
    t = np.array(tangent, np.float64, copy=True)
    p = np.array(poses, np.float64, copy=True)
    lib().oracle_apply_tangent(_p(t), _p(p), t.shape[0])
    return t, p


def sincos(theta):
    """(sin, cos) of an angle in [-pi/2, pi/2] as the checker evaluates them."""
    out = np.empty(2, np.float32)
    lib().oracle_sincosf(float(theta), _p(out))
    return float(out[0]), float(out[1])


def ocam_unproject(intr_row, ip):
    """Unit camera-space ray of pixel ``ip`` of the uncropped OCam image (row = c,d,e,cx,cy + world2cam poly)."""
    row = np.ascontiguousarray(intr_row, np.float32)
    ipa = np.ascontiguousarray(ip, np.float32)
    out = np.empty(3, np.float32)
    lib().oracle_ocam_unproject(_p(row), row.shape[0], _p(ipa), _p(out))
    return out


def ocam_core(intr_row, view_p, cutoff=10.0):
    """(u, v, z) of a camera-space point through the OCam model alone."""
    row = np.ascontiguousarray(intr_row, np.float32)
    pa = np.ascontiguousarray(view_p, np.float32)
    out = np.empty(3, np.float32)
    lib().oracle_ocam_core(_p(pa), _p(row), row.shape[0], float(cutoff), _p(out))
    return out
