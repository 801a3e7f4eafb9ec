"""ctypes mirror of ``include/adop_raster.h`` and loader of the HIP library ``libadop_raster.so``.

The structs below are field-for-field copies of the C declarations; ``tests/test_capi_symbols.py`` checks
the sizes and that every declared entry point is exported.  There is no CPU fallback: if the shared library
has not been built, loading raises.
"""
import ctypes as C
import os

ADOP_MAX_LAYERS = 5

ADOP_OK = 0
ADOP_INVALID_ARG = 1
ADOP_UNSUPPORTED_LAYERS = 2
ADOP_HIP_ERROR = 3
ADOP_WORKSPACE_TOO_SMALL = 4

CAMERA_PINHOLE_DISTORTION = 0
CAMERA_OCAM = 1

TEXTURE_F32 = 0
TEXTURE_F16 = 1


class View(C.Structure):
    _fields_ = [
        ("w", C.c_int32),
        ("h", C.c_int32),
        ("image_index", C.c_int32),
        ("camera_index", C.c_int32),
        ("camera_model_type", C.c_int32),
        ("crop_fx", C.c_float),
        ("crop_fy", C.c_float),
        ("crop_cx", C.c_float),
        ("crop_cy", C.c_float),
        ("crop_s", C.c_float),
    ]


class RenderParams(C.Structure):
    _fields_ = [
        ("test_backward_mode", C.c_int32),
        ("check_normal", C.c_int32),
        ("ghost_gradients", C.c_int32),
        ("drop_out_points_by_radius", C.c_int32),
        ("depth_accept", C.c_float),
        ("drop_out_radius_threshold", C.c_float),
        ("dist_cutoff", C.c_float),
        ("distortion_gradient_factor", C.c_float),
        ("K_gradient_factor", C.c_float),
        ("output_background_mask", C.c_int32),
        ("output_background_mask_value", C.c_float),
        ("normalize_mode", C.c_int32),
        ("forward_path", C.c_int32),
        ("skip_points", C.c_int32),
        ("workspace_flags", C.c_uint32),
    ]


class Scene(C.Structure):
    _fields_ = [
        ("position", C.c_void_p),
        ("normal", C.c_void_p),
        ("index", C.c_void_p),
        ("num_points", C.c_int32),
        ("texture", C.c_void_p),
        ("texture_dtype", C.c_int32),
        ("num_channels", C.c_int32),
        ("num_texels", C.c_int32),
        ("background_color", C.c_void_p),
        ("poses_se3", C.c_void_p),
        ("num_poses", C.c_int32),
        ("intrinsics", C.c_void_p),
        ("num_cameras", C.c_int32),
        ("intrinsics_cols", C.c_int32),
        ("index_is_identity", C.c_int32),
    ]


class Layer(C.Structure):
    _fields_ = [
        ("w", C.c_int32),
        ("h", C.c_int32),
        ("depth_index", C.c_void_p),
        ("depth", C.c_void_p),
        ("weight", C.c_void_p),
        ("out", C.c_void_p),
        ("mask", C.c_void_p),
    ]


class ForwardBuffers(C.Structure):
    _fields_ = [
        ("num_layers", C.c_int32),
        ("layers", Layer * ADOP_MAX_LAYERS),
        ("dropout_points", C.c_void_p),
        ("point_cache", C.c_void_p),
        ("pixel_cache", C.c_void_p),
    ]


class BackwardBuffers(C.Structure):
    _fields_ = [
        ("grad_out", C.c_void_p * ADOP_MAX_LAYERS),
        ("grad_texture", C.c_void_p),
        ("grad_background", C.c_void_p),
        ("grad_points", C.c_void_p),
        ("grad_points_count", C.c_void_p),
        ("grad_pose", C.c_void_p),
        ("grad_pose_count", C.c_void_p),
        ("grad_intrinsics", C.c_void_p),
        ("grad_intrinsics_count", C.c_void_p),
    ]


class Stats(C.Structure):
    _fields_ = [
        ("visible", C.c_uint64 * ADOP_MAX_LAYERS),
        ("accepted", C.c_uint64 * ADOP_MAX_LAYERS),
        ("spatial", C.c_uint64 * ADOP_MAX_LAYERS),
        ("bad_index", C.c_uint64),
    ]


class Tuning(C.Structure):
    """adop_tuning: the process's tuning switches (results never depend on them)."""
    _fields_ = [(n, C.c_int32) for n in (
        "forward_path", "tile_slice_entries", "ghost_concurrent", "bin_shard_shift", "direct_lists", "prepass_ppt",
        "prepass_group_from", "blend_group_from", "list_block", "count_ppt", "scatter_ppt", "tile_k", "normalize_fused",
        "normalize_by_queue")]


WORKSPACE_POINT_CACHE_KEPT = 1
WORKSPACE_NO_TILE_PATH = 2
WORKSPACE_SMALL_BINS = 4


class StageTime(C.Structure):
    _fields_ = [("name", C.c_char * 32), ("total_ms", C.c_float), ("calls", C.c_int32)]


# Entry points declared in include/adop_raster.h (name -> (restype, argtypes)).
ENTRY_POINTS = {
    "adop_workspace_size": (C.c_size_t, [C.POINTER(Scene), C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "adop_workspace_size_for": (C.c_size_t, [C.POINTER(Scene), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_uint32]),
    "adop_tuning_defaults": (None, [C.POINTER(Tuning)]),
    "adop_set_tuning": (C.c_int, [C.POINTER(Tuning)]),
    "adop_get_tuning": (None, [C.POINTER(Tuning)]),
    "adop_forward": (
        C.c_int,
        [C.POINTER(Scene), C.POINTER(View), C.c_int32, C.POINTER(RenderParams), C.POINTER(ForwardBuffers),
         C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p],
    ),
    "adop_backward": (
        C.c_int,
        [C.POINTER(Scene), C.POINTER(View), C.c_int32, C.POINTER(RenderParams), C.POINTER(ForwardBuffers),
         C.POINTER(BackwardBuffers), C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p],
    ),
    "adop_env_sample": (
        C.c_int,
        [C.POINTER(Scene), C.POINTER(View), C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.POINTER(ForwardBuffers),
         C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int32, C.c_void_p],
    ),
    "adop_env_sample_backward": (
        C.c_int,
        [C.POINTER(Scene), C.POINTER(View), C.c_int32, C.c_int32, C.c_int32, C.POINTER(ForwardBuffers),
         C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p],
    ),
    "adop_apply_tangent": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]),
    "adop_knn_workspace_size": (C.c_size_t, [C.c_int32]),
    "adop_knn_distance": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.c_int32, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p, C.c_void_p,
         C.c_size_t, C.c_void_p],
    ),
    "adop_morton_codes": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p, C.c_void_p],
    ),
    "adop_frames_workspace_size": (C.c_size_t, [C.c_int32]),
    "adop_point_distance_to_camera": (
        C.c_int,
        [C.POINTER(Scene), C.POINTER(View), C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "adop_static_max_frames": (C.c_int32, []),
    "adop_point_distance_to_camera_static": (
        C.c_int,
        [C.POINTER(Scene), C.POINTER(View), C.c_int32, C.c_void_p, C.c_void_p],
    ),
    "adop_close_points": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p, C.c_void_p,
         C.c_int32, C.c_int32, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "adop_profile_enable": (C.c_int, [C.c_int32]),
    "adop_profile_read": (C.c_int32, [C.POINTER(StageTime), C.c_int32]),
    "adop_last_error_string": (C.c_char_p, []),
    "adop_version": (C.c_char_p, []),
}

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libadop_raster.so")

_lib = None


def load_library(path=None):
    """Load ``libadop_raster.so`` and bind every entry point.  Raises if the library is missing."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise RuntimeError(
            f"{p} not found: the HIP rasterizer has not been built "
            "(run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C adop_amd/csrc`). "
            "There is no CPU fallback."
        )
    # PyTorch ships a HIP runtime of its own.  Loaded after this library it would come up as a second copy beside the
    # system's one, and only one copy gets the GPU (the other reports "no ROCm-capable device"): import torch first,
    # so that the library binds to the runtime torch has already loaded.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(p)
    for name, (restype, argtypes) in ENTRY_POINTS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if path is None:
        _lib = lib
    return lib


class tuning:
    """Context manager: ``with _capi.tuning(tile_slice_entries=64): ...`` sets fields of the process's adop_tuning for
    the calls issued inside and puts the previous set back afterwards (how the tests and the benchmark reach the
    library's tuning switches)."""

    def __init__(self, **fields):
        self.fields = fields

    def __enter__(self):
        lib = load_library()
        self.before = Tuning()
        lib.adop_get_tuning(C.byref(self.before))
        t = Tuning()
        lib.adop_get_tuning(C.byref(t))
        for k, v in self.fields.items():
            if not hasattr(t, k):
                raise AttributeError(k)
            setattr(t, k, int(v))
        rc = lib.adop_set_tuning(C.byref(t))
        if rc != ADOP_OK:
            raise ValueError(lib.adop_last_error_string().decode())
        return t

    def __exit__(self, *exc):
        load_library().adop_set_tuning(C.byref(self.before))
        return False
