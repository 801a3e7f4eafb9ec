"""The C-ABI library loads and exports every symbol include/adop_raster.h declares; the ctypes mirror has the
same struct sizes as the C header.  No compute call is made (no GPU needed)."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

from adop_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "adop_raster.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(adop_[a-z_0-9]+)\s*\(", text)))


def test_header_and_ctypes_mirror_list_the_same_entry_points():
    assert declared_functions() == sorted(_capi.ENTRY_POINTS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_capi.LIB_PATH):
        pytest.fail(f"{_capi.LIB_PATH} has not been built (python -c 'import __graft_entry__ as g; g.build()')")
    lib = _capi.load_library()
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert b"gfx950" in lib.adop_version()
    assert lib.adop_last_error_string() is not None


def test_loading_a_missing_library_fails_loudly(tmp_path):
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _capi.load_library(str(tmp_path / "libadop_raster.so"))


def test_struct_sizes_match_the_c_header(tmp_path):
    names = {"adop_view": _capi.View, "adop_render_params": _capi.RenderParams, "adop_scene": _capi.Scene,
             "adop_layer": _capi.Layer, "adop_forward_buffers": _capi.ForwardBuffers,
             "adop_backward_buffers": _capi.BackwardBuffers, "adop_stats": _capi.Stats,
             "adop_stage_time": _capi.StageTime}
    src = tmp_path / "sizes.c"
    body = "\n".join(f'printf("{n} %zu\\n", sizeof({n}));' for n in names)
    src.write_text(f'#include <stdio.h>\n#include "{HEADER}"\nint main(void){{\n{body}\nreturn 0;}}\n')
    exe = tmp_path / "sizes"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)])  # header is plain C
    out = subprocess.check_output([str(exe)]).decode().split()
    got = dict(zip(out[::2], map(int, out[1::2])))
    for n, t in names.items():
        assert got[n] == C.sizeof(t), n


def test_workspace_query_needs_no_gpu():
    lib = _capi.load_library()
    s = _capi.Scene()
    s.num_poses, s.num_cameras, s.intrinsics_cols, s.num_channels = 3, 1, 13, 8
    n1 = lib.adop_workspace_size(C.byref(s), 1, 4, 640, 480)
    n4 = lib.adop_workspace_size(C.byref(s), 4, 4, 640, 480)
    pixels = 640 * 480 + 320 * 240 + 160 * 120 + 80 * 60
    assert 64 * pixels < n1 < 64 * pixels + (8 << 20)  # 16 floats per pixel + partial sums + work queue
    assert n1 < n4 < 4 * n1
    assert lib.adop_workspace_size(None, 1, 4, 640, 480) == 0
    assert lib.adop_workspace_size(C.byref(s), 1, 9, 640, 480) == 0


def test_preprocessing_entry_points_reject_bad_arguments_before_any_launch():
    """Argument checks of the point-cloud entry points return a status and a message without touching a device."""
    lib = _capi.load_library()
    INVALID, TOO_SMALL = 1, None
    box_lo, box_hi = (C.c_float * 3)(0, 0, 0), (C.c_float * 3)(1, 1, 1)
    fake = C.c_void_p(256)  # never dereferenced: every call below fails its checks first

    def message():
        return lib.adop_last_error_string().decode()

    # workspace sizes are pure functions of the point count
    w10, w1000 = lib.adop_knn_workspace_size(10), lib.adop_knn_workspace_size(1_000_000)
    assert 0 < w10 < w1000 and lib.adop_knn_workspace_size(-1) == 0
    # below the minimum number of cells the size grows by 2 x 16 B records + 2 x 4 B list entries per point
    w100k = lib.adop_knn_workspace_size(100_000)
    assert abs((w100k - w10) - (100_000 - 10) * 40) <= 4 * 256
    assert w1000 - w100k > 900_000 * 40  # beyond it the cell arrays grow too
    assert lib.adop_frames_workspace_size(0) == 0 and lib.adop_frames_workspace_size(3) >= 3 * 128

    assert lib.adop_knn_distance(None, 100, 4, box_lo, box_hi, fake, fake, w10, None) != 0 and "null" in message()
    assert lib.adop_knn_distance(fake, 100, 0, box_lo, box_hi, fake, fake, w1000, None) != 0 and "rank" in message()
    assert lib.adop_knn_distance(fake, 100, 9, box_lo, box_hi, fake, fake, w1000, None) != 0 and "rank" in message()
    assert lib.adop_knn_distance(fake, 4, 4, box_lo, box_hi, fake, fake, w1000, None) != 0 and "more than" in message()
    assert lib.adop_knn_distance(fake, 100, 4, box_lo, box_hi, fake, fake, 16, None) != 0 and "workspace" in message()
    bad_hi = (C.c_float * 3)(1, float("nan"), 1)
    assert lib.adop_knn_distance(fake, 100, 4, box_lo, bad_hi, fake, fake, w1000, None) != 0 and "finite" in message()
    assert lib.adop_morton_codes(fake, 100, box_lo, bad_hi, fake, None) != 0 and "finite" in message()
    assert lib.adop_morton_codes(fake, 0, box_lo, box_hi, fake, None) == 0  # an empty cloud is no error
    assert lib.adop_close_points(fake, 100, None, box_lo, box_hi, fake, fake, 8, 0, fake, w1000, None) != 0
    assert lib.adop_close_points(fake, 100, fake, box_lo, box_hi, fake, fake, 0, 0, fake, w1000, None) != 0 and "num_rounds" in message()
    assert lib.adop_close_points(fake, 100, fake, box_lo, box_hi, fake, fake, 8, 0, fake, 16, None) != 0 and "workspace" in message()

    s = _capi.Scene()
    s.position, s.num_points = 256, 10
    s.poses_se3, s.num_poses, s.intrinsics, s.num_cameras, s.intrinsics_cols = 256, 2, 256, 1, 13
    v = _capi.View()
    v.w, v.h, v.image_index, v.camera_index, v.camera_model_type = 64, 48, 0, 0, _capi.CAMERA_PINHOLE_DISTORTION
    views = (_capi.View * 1)(v)
    big = lib.adop_frames_workspace_size(1)
    assert lib.adop_point_distance_to_camera(C.byref(s), views, 0, fake, fake, big, None) != 0 and "num_frames" in message()
    assert lib.adop_point_distance_to_camera(C.byref(s), views, 1, fake, fake, 0, None) != 0 and "workspace" in message()
    views[0].image_index = 2
    assert lib.adop_point_distance_to_camera(C.byref(s), views, 1, fake, fake, big, None) != 0 and "range" in message()
    views[0].image_index, views[0].camera_model_type = 0, _capi.CAMERA_OCAM
    assert lib.adop_point_distance_to_camera(C.byref(s), views, 1, fake, fake, big, None) != 0 and "pinhole" in message()
    s.intrinsics_cols = 10
    views[0].camera_model_type = _capi.CAMERA_PINHOLE_DISTORTION
    assert lib.adop_point_distance_to_camera(C.byref(s), views, 1, fake, fake, big, None) != 0 and "13 columns" in message()
