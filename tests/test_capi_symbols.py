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
             "adop_stage_time": _capi.StageTime, "adop_tuning": _capi.Tuning}
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


def test_workspace_variants_and_their_independence_of_the_tuning():
    """adop_workspace_size_for: what a caller may leave out, per point and view; no size depends on the tuning switches
    (the layout of a call must not move with a switch another thread sets between two calls)."""
    lib = _capi.load_library()
    s = _capi.Scene()
    s.num_poses, s.num_cameras, s.intrinsics_cols, s.num_channels, s.num_points = 3, 1, 13, 8, 1_000_000
    B, N = 4, 1_000_000
    args = (C.byref(s), B, 4, 512, 512)
    full = lib.adop_workspace_size(*args)
    assert lib.adop_workspace_size_for(*args, 0) == full
    kept = lib.adop_workspace_size_for(*args, _capi.WORKSPACE_POINT_CACHE_KEPT)
    direct = lib.adop_workspace_size_for(*args, _capi.WORKSPACE_NO_TILE_PATH)
    both = lib.adop_workspace_size_for(*args, _capi.WORKSPACE_POINT_CACHE_KEPT | _capi.WORKSPACE_NO_TILE_PATH)
    slack = 1 << 20
    assert abs((full - kept) - 20 * B * N) < slack    # projected points 16 B + candidate list 4 B per point and view
    # tile word 4 B + two bin entries of 16 B per point and view, + counters, tile order and the rows of split bins
    assert 36 * B * N < full - direct < 36 * B * N + 24 * slack
    assert abs((kept - both) - (full - direct)) < slack
    assert lib.adop_workspace_size_for(*args, 8) == 0  # unknown flag
    small = lib.adop_workspace_size_for(*args, _capi.WORKSPACE_SMALL_BINS)
    assert abs((full - small) - 28 * B * N) < slack  # two entries per point and view -> one per four: 32 -> 4 bytes
    # a cloud beyond what the bin entries can address: the bins are left out of every layout
    s.num_points = (1 << 28) + 5
    assert lib.adop_workspace_size(C.byref(s), 1, 4, 512, 512) == \
        lib.adop_workspace_size_for(C.byref(s), 1, 4, 512, 512, _capi.WORKSPACE_NO_TILE_PATH)
    s.num_points = N
    with _capi.tuning(bin_shard_shift=3, tile_slice_entries=7, forward_path=1, count_ppt=4):
        assert lib.adop_workspace_size(*args) == full
    with _capi.tuning(bin_shard_shift=0):
        assert lib.adop_workspace_size(*args) == full


def test_tuning_set_get_defaults_and_range_checks():
    lib = _capi.load_library()
    d, t = _capi.Tuning(), _capi.Tuning()
    lib.adop_tuning_defaults(C.byref(d))
    lib.adop_get_tuning(C.byref(t))
    assert bytes(d) == bytes(t)  # nothing set yet in this process (the tests put back what they change)
    assert (d.forward_path, d.tile_slice_entries, d.ghost_concurrent, d.bin_shard_shift) == (0, 8192, -1, -1)
    assert (d.count_ppt, d.scatter_ppt, d.tile_k, d.list_block, d.normalize_fused) == (0, 2, 1, 128, 1)
    with _capi.tuning(tile_slice_entries=64, ghost_concurrent=0) as now:
        lib.adop_get_tuning(C.byref(t))
        assert t.tile_slice_entries == 64 and t.ghost_concurrent == 0 and bytes(t) == bytes(now)
    lib.adop_get_tuning(C.byref(t))
    assert bytes(d) == bytes(t)
    for field, bad in (("forward_path", 3), ("tile_slice_entries", 0), ("ghost_concurrent", 2), ("bin_shard_shift", 4),
                       ("count_ppt", 3), ("count_ppt", -1), ("scatter_ppt", 0), ("tile_k", 8), ("list_block", 100), ("prepass_ppt", 3),
                       ("direct_lists", 2), ("prepass_group_from", 6)):
        with pytest.raises(ValueError, match="tuning"):
            with _capi.tuning(**{field: bad}):
                pass
        lib.adop_get_tuning(C.byref(t))
        assert bytes(d) == bytes(t), field  # a refused set changes nothing
    assert lib.adop_set_tuning(None) != 0
    # the library reads no environment variable
    src = "".join(open(os.path.join(ROOT, "adop_amd", "csrc", f)).read()
                  for f in os.listdir(os.path.join(ROOT, "adop_amd", "csrc")) if f.endswith((".hip", ".h")))
    assert "getenv" not in src


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
