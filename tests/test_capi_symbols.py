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
