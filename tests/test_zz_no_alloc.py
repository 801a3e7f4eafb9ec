"""The entry point that allocates nothing: adop_point_distance_to_camera_static keeps the per-frame constants in an
array inside the library instead of a caller's workspace.  Its results must equal adop_point_distance_to_camera's bit
for bit, also on a second, smaller call that finds the array filled by the first."""
import ctypes as C

import numpy as np
import pytest

from helpers import announce

pytestmark = pytest.mark.gpu


def _rig(seed, n, frames):
    import torch
    from adop_amd import scenes

    g = scenes.rng(seed)
    pos = np.concatenate([g.uniform(-1.5, 1.5, (n, 3)), np.zeros((n, 1))], axis=1).astype(np.float32)
    poses = np.stack([scenes.orbit_pose(f, radius=3.0, deg_per_frame=360.0 / frames) for f in range(frames)])
    intr = np.array([[300.0, 310.0, 160.0, 120.0, 0.0, 0.05, -0.01, 0.001, 0.002, 0.0, 0.0, 0.001, -0.0005],
                     [150.0, 150.0, 100.0, 80.0, 0.0, 0, 0, 0, 0, 0, 0, 0, 0]], np.float32)
    views = [scenes.make_view(320, 240, image_index=f, camera_index=0) if f % 3 else
             scenes.make_view(200, 160, image_index=f, camera_index=1) for f in range(frames)]
    return torch.from_numpy(pos).cuda(), torch.from_numpy(poses).cuda(), torch.from_numpy(intr).cuda(), views


def _both(pos, poses, intr, frames):
    import torch
    from adop_amd import _capi, preprocess

    lib = _capi.load_library()
    want = preprocess.PointDistanceToCamera(pos, poses, intr, frames)
    s = _capi.Scene()
    s.position, s.num_points = pos.data_ptr(), int(pos.shape[0])
    s.poses_se3, s.num_poses = poses.data_ptr(), int(poses.shape[0])
    s.intrinsics, s.num_cameras, s.intrinsics_cols = intr.data_ptr(), int(intr.shape[0]), 13
    views = (_capi.View * len(frames))(*frames)
    got = torch.full((s.num_points,), -1.0, dtype=torch.float32, device=pos.device)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.adop_point_distance_to_camera_static(C.byref(s), views, len(frames), C.c_void_p(got.data_ptr()), stream)
    assert rc == _capi.ADOP_OK, lib.adop_last_error_string().decode()
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_entry_point_equals_the_workspace_one():
    from adop_amd import _capi

    lib = _capi.load_library()
    assert lib.adop_static_max_frames() == 1024
    announce("camera distance without a workspace: 200 000 points, 70 frames")
    pos, poses, intr, frames = _rig(1, 200_000, 70)
    got, want = _both(pos, poses, intr, frames)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert (got > 0).all() and (got < np.float32(np.sqrt(105235545.0))).any()
    # second call in a row, smaller in points and frames: the array still holds the 70 frames of the first call
    announce("camera distance without a workspace: 5 000 points, 9 frames (second call)")
    pos2, poses2, intr2, frames2 = _rig(2, 5_000, 9)
    got2, want2 = _both(pos2, poses2, intr2, frames2)
    assert np.array_equal(got2.view(np.uint32), want2.view(np.uint32))
    # and the first input once more gives the first result
    got3, _ = _both(pos, poses, intr, frames)
    assert np.array_equal(got3.view(np.uint32), want.view(np.uint32))
    # what the entry point is for: after the first call on the device (which looks the array's address up) a call
    # allocates and frees no device memory.  Free memory as the driver reports it, around calls that go to buffers
    # allocated beforehand (torch's caching allocator is not asked for anything in between).
    import torch

    s = _capi.Scene()
    s.position, s.num_points = pos.data_ptr(), int(pos.shape[0])
    s.poses_se3, s.num_poses = poses.data_ptr(), int(poses.shape[0])
    s.intrinsics, s.num_cameras, s.intrinsics_cols = intr.data_ptr(), int(intr.shape[0]), 13
    views = (_capi.View * len(frames))(*frames)
    out = torch.empty(s.num_points, dtype=torch.float32, device=pos.device)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        rc = lib.adop_point_distance_to_camera_static(C.byref(s), views, len(frames), C.c_void_p(out.data_ptr()), stream)
        assert rc == _capi.ADOP_OK
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "a call changed the free device memory"
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_static_scratch_entry_point_rejects_too_many_frames():
    import torch
    from adop_amd import _capi

    announce("camera distance without a workspace: 1025 frames are rejected")
    lib = _capi.load_library()
    pos, poses, intr, frames = _rig(3, 100, 4)
    many = [frames[i % 4] for i in range(1025)]
    s = _capi.Scene()
    s.position, s.num_points = pos.data_ptr(), 100
    s.poses_se3, s.num_poses = poses.data_ptr(), 4
    s.intrinsics, s.num_cameras, s.intrinsics_cols = intr.data_ptr(), 2, 13
    out = torch.zeros(100, dtype=torch.float32, device="cuda")
    rc = lib.adop_point_distance_to_camera_static(C.byref(s), (_capi.View * 1025)(*many), 1025,
                                                  C.c_void_p(out.data_ptr()), None)
    assert rc == _capi.ADOP_INVALID_ARG
    assert b"at most 1024 frames" in lib.adop_last_error_string()
    # exactly the maximum is accepted
    rc = lib.adop_point_distance_to_camera_static(C.byref(s), (_capi.View * 1024)(*many[:1024]), 1024,
                                                  C.c_void_p(out.data_ptr()), None)
    assert rc == _capi.ADOP_OK
    torch.cuda.synchronize()
