"""The scene directory format (scenes/README.md:57-95, SceneData.cpp:36-263): files written by hand in the reference's
layout parse to the expected values, the pose stored for the renderer is the inverse of the pose in poses.txt (checked
against a 4x4 matrix inverse), and a scene survives save -> load."""
import os

import numpy as np
import pytest

from adop_amd import scene_io, scenes


def homogeneous(pose):
    m = np.eye(4)
    m[:3, :3] = scenes.quaternion_to_rotation(np.asarray(pose[:4]) / np.linalg.norm(pose[:4]))
    m[:3, 3] = pose[4:7]
    return m


def write(path, text):
    with open(path, "w") as f:
        f.write(text)


def hand_written_scene(d):
    write(d / "dataset.ini", "[SceneDatasetParams]\nfile_model = \nimage_dir = images/\nmask_dir = not set\n"
          "camera_files = camera0.ini camera1.ini\nfile_point_cloud = point_cloud.ply\ncamera_type_int = 0\n"
          "znear = 0.25\nzfar = 500\nrender_scale = 0.5\nscene_exposure_value = 14.5\nup_vector = 0 0 1\n")
    write(d / "camera0.ini", "[SceneCameraParams]\nw = 640\nh = 480\n# fx fy cx cy s\nK = 500.5 501.25 320 240 0.125\n"
          "# 8 paramter distortion model. see distortion.h\ndistortion = 0.1 -0.02 0.003 0 0 0 0.0005 -0.0007\n")
    write(d / "camera1.ini", "[SceneCameraParams]\nw = 1920   # wide\nh = 1080\nK = 1400 1400 960 540 0\n")
    write(d / "poses.txt", "0 0 0 1 0 0 -3\n0 0.70710678118654757 0 0.70710678118654757 1 2 3\n0 0 0 2 0.5 0 0\n")
    write(d / "images.txt", "a.jpg\nb.jpg\nc.jpg\n")
    write(d / "camera_indices.txt", "0\n1\n0\n")
    write(d / "exposure.txt", "13.5\n14\n14.5\n")
    write(d / "white_balance.txt", "1 1 1\n1.1 1 0.9\n1 1 1\n")
    write(d / "point_cloud.ply", "ply\nformat ascii 1.0\ncomment made by hand\nelement vertex 3\nproperty float x\n"
          "property float y\nproperty float z\nproperty float nx\nproperty float ny\nproperty float nz\n"
          "property uchar red\nproperty uchar green\nproperty uchar blue\nelement face 1\n"
          "property list uchar int vertex_indices\nend_header\n"
          "0 0 0 0 0 1 255 0 0\n1 2.5 -3 0 1 0 0 255 0\n-1e-3 4 5 1 0 0 0 0 51\n3 0 1 2\n")


def test_hand_written_files_parse(tmp_path):
    hand_written_scene(tmp_path)
    sd = scene_io.SceneData.load(str(tmp_path))
    dp = sd.dataset_params
    assert dp.camera_files == ["camera0.ini", "camera1.ini"] and dp.image_dir == "images/"
    assert (dp.znear, dp.zfar, dp.render_scale, dp.scene_exposure_value) == (0.25, 500.0, 0.5, 14.5)
    assert dp.camera_model == scene_io.CAMERA_PINHOLE_DISTORTION and list(dp.scene_up_vector) == [0, 0, 1]
    c0, c1 = sd.scene_cameras
    assert (c0.w, c0.h, c1.w, c1.h) == (640, 480, 1920, 1080)
    assert c0.K.dtype == np.float32 and list(c0.K) == [500.5, 501.25, 320, 240, 0.125]
    np.testing.assert_array_equal(c0.distortion, np.float32([0.1, -0.02, 0.003, 0, 0, 0, 0.0005, -0.0007]))
    assert not c1.distortion.any()
    assert [f.camera_index for f in sd.frames] == [0, 1, 0] and [f.image_index for f in sd.frames] == [0, 1, 2]
    assert [(f.w, f.h) for f in sd.frames] == [(640, 480), (1920, 1080), (640, 480)]
    assert [f.target_file for f in sd.frames] == ["a.jpg", "b.jpg", "c.jpg"]
    assert [f.exposure_value for f in sd.frames] == [13.5, 14.0, 14.5]
    np.testing.assert_array_equal(sd.frames[1].white_balance, np.float32([1.1, 1, 0.9]))
    np.testing.assert_array_equal(sd.point_position, np.float32([[0, 0, 0], [1, 2.5, -3], [-1e-3, 4, 5]]))
    np.testing.assert_array_equal(sd.point_normal, np.float32([[0, 0, 1], [0, 1, 0], [1, 0, 0]]))
    np.testing.assert_array_equal(sd.point_color, np.float32([[1, 0, 0], [0, 1, 0], [0, 0, 0.2]]))
    # tensors of the render stage
    K = sd.intrinsics()
    assert K.shape == (2, 13) and K.dtype == np.float32
    np.testing.assert_array_equal(K[0], np.concatenate([c0.K, c0.distortion]))
    np.testing.assert_array_equal(K[1], np.float32([1400, 1400, 960, 540, 0] + [0] * 8))
    P = sd.poses_se3()
    assert P.shape == (3, 8) and P.dtype == np.float64
    # a camera at (0,0,-3) with the identity rotation sees the origin at z = +3
    np.testing.assert_array_equal(P[0], [0, 0, 0, 1, 0, 0, 3, 0])
    # the unnormalised quaternion (0,0,0,2) is the identity rotation
    np.testing.assert_allclose(P[2], [0, 0, 0, 1, -0.5, 0, 0, 0], atol=1e-15)
    v = sd.view(1, scale=0.5)
    assert (v.w, v.h, v.image_index, v.camera_index, v.crop_fx, v.crop_fy) == (960, 540, 1, 1, 0.5, 0.5)


def test_stored_pose_is_the_matrix_inverse():
    g = np.random.default_rng(5)
    for _ in range(50):
        pose = np.concatenate([g.standard_normal(4), g.uniform(-10, 10, 3)])
        pose[:4] /= np.linalg.norm(pose[:4])
        inv = scene_io.invert_pose(pose)
        np.testing.assert_allclose(homogeneous(inv), np.linalg.inv(homogeneous(pose)), atol=1e-13)
        np.testing.assert_allclose(homogeneous(inv) @ homogeneous(pose), np.eye(4), atol=1e-13)
    # look_at_view returns the view transform directly: inverting it gives a camera placed at cam_pos
    view = scenes.look_at_view((1.0, 2.0, -3.0))
    np.testing.assert_allclose(scene_io.invert_pose(view[:7])[4:], [1.0, 2.0, -3.0], atol=1e-14)


def test_save_load_round_trip(tmp_path):
    g = np.random.default_rng(9)
    n = 1000
    sd = scene_io.SceneData()
    sd.dataset_params.camera_files = ["camera0.ini", "camera1.ini"]
    sd.scene_cameras = [scene_io.SceneCameraParams(w=320, h=200, K=np.float32([300.123, 299.7, 160.4, 99.9, 0.01]),
                                                  distortion=g.uniform(-0.01, 0.01, 8).astype(np.float32)),
                        scene_io.SceneCameraParams(w=64, h=48, K=np.float32([60, 61, 32, 24, 0]))]
    for i in range(7):
        view = scenes.look_at_view(3.0 * g.standard_normal(3))
        sd.frames.append(scene_io.FrameData(image_index=i, camera_index=i % 2, pose=scene_io.invert_pose(view[:7]),
                                            exposure_value=float(i) / 4, target_file=f"img{i:04d}.png"))
    sd.point_position = g.standard_normal((n, 3)).astype(np.float32)
    nrm = g.standard_normal((n, 3))
    sd.point_normal = (nrm / np.linalg.norm(nrm, axis=1, keepdims=True)).astype(np.float32)
    sd.point_color = (g.integers(0, 256, (n, 3)) / 255.0).astype(np.float32)
    sd.save(str(tmp_path / "scene"))
    assert sorted(os.listdir(tmp_path / "scene")) == ["camera0.ini", "camera1.ini", "camera_indices.txt", "dataset.ini",
                                                      "exposure.txt", "images.txt", "point_cloud.ply", "poses.txt"]
    ld = scene_io.SceneData.load(str(tmp_path / "scene"))
    np.testing.assert_array_equal(ld.intrinsics(), sd.intrinsics())  # 15 digits carry a float exactly
    np.testing.assert_array_equal(np.stack([f.pose for f in ld.frames]), np.stack([f.pose for f in sd.frames]))
    np.testing.assert_array_equal(ld.poses_se3(), sd.poses_se3())
    assert [(f.camera_index, f.w, f.h, f.target_file, f.exposure_value) for f in ld.frames] == \
           [(i % 2, (320, 64)[i % 2], (200, 48)[i % 2], f"img{i:04d}.png", i / 4) for i in range(7)]
    np.testing.assert_array_equal(ld.point_position, sd.point_position)
    np.testing.assert_array_equal(ld.point_normal, sd.point_normal)
    np.testing.assert_array_equal(ld.point_color, sd.point_color)
    hs = ld.host_scene([0, 2, 4], texture=np.ones((4, n), np.float32), num_layers=3)
    assert hs.position.shape == (n, 4) and hs.batch == 3 and hs.poses_se3.shape == (7, 8)
    np.testing.assert_array_equal(hs.normal, scenes.pack_normals(sd.point_normal))
    assert [(v.w, v.h, v.image_index, v.camera_index) for v in hs.views] == [(320, 200, i, 0) for i in (0, 2, 4)]


def test_ocam_rows(tmp_path):
    hand_written_scene(tmp_path)
    write(tmp_path / "dataset.ini", "[SceneDatasetParams]\ncamera_files = camera.ini\ncamera_type_int = 1\n")
    write(tmp_path / "camera.ini", "[SceneCameraParams]\nw = 2200\nh = 1500\nop = 1.0 0.001 -0.002 1100 750\n"
          "poly_world2cam = 800 500 -30 20 5\npoly_cam2world = -500 0 0.0007\nocam_cutoff = 0.9\n")
    write(tmp_path / "camera_indices.txt", "0\n0\n0\n")
    sd = scene_io.SceneData.load(str(tmp_path))
    K = sd.intrinsics()
    assert K.shape == (1, 10) and K.dtype == np.float32
    np.testing.assert_array_equal(K[0], np.float32([1, 0.001, -0.002, 1100, 750, 800, 500, -30, 20, 5]))
    assert sd.scene_cameras[0].ocam_cutoff == 0.9 and sd.view(0).camera_model_type == scene_io.CAMERA_OCAM


def test_inconsistent_scenes_are_rejected(tmp_path):
    with pytest.raises(AssertionError, match="dataset.ini"):
        scene_io.SceneData.load(str(tmp_path))
    hand_written_scene(tmp_path)
    write(tmp_path / "camera_indices.txt", "0\n1\n")
    with pytest.raises(AssertionError, match="camera_indices"):
        scene_io.SceneData.load(str(tmp_path))
    write(tmp_path / "camera_indices.txt", "0\n1\n0\n")
    write(tmp_path / "poses.txt", "0 0 0 1 0 0\n")
    with pytest.raises(AssertionError, match="pose line"):
        scene_io.SceneData.load(str(tmp_path))
    os.remove(tmp_path / "camera1.ini")
    with pytest.raises(AssertionError, match="camera1.ini"):
        scene_io.SceneData.load(str(tmp_path))
