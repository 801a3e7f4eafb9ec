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


def window_in_image(row, crop):
    """corners of the crop window in pixels of the input image: (crop pixel - c) / zoom"""
    z = row[0]
    lo = np.array([-row[2], -row[3]]) / z
    return lo, lo + np.asarray(crop) / z


@pytest.mark.parametrize("prefer_border", [False, True])
def test_random_crops_stay_inside_the_image(prefer_border):
    g = np.random.default_rng(3)
    size_in, crop = (1920, 1080), (512, 512)
    rows = scene_io.RandomImageCrop(400, 1, size_in, crop, prefer_border, True, (0.75, 1.5), g)
    assert rows.shape == (400, 5) and rows.dtype == np.float32
    np.testing.assert_array_equal(rows[:, 0], rows[:, 1])
    assert np.all(rows[:, 4] == 0) and rows[:, 0].min() >= 0.75 and rows[:, 0].max() <= 1.5
    assert rows[:, 0].max() - rows[:, 0].min() > 0.6  # the zoom range is used
    touching = 0
    for r in rows:
        lo, hi = window_in_image(r, crop)
        assert np.all(lo >= -1e-3) and np.all(hi <= np.array(size_in) + 1e-3), (r, lo, hi)
        touching += bool(np.any(lo < 1e-3) or np.any(hi > np.array(size_in) - 1e-3))
    # clamping a wider range puts many windows against the border; a plain uniform offset almost none
    assert (touching > 100) if prefer_border else (touching < 20)


def test_crops_without_translation_and_small_images_are_centred():
    rows = scene_io.RandomImageCrop(5, 1, (640, 480), (256, 128), True, False, (1.0, 1.0), np.random.default_rng(0))
    np.testing.assert_array_equal(rows, np.tile(np.float32([1, 1, -192, -176, 0]), (5, 1)))
    # the zoomed image (160 x 120) is smaller than the crop: centred, cx > 0
    rows = scene_io.RandomImageCrop(3, 2, (640, 480), (256, 128), True, True, (0.25, 0.25), np.random.default_rng(0))
    np.testing.assert_array_equal(rows, np.tile(np.float32([0.25, 0.25, 48, 4, 0]), (3, 1)))


def test_more_tries_spread_the_crops():
    def mean_nearest(tries):
        out = []
        for seed in range(20):
            rows = scene_io.RandomImageCrop(8, tries, (1920, 1080), (256, 256), False, True, (1, 1),
                                            np.random.default_rng(seed))
            c = (-rows[:, 2:4] + 128) / rows[:, :1]
            d = np.linalg.norm(c[:, None] - c[None], axis=2) + 1e9 * np.eye(8)
            out.append(d.min(1).mean())
        return np.mean(out)

    assert mean_nearest(8) > 1.3 * mean_nearest(1)


def test_train_sampler_views(tmp_path):
    hand_written_scene(tmp_path)
    sd = scene_io.SceneData.load(str(tmp_path))
    sampler = scene_io.SceneDataTrainSampler(sd, [2, 1], True, (256, 192), 4, seed=1)
    assert len(sampler) == 2
    views, zoom = sampler.Get(1)
    assert len(views) == 4 and zoom.shape == (4,)
    for v, z in zip(views, zoom):
        assert (v.w, v.h, v.image_index, v.camera_index, v.crop_s) == (256, 192, 1, 1, 0.0)
        assert v.crop_fx == v.crop_fy == z and 0.75 <= z <= 1.5
    full = scene_io.SceneDataTrainSampler(sd, [0], False, (0, 0), 2)
    views, zoom = full.Get(0)
    assert [(v.w, v.h, v.crop_fx, v.crop_cx, v.crop_cy) for v in views] == [(640, 480, 1.0, 0.0, 0.0)] * 2
    assert list(zoom) == [1.0, 1.0]


def test_render_params_from_an_experiment_file(tmp_path):
    # the section as the reference's experiment files hold it (values of its boat experiment)
    write(tmp_path / "train.ini", "[TrainParams]\nbatch_size = 4\n\n[RenderParams]\nrender_outliers = false\n"
          "check_normal = true\nghost_gradients = true\ndrop_out_points_by_radius = true\noutlier_count = 1000000\n"
          "drop_out_radius_threshold = 0.6000000238\ndropout = 0.2500000000\ndepth_accept = 0.0099999998\n"
          "test_backward_mode = 0\ndistortion_gradient_factor = 0.0099999998\nK_gradient_factor = 0.5000000000\n\n"
          "[PipelineParams]\ntrain = true\n")
    p, dropout = scene_io.RenderParamsFromIni(str(tmp_path / "train.ini"))
    assert (p.check_normal, p.ghost_gradients, p.drop_out_points_by_radius, p.test_backward_mode) == (1, 1, 1, 0)
    assert dropout == 0.25
    assert np.float32(p.depth_accept) == np.float32(0.01) and np.float32(p.drop_out_radius_threshold) == np.float32(0.6)
    assert np.float32(p.distortion_gradient_factor) == np.float32(0.01) and p.K_gradient_factor == 0.5
    # a file without the section: the defaults of the reference's struct
    write(tmp_path / "empty.ini", "[TrainParams]\nbatch_size = 1\n")
    p, dropout = scene_io.RenderParamsFromIni(str(tmp_path / "empty.ini"))
    assert (p.check_normal, p.ghost_gradients, p.drop_out_points_by_radius, dropout) == (1, 0, 1, 0.25)
    assert np.float32(p.distortion_gradient_factor) == np.float32(0.005)
    write(tmp_path / "outliers.ini", "[RenderParams]\nrender_outliers = true\n")
    with pytest.raises(AssertionError, match="outlier"):
        scene_io.RenderParamsFromIni(str(tmp_path / "outliers.ini"))
