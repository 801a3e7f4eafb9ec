"""A scene written to the reference's directory format and loaded back renders, through the HIP path, what the CPU
checker computes from the loaded tensors, and the same as the scene it was written from."""
import numpy as np
import pytest

from helpers import announce, check_forward, download_forward, run_hip_forward

pytestmark = pytest.mark.gpu


def unpack_normals(packed):
    q = np.stack([packed & 1023, (packed >> 10) & 1023, (packed >> 20) & 1023], 1).astype(np.float32)
    return q / np.float32(1023.0) * np.float32(2.0) - np.float32(1.0)


def test_scene_from_disk_renders_like_its_source(oracle_mod, tmp_path):
    from adop_amd import scene_io, scenes

    src = scenes.config2(n=30000, w=128, h=96, levels=3, batch=3, seed=4, ghost=False)
    src.intrinsics[0, 5:] = [0.02, -0.004, 0.001, 0.01, 0.0, 0.0, 0.0005, -0.0005]
    sd = scene_io.SceneData()
    sd.scene_cameras = [scene_io.SceneCameraParams(w=128, h=96, K=src.intrinsics[0, :5], distortion=src.intrinsics[0, 5:])]
    sd.frames = [scene_io.FrameData(image_index=i, pose=scene_io.invert_pose(p[:7])) for i, p in enumerate(src.poses_se3)]
    sd.point_position = src.position[:, :3]
    sd.point_normal = unpack_normals(src.normal)
    sd.save(str(tmp_path / "scene"))

    ld = scene_io.SceneData.load(str(tmp_path / "scene"))
    hs = ld.host_scene(range(3), texture=src.texture, num_layers=3)
    np.testing.assert_array_equal(hs.intrinsics, src.intrinsics)
    np.testing.assert_array_equal(hs.normal, src.normal)  # quantise(unquantise(q)) == q
    np.testing.assert_allclose(hs.poses_se3, src.poses_se3, atol=1e-14)
    announce("scene loaded from disk: N=30000 128x96 L=3 B=3")
    scene, info, ctx, images, masks = run_hip_forward(hs)
    check_forward(hs, oracle_mod.forward(hs), ctx, images, masks, info)
    got = download_forward(hs, info, images, masks)
    scene, info, ctx, images, masks = run_hip_forward(src)
    want = download_forward(src, info, images, masks)
    for a, b in zip(got.out, want.out):  # poses differ by a double rounding: all but a stray pixel agree
        assert np.mean(a != b) < 1e-3


@pytest.mark.parametrize("forward_path", [1, 2], ids=["direct", "tiles"])
def test_crop_view_is_a_window_of_the_full_render(forward_path):
    """A crop transform with zoom 1 and an offset that is a multiple of 2^(levels-1) pixels shifts every level by whole
    pixels (the subtraction is exact in fp32 for the points inside the window), so the crop renders exactly the
    window of the full image: packed depth and depth bit for bit, weights equal, descriptors to summation order."""
    from adop_amd import scenes

    n, w, h, levels = 80000, 256, 192, 4
    ox, oy, cw, ch = 64, 40, 128, 96
    full = scenes.config2(n=n, w=w, h=h, levels=levels, batch=1, seed=2, ghost=False)
    full.params.forward_path = forward_path
    crop = scenes.config2(n=n, w=w, h=h, levels=levels, batch=1, seed=2, ghost=False)
    crop.params.forward_path = forward_path
    crop.views = [scenes.make_view(cw, ch, crop=(1.0, 1.0, -float(ox), -float(oy), 0.0))]
    announce(f"crop window {cw}x{ch}+{ox}+{oy} of {w}x{h}, N={n} L={levels} forward_path={forward_path}")
    scene, info, ctx, images, masks = run_hip_forward(full)
    F = download_forward(full, info, images, masks)
    scene, info, ctx, images, masks = run_hip_forward(crop)
    G = download_forward(crop, info, images, masks)
    ids = (1 << 32) - 1
    for l in range(levels):
        x0, y0 = ox >> l, oy >> l
        win = (slice(None), slice(None), slice(y0, y0 + (ch >> l)), slice(x0, x0 + (cw >> l)))
        # the same depth wins; where two points tie in depth the id breaks the tie the same way
        assert np.array_equal(G.depth_index[l], F.depth_index[l][win]), l
        assert np.array_equal(G.depth[l].view(np.uint32), F.depth[l][win].view(np.uint32)), l
        assert np.array_equal(G.weight[l], F.weight[l][win]), l
        assert (G.depth_index[l] & ids != ids).mean() > 0.3  # the window is not empty
        a, b = G.out[l], F.out[l][win]
        assert np.abs(a - b).max() <= 1e-5 * max(1.0, np.abs(b).max()), l
