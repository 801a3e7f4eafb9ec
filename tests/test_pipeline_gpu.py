"""The pieces in the order a user of the reference meets them: a scene directory on disk -> loader -> point filters and
reordering on the device -> a training batch of random crops -> forward and backward through the autograd function.
The render results are held against the CPU checker on the same tensors."""
import numpy as np
import pytest

from helpers import announce, check_backward, check_forward, download_forward

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_scene_directory_to_gradients(oracle_mod, tmp_path, collect_stats):
    import torch
    from adop_amd import preprocess, render, scene_io, scenes

    # a scene on disk: Gaussian blob with a few stray points, 6 frames on a ring, one camera
    g = np.random.default_rng(12)
    n = 60000
    sd = scene_io.SceneData()
    sd.scene_cameras = [scene_io.SceneCameraParams(w=256, h=192, K=np.float32([220, 220, 128, 96, 0]),
                                                  distortion=np.float32([0.05, -0.01, 0, 0, 0, 0, 0.001, -0.001]))]
    for i in range(6):
        a = 2 * np.pi * i / 6
        view = scenes.look_at_view((3.0 * np.sin(a), 0.4, -3.0 * np.cos(a)))
        sd.frames.append(scene_io.FrameData(image_index=i, pose=scene_io.invert_pose(view[:7])))
    xyz = (g.standard_normal((n, 3)) * 0.5).astype(np.float32)
    xyz[:30] = (g.standard_normal((30, 3)) * 40).astype(np.float32)  # strays: lonely, mostly unseen
    sd.point_position = xyz
    nrm = xyz / np.maximum(np.linalg.norm(xyz, axis=1, keepdims=True), 1e-9)
    sd.point_normal = nrm.astype(np.float32)
    sd.save(str(tmp_path / "scene"))

    ld = scene_io.SceneData.load(str(tmp_path / "scene"))
    announce("pipeline: load, filter, reorder, crops, render, gradients; N=60000, 6 frames")
    pos = torch.zeros(n, 4, device="cuda")
    pos[:, :3] = torch.from_numpy(ld.point_position).cuda()
    poses = torch.from_numpy(ld.poses_se3()).cuda()
    intr = torch.from_numpy(ld.intrinsics()).cuda()
    frames = [ld.view(i) for i in range(6)]
    ids = preprocess.FilterPointCloud(pos, poses, intr, frames, lonely=(5, 0.05))
    kept = ids.cpu().numpy()
    assert 0.5 * n < len(kept) < n and not np.isin(np.arange(30), kept).all()  # strays went
    pos = pos[ids].contiguous()
    normal = torch.from_numpy(scenes.pack_normals(ld.point_normal)).cuda()[ids]
    pos, normal, data, order = preprocess.PreprocessPointCloud(pos, normal, seed=1)
    m = int(pos.shape[0])
    assert m == len(kept) and float(pos[:, 3].min()) > 0  # every point has its LOD radius

    # a training batch: 3 random crops of frame 2
    sampler = scene_io.SceneDataTrainSampler(ld, [2], True, (128, 96), 3, seed=5)
    views, zoom = sampler.Get(0)
    params = scenes.default_params(check_normal=0, drop_out_points_by_radius=1, drop_out_radius_threshold=0.6,
                                   ghost_gradients=0, normalize_mode=1)
    tex = g.random((4, m), dtype=np.float32)
    hs = scenes.HostScene(position=pos.cpu().numpy(), normal=normal.cpu().numpy().reshape(-1), index=np.arange(m, dtype=np.int32),
                          texture=tex, background=np.float32([0.1, 0.2, 0.3, 0.4]), poses_se3=ld.poses_se3(),
                          intrinsics=ld.intrinsics(), views=views, params=params, num_layers=3)
    scene = render.NeuralScene.from_host(hs, "cuda")
    scene.texture.requires_grad_(True)
    scene.tangent_poses.requires_grad_(True)
    info = render.NeuralRenderInfo(scene=scene, images=list(views), params=params, num_layers=3,
                                   cache=render.PointRendererCache(), collect_stats=collect_stats, train=True)
    images = render.BlendPointCloud(info)[:3]
    ref = oracle_mod.forward(hs)
    check_forward(hs, ref, None, [im.detach() for im in images], [], info, stats=collect_stats)
    assert all(float((L.weight > 0).float().mean()) > 0.05 for L in info.cache.layers_cuda)  # the crops see the blob
    gout = scenes.upstream_grads(hs, 3)
    loss = sum((im * torch.from_numpy(go).cuda()).sum() for im, go in zip(images, gout))
    loss.backward()
    saved = download_forward(hs, info, [im.detach() for im in images], [])
    refb = oracle_mod.backward(hs, saved, gout, False, True, False)
    np.testing.assert_allclose(scene.texture.grad.cpu().numpy(), refb.grad_texture, rtol=1e-4, atol=1e-6)
    got_pose = scene.tangent_poses.grad.cpu().numpy()
    scale = np.abs(refb.grad_pose).max()
    assert np.abs(got_pose - refb.grad_pose).max() <= 1e-4 * scale
    assert np.abs(got_pose[2]).max() > 0 and not got_pose[[0, 1, 3, 4, 5]].any()  # only the rendered frame's pose
