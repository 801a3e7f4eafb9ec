"""The C++ libTorch wrapper (adop_amd/csrc/torch: PointRendererCache, PointRender autograd function, BlendPointCloud,
PointRenderModuleForward, ApplyTangentToPose) driven through its pybind front end, against the CPU checker."""
import os
import sys

import numpy as np
import pytest

from helpers import announce, assert_close, assert_close_accounted, assert_norm_close, count_misses

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _module():
    sys.path.insert(0, os.path.join(ROOT, "adop_amd", "csrc", "torch"))
    import torch  # noqa: F401  (libtorch must be loaded first)
    import adop_torch

    return adop_torch


def _views(hs):
    return [(v.w, v.h, v.image_index, v.camera_index, v.camera_model_type, v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy,
             v.crop_s) for v in hs.views]


def _params(hs, **extra):
    p = hs.params
    d = dict(test_backward_mode=p.test_backward_mode, check_normal=bool(p.check_normal),
             ghost_gradients=bool(p.ghost_gradients), drop_out_points_by_radius=bool(p.drop_out_points_by_radius),
             depth_accept=p.depth_accept, drop_out_radius_threshold=p.drop_out_radius_threshold,
             dist_cutoff=p.dist_cutoff, distortion_gradient_factor=p.distortion_gradient_factor,
             K_gradient_factor=p.K_gradient_factor, output_background_mask=bool(p.output_background_mask),
             output_background_mask_value=p.output_background_mask_value, normalize_mode=p.normalize_mode)
    d.update(extra)
    return d


def _scene(mod, hs, env=None):
    import torch

    t = dict(
        position=torch.from_numpy(hs.position).cuda().requires_grad_(True),
        normal=None if hs.normal is None else torch.from_numpy(hs.normal).cuda().reshape(-1, 1),
        index=torch.from_numpy(hs.index).cuda().reshape(-1, 1),
        texture=torch.from_numpy(hs.texture).cuda().requires_grad_(True),
        background=torch.from_numpy(hs.background).cuda().requires_grad_(True),
        poses_se3=torch.from_numpy(hs.poses_se3).cuda(),
        tangent_poses=torch.zeros(hs.poses_se3.shape[0], 6, dtype=torch.float64, device="cuda").requires_grad_(True),
        intrinsics=torch.from_numpy(hs.intrinsics).cuda().requires_grad_(True),
    )
    s = mod.Scene(t["position"], t["normal"], t["index"], t["texture"], t["background"], t["poses_se3"],
                  t["tangent_poses"], t["intrinsics"], env)
    return s, t


def test_point_render_autograd_matches_checker(oracle_mod, capfd):
    import torch
    from adop_amd import scenes

    announce("libTorch wrapper: PointRender forward + autograd backward, no dropout, spatial gradients of rendered points")
    mod = _module()
    hs = scenes.config3(n=200_000, w=320, h=180, channels=8)
    hs.dropout = None
    hs.params.ghost_gradients = 0
    hs.params.output_background_mask = 1
    ref = oracle_mod.forward(hs)
    s, t = _scene(mod, hs)
    capfd.readouterr()
    outs = mod.render(s, _views(hs), _params(hs, dropout=0.0, debug_print_num_rendered_points=True), hs.num_layers)
    L = hs.num_layers
    # RenderParams::debug_print_num_rendered_points (PointRenderer.cu:1502-1512): the sum of the weights of all levels
    assert f"# Rasterized Points = {sum(int(a) for a in ref.stats.accepted[:L])}" in capfd.readouterr().out
    assert len(outs) == 2 * L  # images then masks (RenderInfo.cpp:39-41)
    for l in range(L):
        assert_close(outs[l].detach().cpu().numpy(), ref.out[l], 1e-5, 1e-7, f"out {l}")
        # the masks leave PointRender as graph outputs (RenderModule.cpp:77-81 detaches them afterwards)
        assert np.array_equal(outs[L + l].detach().cpu().numpy(), ref.mask[l])
    gout = scenes.upstream_grads(hs, 3)
    loss = sum((o * torch.from_numpy(g).cuda()).sum() for o, g in zip(outs[:L], gout))
    loss.backward()
    refb = oracle_mod.backward(hs, ref, gout)
    # the bars of helpers.check_backward: 1e-4 relative / 1e-6 absolute; the background gradient (a cancelling sum over
    # the empty pixels) with its sqrt(pixels) absolute bar, the elements that need it counted and printed
    assert_close(t["texture"].grad.cpu().numpy(), refb.grad_texture, 1e-4, 1e-6, "grad texture")
    n_pixels = hs.batch * sum(w * h for (w, h) in hs.level_sizes())
    assert_close_accounted(t["background"].grad.cpu().numpy(), refb.grad_background, 1e-4, 1e-6, 1e-4,
                           max(1e-5, 2.4e-7 * np.sqrt(n_pixels)), "grad background", "grad_background",
                           "libTorch wrapper")
    # The checker ran its own forward here (the wrapper keeps its depth / weight buffers to itself), so the spatial
    # gradients see images that differ by summation order: tensor-level bound, and the element-wise bar (1e-4 relative
    # / 1e-6 absolute) with the ceilings of tests/test_parity_gpu.py on how many elements miss it and by how much.
    for name, got, want in (("grad points", t["position"].grad, refb.grad_points),
                            ("grad pose", t["tangent_poses"].grad, refb.grad_pose),
                            ("grad intrinsics", t["intrinsics"].grad, refb.grad_intrinsics)):
        assert_norm_close(got.cpu().numpy(), want, 1e-4, name)
        misses, size, worst = count_misses(got.cpu().numpy(), want)
        assert misses <= max(1, int(1e-4 * size)) and worst <= 1e-6, (name, misses, size, worst)


def test_render_points_switched_off():
    """RenderParams::render_points = false (PointRenderer.cu:1417,1433): background images, masks of the mask value."""
    from adop_amd import scenes

    announce("libTorch wrapper: render_points = false")
    mod = _module()
    hs = scenes.config3(n=50_000, w=160, h=90, channels=4)
    hs.background[:] = [0.1, 0.2, 0.3, 0.4]
    hs.params.output_background_mask = 1
    hs.params.output_background_mask_value = 0.25
    s, t = _scene(mod, hs)
    outs = mod.render(s, _views(hs), _params(hs, dropout=0.25, render_points=False), hs.num_layers)
    L = hs.num_layers
    for l in range(L):
        o = outs[l].detach().cpu().numpy()
        for c in range(4):
            assert (o[:, c] == hs.background[c]).all()
        assert (outs[L + l].detach().cpu().numpy() == 0.25).all()


def test_dropout_is_drawn_like_the_reference_and_eval_disables_it(oracle_mod):
    import torch
    from adop_amd import scenes

    announce("libTorch wrapper: bernoulli_ dropout mask, eval mode -> no dropout")
    mod = _module()
    hs = scenes.config2(n=100_000, w=128, h=128, batch=2)
    s, t = _scene(mod, hs)
    torch.manual_seed(1234)
    outs = mod.render(s, _views(hs), _params(hs, dropout=0.25), hs.num_layers)
    torch.manual_seed(1234)
    mask = torch.empty(2, hs.num_points, device="cuda").bernoulli_(0.25)  # PointRenderer.cu:1083
    hs.dropout = mask.cpu().numpy()
    ref = oracle_mod.forward(hs)
    for l in range(hs.num_layers):
        assert_close(outs[l].detach().cpu().numpy(), ref.out[l], 1e-5, 1e-7, f"out {l}")
    # through the module in eval mode: dropout forced to 0 (RenderModule.cpp:25-28)
    outs = mod.render(s, _views(hs), _params(hs, dropout=0.25), hs.num_layers, training=False, through_module=True)
    hs.dropout = None
    ref = oracle_mod.forward(hs)
    for l in range(hs.num_layers):
        assert_close(outs[l].detach().cpu().numpy(), ref.out[l], 1e-5, 1e-7, f"eval out {l}")


def _host_environment(oracle_mod, hs, env_np, ref, pooled):
    """The reference's composition on the host (RenderModule.cpp:54-127): torch's grid_sample (bilinear, border,
    align_corners) on the checker's uv, images + (1 - mask) * env; `pooled`: 2x2 average pool of a render at twice the
    size first.  Returns per level (image, mask, env sample) as torch tensors with the texture in the autograd graph."""
    import torch

    tex = torch.from_numpy(env_np).clone().requires_grad_(True)
    out = []
    for l in range(hs.num_layers):
        img, m = torch.from_numpy(ref.out[l]), torch.from_numpy(ref.mask[l])
        if pooled:
            img, m = torch.nn.functional.avg_pool2d(img, 2), torch.nn.functional.avg_pool2d(m, 2)
        uv = torch.stack([torch.from_numpy(oracle_mod.env_uv(hs, b, l)) for b in range(hs.batch)])
        e = torch.nn.functional.grid_sample(tex[None].expand(hs.batch, -1, -1, -1), uv, mode="bilinear",
                                            padding_mode="border", align_corners=True)
        out.append((img, m, e))
    return tex, out


@pytest.mark.parametrize("camera", ["pinhole", "ocam"])
@pytest.mark.parametrize("super_sampling", [True, False], ids=["supersampled", "plain"])
def test_module_forward_with_the_environment_map_and_its_gradient(oracle_mod, camera, super_sampling):
    """PointRenderModuleForward composes the environment map through the library's fused kernels
    (torch::autograd::EnvironmentMapCompose): the composed images, and the gradients the loss sends to the map's
    texture and to the descriptors, against torch's grid_sample autograd on the checker's texture coordinates and the
    checker's render.  Pinhole views as the reference, OCam views as the extension; with super-sampling the masks are
    fractional after the 2x2 pool."""
    import copy

    import torch
    from adop_amd import scenes

    announce(f"libTorch wrapper: module forward + backward with the environment map, {camera}, super_sampling={super_sampling}")
    mod = _module()
    if camera == "pinhole":
        hs = scenes.config3(n=100_000, w=160, h=96, channels=4, levels=3)
        hs.views.append(scenes.make_view(160, 96, crop=(1.5, 1.5, -40.0, -30.0, 0.0)))
    else:
        hs = scenes.config5(n=60_000, w=132, h=90, levels=3, batch=2, patches=60, seed=4)
    hs.dropout = None
    hs.params.ghost_gradients = 0
    hs.params.output_background_mask = 1
    env_np = scenes.rng(5).random((4, 32, 64), dtype=np.float32)
    env = torch.from_numpy(env_np).cuda().requires_grad_(True)
    s, t = _scene(mod, hs, env)
    outs = mod.render(s, _views(hs), _params(hs, dropout=0.0, super_sampling=super_sampling), hs.num_layers,
                      training=True, through_module=True)
    L = hs.num_layers
    assert [tuple(o.shape[2:]) for o in outs[:L]] == [(h, w) for (w, h) in hs.level_sizes()]
    hs2 = hs
    if super_sampling:  # render at 2x, 2x2 average pool (RenderModule.cpp:54-104)
        hs2 = copy.copy(hs)
        hs2.views = [scenes.make_view(2 * v.w, 2 * v.h, v.image_index, v.camera_index, v.camera_model_type,
                                      (2 * v.crop_fx, 2 * v.crop_fy, 2 * v.crop_cx, 2 * v.crop_cy, 2 * v.crop_s))
                     for v in hs.views]
    ref = oracle_mod.forward(hs2)
    tex_host, levels = _host_environment(oracle_mod, hs, env_np, ref, super_sampling)
    gout = scenes.upstream_grads(hs, 17)
    loss_host = 0
    for l, (img, m, e) in enumerate(levels):
        want = img + (1 - m) * e
        assert_close(outs[l].detach().cpu().numpy(), want.detach().numpy(), 2e-5, 2e-6, f"module out {l}")
        assert_close(outs[L + l].cpu().numpy(), m.numpy(), 1e-6, 1e-7, f"module mask {l}")
        loss_host = loss_host + (want * torch.from_numpy(gout[l])).sum()
    loss_host.backward()
    sum((o * torch.from_numpy(g).cuda()).sum() for o, g in zip(outs[:L], gout)).backward()
    # texture gradient of the map: per-tile fixed-point sums + one float atomic per texel here, torch's scatter there
    assert_norm_close(env.grad.cpu().numpy(), tex_host.grad.numpy(), 2e-5, "environment map gradient")
    assert_close(env.grad.cpu().numpy(), tex_host.grad.numpy(), 1e-4, 1e-4 * float(tex_host.grad.abs().max()),
                 "environment map gradient, element-wise")
    # the descriptors still receive the rasterizer's gradient through the composition (d composed / d image = 1)
    gout2 = gout
    if super_sampling:
        # the pool's adjoint: a quarter of the upstream gradient to each of the four pixels; a last odd row or column
        # of the large image is dropped by the pool and receives nothing
        gout2 = []
        for g, (w2, h2) in zip(gout, hs2.level_sizes()):
            big = np.zeros(g.shape[:2] + (h2, w2), np.float32)
            big[:, :, : 2 * g.shape[2], : 2 * g.shape[3]] = np.repeat(np.repeat(g, 2, axis=2), 2, axis=3) * np.float32(0.25)
            gout2.append(big)
    refb = oracle_mod.backward(hs2, ref, gout2)
    assert_close(t["texture"].grad.cpu().numpy(), refb.grad_texture, 1e-4, 1e-6, "grad texture through the composition")


def test_module_forward_cat_env_to_color(oracle_mod):
    """PipelineParams::cat_env_to_color (RenderModule.cpp:112-118): the sampled map of every pixel is concatenated to
    the image instead of composed; its texture gradient then carries no (1 - mask) factor."""
    import torch
    from adop_amd import scenes

    announce("libTorch wrapper: module forward with cat_env_to_color")
    mod = _module()
    hs = scenes.config3(n=60_000, w=96, h=64, channels=4, levels=2)
    hs.dropout = None
    hs.params.ghost_gradients = 0
    hs.params.output_background_mask = 1
    env_np = scenes.rng(6).random((4, 16, 32), dtype=np.float32)
    env = torch.from_numpy(env_np).cuda().requires_grad_(True)
    s, t = _scene(mod, hs, env)
    outs = mod.render(s, _views(hs), _params(hs, dropout=0.0), hs.num_layers, training=True, through_module=True,
                      cat_env_to_color=True)
    L = hs.num_layers
    ref = oracle_mod.forward(hs)
    tex_host, levels = _host_environment(oracle_mod, hs, env_np, ref, False)
    g = scenes.rng(3)
    loss_host = 0
    loss = 0
    for l, (img, m, e) in enumerate(levels):
        assert outs[l].shape[1] == 8
        assert_close(outs[l][:, :4].detach().cpu().numpy(), img.numpy(), 1e-5, 1e-7, f"image part {l}")
        assert_close(outs[l][:, 4:].detach().cpu().numpy(), e.detach().numpy(), 2e-5, 2e-6, f"environment part {l}")
        go = torch.from_numpy(g.standard_normal(e.shape).astype(np.float32))
        loss_host = loss_host + (e * go).sum()
        loss = loss + (outs[l][:, 4:] * go.cuda()).sum()
    loss_host.backward()
    loss.backward()
    assert_norm_close(env.grad.cpu().numpy(), tex_host.grad.numpy(), 2e-5, "environment map gradient (cat)")


def test_stage_timer_system_receives_the_stage_times(oracle_mod):
    """NeuralRenderInfo::timer_system (PointRenderer.h:32): with a timer system attached the stages of a forward and a
    backward pass arrive under the reference's names (SAIGA_OPTIONAL_TIME_MEASURE, PointRenderer.cu:906-1610), frame by
    frame; without one nothing is recorded."""
    import torch
    from adop_amd import scenes

    announce("libTorch wrapper: stage timers through NeuralRenderInfo::timer_system")
    mod = _module()
    hs = scenes.config3(n=200_000, w=640, h=360, channels=8)
    hs.dropout = None
    s, t = _scene(mod, hs)
    params = _params(hs, dropout=0.25)
    for frame in range(3):
        s.begin_frame()
        outs = mod.render(s, _views(hs), params, hs.num_layers, timed=True)
        sum(o.sum() for o in outs[: hs.num_layers]).backward()
        s.end_frame()
    times = s.stage_times()
    forward = {"Initialize", "CombineAndFill"}
    backward = {"Prepare Backward", "CombineAndFillBackward", "RenderBackward/descriptor", "RenderBackward/spatial",
                "Post Process Gradient"}
    assert forward | backward <= set(times), sorted(times)
    assert ({"DepthPrepass", "RenderForward"} <= set(times)) or ({"BinCount", "BinScatter", "TileDepth", "TileBlend"} <= set(times))
    for name, (last_ms, total_ms, calls, frames) in times.items():
        assert frames == 3 and calls >= 3 and 0 < last_ms < 50 and total_ms >= last_ms, (name, last_ms, total_ms, calls, frames)
    # a frame without a timer system adds nothing
    s.begin_frame()
    mod.render(s, _views(hs), params, hs.num_layers)
    s.end_frame()
    assert all(v[3] == 3 for v in s.stage_times().values())


def test_apply_tangent(oracle_mod):
    import torch
    from adop_amd import scenes

    announce("libTorch wrapper: PoseModule::ApplyTangent")
    mod = _module()
    hs = scenes.config1(n=10, w=16, h=16, levels=1)
    s, t = _scene(mod, hs)
    with torch.no_grad():
        t["tangent_poses"][0] = torch.tensor([0.1, -0.2, 0.05, 0.02, 0.01, -0.03], dtype=torch.float64)
    tang, want = oracle_mod.apply_tangent(t["tangent_poses"].detach().cpu().numpy(), hs.poses_se3)
    with torch.no_grad():
        s.apply_tangent()
    torch.cuda.synchronize()
    assert np.abs(t["poses_se3"].cpu().numpy() - want).max() < 1e-12
    assert float(t["tangent_poses"].detach().abs().sum()) == 0


def test_scene_data_processing_in_cpp():
    """SceneDataHip.cpp (the point-cloud processing of a new scene over libTorch tensors) gives what the ctypes mirror
    gives, which the preprocessing tests hold against the checker."""
    import torch
    from adop_amd import preprocess, scenes

    mod = _module()
    g = np.random.default_rng(6)
    n = 30000
    p = np.zeros((n, 4), np.float32)
    p[:, :3] = g.standard_normal((n, 3)) * 0.6
    p[1000:1300, :3] = p[:300, :3] + np.float32(2e-6)  # near-duplicates for the close-point filter
    announce("C++ scene data processing: N=30000, 9 frames")
    pos = torch.from_numpy(p).cuda()
    assert torch.equal(mod.knn_distance(pos, 4), preprocess.KNearestNeighbourDistance(pos, 4))
    assert torch.equal(mod.knn_distance(pos, 7), preprocess.KNearestNeighbourDistance(pos, 7))
    assert torch.equal(mod.morton_codes(pos), preprocess.MortonCodes(pos))
    assert torch.equal(mod.reorder_morton64(pos), preprocess.ReorderMorton64(pos))
    views = np.stack([scenes.look_at_view(3.0 * d / np.linalg.norm(d)) for d in g.standard_normal((9, 3))])
    K = scenes.pinhole_row(300, 300, 160, 120, 0.0, [0.05, -0.01, 0.002, 0.0, 0.0, 0.0, 0.001, 0.0])[None, :]
    frames = [scenes.make_view(320, 240, image_index=f) for f in range(9)]
    tuples = [(v.w, v.h, v.image_index, v.camera_index, v.camera_model_type, v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy,
               v.crop_s) for v in frames]
    poses, intr = torch.from_numpy(views).cuda(), torch.from_numpy(K).cuda()
    cam = mod.point_distance_to_camera(pos, poses, intr, tuples)
    assert torch.equal(cam, preprocess.PointDistanceToCamera(pos, poses, intr, frames))
    assert torch.equal(mod.remove_lonely_points(pos, cam, 5, 0.05), preprocess.RemoveLonelyPoints(pos, cam, 5, 0.05))
    keep = mod.remove_close_points(pos, cam, 0.00005)
    assert torch.equal(keep, preprocess.RemoveClosePoints(pos, cam, 0.00005))
    assert 250 <= int((~keep).sum()) <= 320
    radius = torch.rand(n, device="cuda")
    assert torch.equal(mod.sort_blocks_by_radius(radius, 256), preprocess.SortBlocksByRadius(radius, 256))
    # the two compositions of SceneData.cpp:98-104 in C++: the filters, and the processing of what they leave
    assert torch.equal(mod.filter_point_cloud(pos, poses, intr, tuples), preprocess.FilterPointCloud(pos, poses, intr, frames))
    nrm = torch.randint(0, 1 << 30, (n, 1), dtype=torch.int32, device="cuda")
    got = mod.preprocess_point_cloud(pos, nrm, 4, 256, 3)
    want = preprocess.PreprocessPointCloud(pos, nrm, 4, 256, 3)
    for a, b, what in zip(got, want, ("position", "normal", "data", "order")):
        assert torch.equal(a, b), what
    assert bool((got[0][:, 3] > 0).all()) and sorted(got[3].tolist()) == list(range(n))
    with pytest.raises(RuntimeError):
        mod.knn_distance(pos[:3], 4)
