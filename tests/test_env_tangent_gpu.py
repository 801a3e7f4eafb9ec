"""GPU parity of the environment-map entry points (EnvironmentMap.cu:41-157 + RenderModule.cpp:106-127) and of
ApplyTangentToPose (PointRenderer.cu:1646-1665), through the C-ABI."""
import os

import numpy as np
import pytest

from helpers import announce, assert_close, assert_norm_close, run_hip_forward

pytestmark = pytest.mark.gpu


def _env_scene():
    from adop_amd import scenes

    hs = scenes.config3(n=100_000, w=200, h=120, channels=4, levels=3)
    hs.intrinsics[0, 5:] = [0.03, -0.01, 0.002, 0.005, 0.001, -0.0005, 0.0008, -0.001]
    hs.params.output_background_mask = 1
    hs.params.output_background_mask_value = 0.0
    hs.env_texture = scenes.rng(17).random((4, 64, 128), dtype=np.float32)
    # a second view from another pose, cropped
    hs.poses_se3 = np.stack([hs.poses_se3[0], scenes.look_at_view((2.0, 1.5, 1.8))])
    hs.views.append(scenes.make_view(200, 120, image_index=1, crop=(0.8, 0.8, 10.0, -5.0, 0.0)))
    hs.dropout = scenes.bernoulli_mask(3, 2, hs.num_points, 0.25)
    return hs


def _check_sampling_and_composition(oracle_mod, hs, min_empty=1000):
    """uv and samples of every pixel against the checker; the composition in place and out of place."""
    import torch
    from adop_amd import render

    scene, info, ctx, images, masks = run_hip_forward(hs)
    before = [im.clone() for im in images]
    uv, env = render.EnvironmentMapSample(info, add_to_out=False, want_uv=True, want_env=True)
    torch.cuda.synchronize()
    empty = 0
    for l in range(hs.num_layers):
        assert bool((images[l] == before[l]).all())
        for b in range(hs.batch):
            want_uv = oracle_mod.env_uv(hs, b, l)
            got_uv = uv[l][b].cpu().numpy()
            # (far outside a strongly distorted image the five-step undistortion leaves the range of fp32: the same
            # pixels in the checker; grid_sample's clamp, written with fmin / fmax as the CUDA sampler's, takes a NaN
            # to texel 0)
            fin = np.isfinite(want_uv).all(axis=-1)
            assert np.array_equal(np.isfinite(got_uv).all(axis=-1), fin), (l, b)
            assert fin.mean() > 0.9
            assert np.abs(got_uv - want_uv)[fin].max() <= 1e-6, (l, b, np.abs(got_uv - want_uv)[fin].max())
            # sampling of the HIP uv with the checker's bilinear rule
            want_env = oracle_mod.grid_sample(hs.env_texture, got_uv)
            assert_close(env[l][b].cpu().numpy(), want_env, 1e-5, 1e-6, f"env level {l} view {b}")
        # library cross-check: torch grid_sample on the same uv
        grid = torch.nan_to_num(uv[l].cpu(), nan=-1.0, posinf=1.0, neginf=-1.0)
        ref = torch.nn.functional.grid_sample(torch.from_numpy(hs.env_texture)[None].repeat(hs.batch, 1, 1, 1),
                                              grid, mode="bilinear", padding_mode="border", align_corners=True)
        assert_close(env[l].cpu().numpy(), ref.numpy(), 1e-5, 2e-6, f"env vs torch level {l}")
        empty += int((masks[l] == 0).sum())
    assert empty > min_empty  # the scene leaves pixels for the environment map
    # out of place (as the reference composes, RenderModule.cpp:121-125): the rasterizer's images stay as they are
    _, composed = render.EnvironmentMapSample(info, add_to_out=2)
    torch.cuda.synchronize()
    for l in range(hs.num_layers):
        m = masks[l].cpu().numpy()
        want = before[l].cpu().numpy() + (1 - m) * env[l].cpu().numpy()
        assert_close(composed[l].cpu().numpy(), want, 1e-6, 1e-7, f"composition out of place, level {l}")
        assert bool((images[l] == before[l]).all())
    # in place: the same numbers in the images; uv and samples only where the composition samples
    uv1 = [torch.full_like(u, float("nan")) for u in uv]
    fb = info.cache.forward_struct()
    import ctypes as C
    L = hs.num_layers
    env1 = [torch.full_like(e, 7.0) for e in env]
    s = scene.struct()
    tex = scene.environment_map
    rc = info.cache.lib.adop_env_sample(C.byref(s), info.cache.views_array(), hs.batch, C.c_void_p(tex.data_ptr()),
                                        int(tex.shape[1]), int(tex.shape[2]), C.byref(fb),
                                        (C.c_void_p * L)(*[t.data_ptr() for t in uv1]),
                                        (C.c_void_p * L)(*[t.data_ptr() for t in env1]), 1, None)
    assert rc == 0
    torch.cuda.synchronize()
    for l in range(L):
        assert bool((images[l] == composed[l]).all()), l
        m = masks[l]
        sampled = (m == 0)
        assert bool(torch.isnan(uv1[l][~sampled[:, 0]]).all())
        same_bits = uv1[l][sampled[:, 0]].view(torch.int32) == uv[l][sampled[:, 0]].view(torch.int32)  # (a NaN is a NaN)
        assert bool(same_bits.all())
        assert bool((env1[l] == torch.where(sampled.expand_as(env[l]), env[l], torch.zeros_like(env[l]))).all())
    return scene, info, masks, uv1


def test_env_uv_sample_and_composition(oracle_mod):
    announce("environment map: uv, bilinear sample, composition in place and out of place")
    _check_sampling_and_composition(oracle_mod, _env_scene())


def test_env_backward_matches_autograd_of_grid_sample():
    import torch
    from adop_amd import render, scenes

    announce("environment map: gradient w.r.t. the texture")
    hs = _env_scene()
    scene, info, ctx, images, masks = run_hip_forward(hs)
    uv, env = render.EnvironmentMapSample(info, add_to_out=False, want_uv=True, want_env=False)
    gout = [torch.from_numpy(g).cuda() for g in scenes.upstream_grads(hs, 9)]
    g_env = render.EnvironmentMapSampleBackward(info, gout, uv=uv)
    torch.cuda.synchronize()
    tex = torch.from_numpy(hs.env_texture).double().requires_grad_(True)
    loss = 0
    for l in range(hs.num_layers):
        s = torch.nn.functional.grid_sample(tex[None].repeat(hs.batch, 1, 1, 1), uv[l].cpu().double(), mode="bilinear",
                                            padding_mode="border", align_corners=True)
        loss = loss + (s * (1 - masks[l].cpu().double()) * gout[l].cpu().double()).sum()
    loss.backward()
    # every texel sums hundreds of N(0,1)-weighted terms with fp32 atomics; autograd here runs in f64:
    # bound the error against the size of the sums (tensor-level), not against each cancelled result
    assert_norm_close(g_env.cpu().numpy(), tex.grad.numpy(), 2e-5, "grad env texture")


def _ocam_env_scene():
    from adop_amd import _capi, scenes

    hs = scenes.config5(n=60_000, w=176, h=120, levels=3, batch=2, patches=40, env_hw=(48, 96))
    # an affine part, so that the inverse has to undo it; the second view is a crop window of the same camera
    hs.intrinsics[0, :3] = [1.03, 0.02, -0.015]
    hs.views[1] = scenes.make_view(176, 120, image_index=1, model=_capi.CAMERA_OCAM, crop=(1.25, 1.25, -30.0, -12.0, 0.0))
    hs.params.output_background_mask_value = 0.0
    hs.dropout = scenes.bernoulli_mask(5, 2, hs.num_points, 0.25)
    return hs


def test_env_on_ocam_views(oracle_mod):
    """Environment map on OCam views (an extension: the reference asserts pinhole, EnvironmentMap.cu:129): the ray of
    a pixel comes from the inverted world2cam polynomial."""
    import torch
    from adop_amd import render, scenes

    announce("environment map on OCam views: uv, sample, composition, texture gradient")
    hs = _ocam_env_scene()
    scene, info, masks, uv = _check_sampling_and_composition(oracle_mod, hs)
    # (uv holds coordinates at the sampled pixels only, NaN elsewhere: the backward pass must not read those)
    gout = [torch.from_numpy(g).cuda() for g in scenes.upstream_grads(hs, 9)]
    g_env = render.EnvironmentMapSampleBackward(info, gout)
    g_env_uv = render.EnvironmentMapSampleBackward(info, gout, uv=uv)  # the coordinates kept from the forward call
    torch.cuda.synchronize()
    tex = torch.from_numpy(hs.env_texture).double().requires_grad_(True)
    loss = 0
    for l in range(hs.num_layers):
        grid = torch.nan_to_num(uv[l].cpu().double(), nan=0.0)
        s = torch.nn.functional.grid_sample(tex[None].repeat(hs.batch, 1, 1, 1), grid, mode="bilinear",
                                            padding_mode="border", align_corners=True)
        loss = loss + (s * (1 - masks[l].cpu().double()) * gout[l].cpu().double()).sum()
    loss.backward()
    assert_norm_close(g_env.cpu().numpy(), tex.grad.numpy(), 2e-5, "grad env texture (OCam)")
    assert_norm_close(g_env_uv.cpu().numpy(), tex.grad.numpy(), 2e-5, "grad env texture (OCam, uv from the forward call)")
    # the sums are integer sums per tile: the same inputs give the same bits, and the kept coordinates are the inputs
    assert_norm_close(g_env_uv.cpu().numpy(), g_env.cpu().numpy(), 1e-6, "grad env texture: kept uv vs computed uv")


def _random_env_scene(seed):
    from adop_amd import _capi, scenes

    g = np.random.default_rng(5100 + seed)
    levels = int(g.integers(1, 6))
    w = int(g.integers(max(20, 1 << (levels - 1)), 260))
    h = int(g.integers(max(20, 1 << (levels - 1)), 200))
    batch = int(g.integers(1, 4))
    ocam = g.random() < 0.4
    eh, ew = int(g.integers(2, 90)), int(g.integers(2, 150))  # also taller than wide, as the reference's default map
    if ocam:
        hs = scenes.config5(n=20_000, w=w, h=h, levels=levels, batch=batch, patches=20, seed=seed, env_hw=(eh, ew))
        if g.random() < 0.5:
            hs.intrinsics[0, :3] = [float(g.uniform(0.95, 1.05)), float(g.uniform(-0.03, 0.03)), float(g.uniform(-0.03, 0.03))]
        model = _capi.CAMERA_OCAM
    else:
        hs = scenes.config2(n=20_000, w=w, h=h, levels=levels, batch=batch, seed=seed)
        if g.random() < 0.6:
            hs.intrinsics[0, 5:] = g.uniform(-1.0, 1.0, 8) * [0.05, 0.02, 0.005, 0.02, 0.01, 0.002, 0.002, 0.002]
        if g.random() < 0.3:
            hs.intrinsics[0, 4] = g.uniform(-0.2, 0.2)  # shear
        model = _capi.CAMERA_PINHOLE_DISTORTION
    C = int(g.choice([1, 3, 4, 8]))
    hs.texture = g.random((C, hs.num_points), dtype=np.float32)
    hs.background = g.random(C, dtype=np.float32)
    hs.env_texture = g.random((C, eh, ew), dtype=np.float32)
    for k, v in enumerate(hs.views):
        if g.random() < 0.5:
            sc = float(g.uniform(0.6, 2.0))
            hs.views[k] = scenes.make_view(w, h, image_index=v.image_index, camera_index=v.camera_index, model=model,
                                           crop=(sc, sc, float(g.uniform(-0.8, 0.1) * w), float(g.uniform(-0.8, 0.1) * h), 0.0))
    hs.params.output_background_mask = 1
    hs.params.output_background_mask_value = 0.0
    hs.dropout = scenes.bernoulli_mask(seed, batch, hs.num_points, 0.5)
    what = f"seed {seed}: {w}x{h} L={levels} B={batch} C={C} {'ocam' if ocam else 'pinhole'} map {ew}x{eh}"
    return hs, what


# (ADOP_ENV_SWEEP_SEEDS="first:count" draws other scenes than the 24 of a default run)
_first, _count = (int(x) for x in os.environ.get("ADOP_ENV_SWEEP_SEEDS", "0:24").split(":"))
_seeds = list(range(_first, _first + _count))
if "ADOP_ENV_SWEEP_SEEDS" not in os.environ:
    _seeds += [86, 148]  # a few pixels of these have coordinates that are not finite (in the checker too)


@pytest.mark.parametrize("seed", _seeds)
def test_env_random_scenes(oracle_mod, seed):
    """Randomly drawn image sizes (not multiples of the 16 x 16 tiles of the backward kernel), level counts, views with
    crop windows, camera models, channel counts and map sizes: coordinates, samples, both compositions against the
    checker, the texture gradient against autograd of grid_sample in f64."""
    import torch
    from adop_amd import render, scenes

    hs, what = _random_env_scene(seed)
    announce("environment map, " + what)
    scene, info, masks, uv = _check_sampling_and_composition(oracle_mod, hs, min_empty=0)
    gout = [torch.from_numpy(g).cuda() for g in scenes.upstream_grads(hs, seed + 9)]
    g_env = render.EnvironmentMapSampleBackward(info, gout)
    g_env_uv = render.EnvironmentMapSampleBackward(info, gout, uv=uv)
    torch.cuda.synchronize()
    tex = torch.from_numpy(hs.env_texture).double().requires_grad_(True)
    loss = 0
    for l in range(hs.num_layers):
        grid = torch.nan_to_num(uv[l].cpu().double(), nan=-1.0, posinf=1.0, neginf=-1.0)
        s = torch.nn.functional.grid_sample(tex[None].repeat(hs.batch, 1, 1, 1), grid, mode="bilinear",
                                            padding_mode="border", align_corners=True)
        loss = loss + (s * (1 - masks[l].cpu().double()) * gout[l].cpu().double()).sum()
    loss.backward()
    assert_norm_close(g_env.cpu().numpy(), tex.grad.numpy(), 2e-5, "grad env texture")
    assert_norm_close(g_env_uv.cpu().numpy(), tex.grad.numpy(), 2e-5, "grad env texture (uv from the forward call)")


def test_env_rejects_unknown_model_and_bad_rows():
    import ctypes as C
    from adop_amd import _capi, scenes

    announce("environment map: argument checks of the camera model")
    hs = scenes.config5(n=1000, w=44, h=30, batch=1, patches=10)
    scene, info, ctx, images, masks = run_hip_forward(hs)
    cache = info.cache
    s = scene.struct()
    fb = cache.forward_struct()
    env = scene.environment_map
    views = cache.views_array()
    views[0].camera_model_type = 7
    rc = cache.lib.adop_env_sample(C.byref(s), views, 1, C.c_void_p(env.data_ptr()), int(env.shape[1]),
                                   int(env.shape[2]), C.byref(fb), None, None, 1, None)
    assert rc == _capi.ADOP_INVALID_ARG
    # a pinhole view needs rows of 13 floats; this scene's rows are OCam rows of 11
    views[0].camera_model_type = _capi.CAMERA_PINHOLE_DISTORTION
    rc = cache.lib.adop_env_sample(C.byref(s), views, 1, C.c_void_p(env.data_ptr()), int(env.shape[1]),
                                   int(env.shape[2]), C.byref(fb), None, None, 1, None)
    assert rc == _capi.ADOP_INVALID_ARG


def test_apply_tangent(oracle_mod):
    import torch
    from adop_amd import render, scenes

    announce("ApplyTangentToPose")
    g = scenes.rng(4)
    F = 300
    q = g.standard_normal((F, 4))
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    poses = np.concatenate([q, g.uniform(-3, 3, (F, 3)), np.zeros((F, 1))], axis=1)
    tang = g.standard_normal((F, 6)) * g.choice([1e-12, 1e-4, 0.1, 1.5], (F, 1))
    t_ref, p_ref = oracle_mod.apply_tangent(tang, poses)
    t = torch.from_numpy(tang.copy()).cuda()
    p = torch.from_numpy(poses.copy()).cuda()
    render.ApplyTangentToPose(t, p)
    torch.cuda.synchronize()
    assert (t == 0).all()
    assert np.abs(p.cpu().numpy() - p_ref).max() < 1e-12
