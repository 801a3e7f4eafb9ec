"""GPU parity: the HIP path (through the C-ABI) against the CPU checker on identical seeded scenes.

Bars: depth / index buffers and weights bit-exact; blended descriptors within 1e-5 relative; gradients within
1e-4 relative or 1e-6 absolute.
"""
import ctypes

import numpy as np
import pytest

from helpers import (announce, assert_norm_close, check_backward, check_forward, download_forward,
                     run_hip_forward)

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=[1, 2], ids=["direct", "tiles"])
def forward_path(request):
    """Every case runs through both forward paths of the library."""
    import helpers

    helpers.FORWARD_PATH = request.param
    yield request.param
    helpers.FORWARD_PATH = 0


def _torch_grads(grads):
    import torch

    return [torch.from_numpy(g).cuda() for g in grads]


# Ceilings of the end-to-end check in _fwd_bwd: share of a gradient tensor's elements that may miss the element-wise
# bar when the checker runs its own forward, and how far such an element may be off, relative to the tensor's largest
# magnitude.  Measured on every case of this file (printed by its last test): only grad_points has such elements,
# at most 2.5e-5 of them (30 of 1.2 M, the OCam case), each off by at most 5e-8 of the tensor's largest magnitude.
END_TO_END_MISS_SHARE = 1e-4
END_TO_END_MISS_SIZE = 1e-6
end_to_end_misses = {}  # case -> {tensor: (misses, size, worst)}: printed by the last test of the file


def _fwd_bwd(hs, oracle_mod, needs=(True, True, True), seed=5, collect_stats=True, poison=False, pixel_records=True,
             workspace_flags=0):
    import torch
    from adop_amd import render, scenes

    from helpers import count_misses

    ref = oracle_mod.forward(hs)
    scene, info, ctx, images, masks = run_hip_forward(hs, collect_stats=collect_stats, poison=poison,
                                                      pixel_records=pixel_records, workspace_flags=workspace_flags)
    check_forward(hs, ref, ctx, images, masks, info, stats=collect_stats)
    gout = scenes.upstream_grads(hs, seed)
    grads = render.BlendPointCloudBackward(ctx, info, _torch_grads(gout), needs)
    torch.cuda.synchronize()
    # (a) backward from the same saved variables the HIP backward consumed: element-wise bar
    saved = download_forward(hs, info, images, masks)
    refb = oracle_mod.backward(hs, saved, gout, *needs)
    check_backward(hs, refb, grads, info, stats=collect_stats)
    # (b) backward from the checker's own forward: the blended image differs by fp32 summation order (<=1e-5), which
    # cancellation in the ghost gradient amplifies for a few points.  Tensor-level bound, and the element-wise bar
    # (1e-4 relative / 1e-6 absolute) with a ceiling on how many elements miss it and by how much.
    refb2 = oracle_mod.backward(hs, ref, gout, *needs)
    names = ["grad_texture", "grad_background", "grad_points", "grad_pose", "grad_intrinsics"]
    rec = {}
    for name, g in zip(names, grads):
        if g is not None:
            want = getattr(refb2, name)
            assert_norm_close(g.cpu().numpy(), want, 1e-4, name + " (checker forward)")
            misses, size, worst = count_misses(g.cpu().numpy(), want)
            rec[name] = (misses, size, worst)
            assert misses <= max(1, int(END_TO_END_MISS_SHARE * size)), (name, misses, size, worst)
            assert worst <= END_TO_END_MISS_SIZE, (name, misses, size, worst)
    end_to_end_misses[f"{hs.name} N={hs.num_points} B={hs.batch} #{len(end_to_end_misses)}"] = rec
    return ref, refb


def test_config1_forward(oracle_mod):
    from adop_amd import scenes

    announce("config1 100k pts 256x256 L4 forward")
    hs = scenes.config1()
    ref = oracle_mod.forward(hs)
    scene, info, ctx, images, masks = run_hip_forward(hs)
    check_forward(hs, ref, ctx, images, masks, info)
    # known answer: untouched pixels keep bits(100000.f) | 0xFFFFFFFF
    di = info.cache.layers_cuda[0].depth_index_tensor.cpu().numpy().view(np.uint64)
    empty = ref.weight[0] == 0
    assert (di[empty & (ref.depth[0] == 100000.0)] == ((0x47C35000 << 32) | 0xFFFFFFFF)).all()


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_forward_without_point_cache_dense_cloud(oracle_mod, collect_stats):
    """Inference (no backward pass follows, the caller keeps no point cache): the direct path hands the blend
    compacted lists of the points that can still pass a depth test.  ~24 points per level-0 pixel, a dropout mask,
    two views; without the counters only the candidates are listed, with them every projected point."""
    from adop_amd import scenes

    announce(f"400k pts B=2 128x128 L4 forward without point cache, dropout 0.3, counters={collect_stats}")
    hs = scenes.config2(n=400_000, w=128, h=128, batch=2)
    hs.dropout = scenes.bernoulli_mask(11, 2, 400_000, 0.3)
    ref = oracle_mod.forward(hs)
    scene, info, ctx, images, masks = run_hip_forward(hs, collect_stats=collect_stats, train=False)
    assert info.cache.point_cache is None
    check_forward(hs, ref, ctx, images, masks, info, stats=collect_stats)


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_config2_forward_backward(oracle_mod, collect_stats):
    """Without the counters (how the wrappers and the benchmark call the library) the kernels compile to other
    variants: both are held to the checker; the plain run starts from a poisoned point cache and workspace."""
    from adop_amd import scenes

    announce(f"config2 1M pts B=4 512x512 L4 fwd+bwd ghost, counters={collect_stats}")
    hs = scenes.config2()
    _fwd_bwd(hs, oracle_mod, needs=(True, True, True), collect_stats=collect_stats, poison=not collect_stats)


def test_config2_no_ghost(oracle_mod):
    from adop_amd import scenes

    announce("config2 200k pts B=2 256x256 no ghost, no dropout")
    hs = scenes.config2(n=200_000, w=256, h=256, batch=2, ghost=False)
    _fwd_bwd(hs, oracle_mod, needs=(True, False, False))


@pytest.mark.parametrize("pixel_records", [True, False], ids=["records_from_forward", "records_from_out"])
@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_config3_reduced_all_grads(oracle_mod, collect_stats, pixel_records):
    """pixel_records: the forward pass leaves the resolved images pixel by pixel for the spatial gradients
    (adop_forward_buffers.pixel_cache), or the backward pass builds those records from `out`."""
    from adop_amd import scenes

    announce(f"config3 reduced 500k pts 480x270 C=8 all grads, counters={collect_stats}, pixel records from the "
             f"forward pass={pixel_records}")
    hs = scenes.config3(n=500_000, w=480, h=270)
    _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats, pixel_records=pixel_records)


@pytest.mark.parametrize("channels", [3, 4])
def test_backward_reads_the_image_the_forward_rendered(oracle_mod, channels):
    """With pixel records kept from the forward pass, the image I of the spatial gradients is what that forward
    rendered, whatever happened to `out` since (the reference composes the environment map out of place,
    RenderModule.cpp:121-125, so its backward sees the rasterizer's own output too); without them it is `out` as it
    is when the backward pass runs.  Three views, so that the records of all images and levels are addressed."""
    import torch
    from adop_amd import render, scenes

    announce(f"backward after `out` was changed in place, C={channels}")
    hs = scenes.config2(n=60_000, w=160, h=120, levels=3, batch=3, seed=6)
    hs.texture = np.ascontiguousarray(np.random.default_rng(1).random((channels, hs.num_points), dtype=np.float32))
    hs.background = np.zeros(channels, np.float32)
    gout = scenes.upstream_grads(hs, 5)
    for kept in (True, False):
        scene, info, ctx, images, masks = run_hip_forward(hs, pixel_records=kept)
        rendered = download_forward(hs, info, images, masks)
        for im in images:
            im.mul_(0.5).add_(0.25)  # (an environment map added in place, a tone curve, ...)
        torch.cuda.synchronize()
        changed = download_forward(hs, info, images, masks)
        grads = render.BlendPointCloudBackward(ctx, info, _torch_grads(gout), (True, True, True))
        torch.cuda.synchronize()
        refb = oracle_mod.backward(hs, rendered if kept else changed, gout, True, True, True)
        check_backward(hs, refb, grads, info)


def test_backward_without_point_gradients(oracle_mod):
    """No point gradient is asked for: nothing normalises point rows, the reduction of the pose / intrinsics /
    background partial sums runs as a kernel of its own."""
    from adop_amd import scenes

    announce("config3 reduced 150k pts 320x180 C=8, gradients: descriptors, pose, intrinsics (no points)")
    hs = scenes.config3(n=150_000, w=320, h=180)
    _fwd_bwd(hs, oracle_mod, needs=(False, True, True))


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_render_points_switched_off(oracle_mod, collect_stats):
    """RenderParams::render_points = false (PointRenderer.cu:1417,1433): the forward pass leaves the cloud out, every
    pixel holds the background; the backward pass still runs over the cloud (:1598-1604) against the empty depth and
    weight buffers, where only dropped points receive a (ghost) gradient."""
    from adop_amd import scenes

    announce(f"config3 reduced 100k pts 240x136, render_points = false, counters={collect_stats}")
    hs = scenes.config3(n=100_000, w=240, h=136, channels=4)
    hs.params.skip_points = 1
    hs.params.output_background_mask = 1
    hs.background[:] = [0.1, 0.2, 0.3, 0.4]
    ref = oracle_mod.forward(hs)
    assert all(float(w.max()) == 0.0 for w in ref.weight) and float(ref.out[0][0, 2].min()) == np.float32(0.3)
    _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats)


def test_empty_cloud(oracle_mod):
    """No points at all (the pointers of the cloud are NULL): background images, background gradient, empty gradients."""
    from adop_amd import scenes

    announce("config2 without points, B=2 96x80 L3 fwd+bwd")
    hs = scenes.config2(n=1000, w=96, h=80, levels=3, batch=2)
    hs.position, hs.normal, hs.index = hs.position[:0].copy(), hs.normal[:0].copy(), hs.index[:0].copy()
    hs.dropout = None
    hs.params.output_background_mask = 1
    hs.background[:] = [0.5, 0.25, 0.125, 1.0]
    assert hs.num_points == 0
    _fwd_bwd(hs, oracle_mod)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("coefficients", [1, 2, 6, 19])
def test_ocam_cameras_with_other_polynomials(oracle_mod, coefficients, mode):
    """Three OCam cameras (rows of 5 + P floats; P = 19 fills the widest row the library takes), five views spread
    over them, both normalisation modes (mode 0 divides the intrinsics gradient as rows of 13 floats whatever the row
    width, PointRenderer.cu:1633)."""
    from adop_amd import scenes

    P, K = coefficients, 3
    announce(f"OCam, {K} cameras with {P} polynomial coefficients, 5 views, normalize_mode={mode}")
    hs = scenes.config5(n=60_000, w=176, h=120, levels=3, batch=5, patches=40, seed=P)
    hs.env_texture = None
    row = hs.intrinsics[0]
    intr = np.zeros((K, 5 + P), np.float32)
    for k in range(K):
        intr[k, :5] = row[:5] + np.array([0.01 * k, 0.002 * k, -0.003 * k, 2.0 * k, -1.5 * k], np.float32)
        m = min(P, 6)
        intr[k, 5:5 + m] = row[5:5 + m] * (1 + 0.02 * k)
        if P > 6:
            intr[k, 11:] = np.random.default_rng(P + k).uniform(-0.05, 0.05, P - 6)
    hs.intrinsics = intr
    for i, v in enumerate(hs.views):
        v.camera_index = i % K
    hs.dropout = scenes.bernoulli_mask(3, 5, hs.num_points, 0.3)
    hs.params.ghost_gradients = 1
    hs.params.normalize_mode = mode
    _fwd_bwd(hs, oracle_mod)


@pytest.mark.parametrize("mode", [0, 1])
def test_pinhole_cameras_shared_by_views(oracle_mod, mode):
    """Three pinhole cameras with intrinsics and distortion of their own, six views over four frames: the pose and
    intrinsics gradients of views that share a frame or a camera add up in the order of the views."""
    from adop_amd import scenes

    announce(f"pinhole, 3 cameras, 6 views over 4 frames, normalize_mode={mode}")
    hs = scenes.config2(n=80_000, w=160, h=120, levels=3, batch=6, seed=3)
    K = 3
    intr = np.repeat(hs.intrinsics, K, axis=0).copy()
    g = np.random.default_rng(1)
    for k in range(K):
        intr[k, :4] *= 1 + 0.05 * k
        intr[k, 5:] = g.uniform(-1, 1, 8) * [0.05, 0.02, 0.005, 0.02, 0.01, 0.002, 0.002, 0.002]
    hs.intrinsics = intr
    for i, v in enumerate(hs.views):
        v.camera_index = (2 * i) % K
        v.image_index = i % 4
    hs.params.normalize_mode = mode
    _fwd_bwd(hs, oracle_mod)


def test_debug_print_num_rendered_points(oracle_mod, capsys):
    """RenderParams::debug_print_num_rendered_points (PointRenderer.cu:1502-1512): the sum of the weights after a
    forward pass, printed as the reference prints it."""
    import torch
    import helpers
    from adop_amd import render, scenes

    announce("debug_print_num_rendered_points")
    hs = scenes.config3(n=100_000, w=240, h=136, channels=4)
    ref = oracle_mod.forward(hs)
    hs.params.forward_path = helpers.FORWARD_PATH
    info = render.NeuralRenderInfo(scene=render.NeuralScene.from_host(hs, "cuda"), images=list(hs.views),
                                   params=hs.params, num_layers=hs.num_layers, cache=render.PointRendererCache(),
                                   dropout_points=torch.from_numpy(hs.dropout), train=False,
                                   debug_print_num_rendered_points=True)
    capsys.readouterr()
    render.BlendPointCloudForward(None, info)
    want = sum(int(a) for a in ref.stats.accepted[: hs.num_layers])
    assert f"# Rasterized Points = {want}" in capsys.readouterr().out


def test_more_views_than_one_constant_chunk(oracle_mod):
    """34 views: the per-view constants take the chunked path (32 per launch), the descriptor pass fills 34 work
    queues, every view accumulates into the same point / pose / intrinsics gradients."""
    from adop_amd import scenes

    announce("config2 30k pts B=34 96x96 L3 fwd+bwd ghost")
    hs = scenes.config2(n=30_000, w=96, h=96, levels=3, batch=34)
    _fwd_bwd(hs, oracle_mod)


@pytest.mark.parametrize("shift", ["0", "1", "2", "3"])
def test_tile_counters_in_shards(oracle_mod, shift, forward_path):
    """The binning passes keep 1, 2, 4 or 8 counters per tile (runs of 256 points take them in turn; by default as many
    as a call of up to 4 096 tiles can have within 16 384 counters): a bin is the concatenation of its shards' parts,
    whatever their number.  Two views of 640 x 360 = 1 840 tiles."""
    from adop_amd import scenes

    if forward_path != 2:
        pytest.skip("the tile counters belong to the tile path")
    from adop_amd import _capi

    announce(f"config2 300k pts B=2 640x360, adop_tuning.bin_shard_shift={shift}")
    hs = scenes.config2(n=300_000, w=640, h=360, levels=4, batch=2, seed=8)
    with _capi.tuning(bin_shard_shift=int(shift)):
        _fwd_bwd(hs, oracle_mod, collect_stats=int(shift) % 2 == 0, poison=int(shift) % 2 == 1)


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_more_views_than_bits_of_the_view_masks(oracle_mod, collect_stats):
    """70 crop windows: the runs of 64 points that miss a window are marked (and their records left unwritten) for the
    first 64 views of a call only; the loops that jump from one live view to the next keep their masks in 64 bits."""
    from adop_amd import scenes

    announce(f"config2 20k pts B=70 crop windows 96x80 L3 fwd+bwd ghost, counters={collect_stats}")
    hs = scenes.config2(n=20_000, w=96, h=80, levels=3, batch=70, seed=70)
    g = np.random.default_rng(70)
    for v in hs.views:
        s = float(g.uniform(0.8, 3.0))
        v.crop_fx, v.crop_fy = s, s
        v.crop_cx, v.crop_cy = float(g.uniform(-2.0, 0.2) * 96), float(g.uniform(-2.0, 0.2) * 80)
    _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats)


@pytest.mark.parametrize("concurrent", ["0", "1"], ids=["per_view", "concurrent"])
@pytest.mark.parametrize("batch", [2, 5, 13, 24, 25, 34])
def test_spatial_gradients_per_view_and_of_all_views_at_once(oracle_mod, concurrent, batch):
    """With several views the spatial-gradient pass runs all views side by side in one launch (up to 24 views: a point
    that several views see is summed with atomics, every other row has one owner) or once per view, in the order of
    the views (more views, or adop_tuning.ghost_concurrent = 0): both against the checker, with batch sizes on either side of
    the limit and of the 32-view chunk of constants.  The views of this scene look at one small cloud, so that most
    points are shared by several views."""
    from adop_amd import scenes

    from adop_amd import _capi

    announce(f"config2 40k pts B={batch} 96x80 L3 fwd+bwd ghost, adop_tuning.ghost_concurrent={concurrent}")
    hs = scenes.config2(n=40_000, w=96, h=80, levels=3, batch=batch, seed=batch)
    with _capi.tuning(ghost_concurrent=int(concurrent)):
        _fwd_bwd(hs, oracle_mod)


@pytest.mark.parametrize("mode", [0, 1])
def test_normalize_modes_and_backward_mode4(oracle_mod, mode):
    from adop_amd import scenes

    announce(f"config3 reduced, test_backward_mode=4, normalize_mode={mode}")
    hs = scenes.config3(n=200_000, w=320, h=180, channels=4)
    hs.params.test_backward_mode = 4
    hs.params.normalize_mode = mode
    _fwd_bwd(hs, oracle_mod)


def test_distortion_crop_lod_mask(oracle_mod):
    from adop_amd import scenes

    announce("distortion + crop transform + LOD radius + background mask")
    hs = scenes.config3(n=300_000, w=400, h=300, channels=4)
    hs.intrinsics[0, 5:] = [0.05, -0.02, 0.003, 0.01, 0.002, -0.001, 0.001, -0.0015]
    hs.intrinsics[0, 4] = 0.3  # shear
    hs.params.dist_cutoff = 1.2
    v = hs.views[0]
    v.crop_fx, v.crop_fy, v.crop_cx, v.crop_cy, v.crop_s = 1.25, 1.25, -60.0, -35.0, 0.0
    hs.position[:, 3] = np.random.default_rng(3).uniform(0.001, 0.02, hs.num_points).astype(np.float32)
    hs.params.drop_out_points_by_radius = 1
    hs.params.output_background_mask = 1
    hs.params.output_background_mask_value = 0.25
    hs.background[:] = [0.1, 0.2, 0.3, 0.4]
    _fwd_bwd(hs, oracle_mod)


def test_shared_texels_use_the_atomic_path(oracle_mod):
    """index is not the identity: two points share a texel, a permutation for the rest."""
    from adop_amd import scenes

    announce("shared texels / permuted index (atomic descriptor-gradient path), C=8 and C=3")
    for channels in (8, 3):
        hs = scenes.config3(n=200_000, w=320, h=180, channels=channels)
        n = hs.num_points
        idx = np.random.default_rng(5).permutation(n).astype(np.int32) // 2
        hs.index = idx
        hs.texture = np.ascontiguousarray(hs.texture[:, : n // 2 + 1])
        _fwd_bwd(hs, oracle_mod)


def test_ocam_forward_backward(oracle_mod):
    from adop_amd import scenes

    announce("config5 reduced OCam 300k pts B=2 440x300")
    hs = scenes.config5(n=300_000, w=440, h=300, batch=2, patches=200)
    hs.params.ghost_gradients = 0
    _fwd_bwd(hs, oracle_mod)


def test_fp16_texture_forward(oracle_mod):
    from adop_amd import scenes

    announce("config4 reduced fp16 descriptors 500k pts 480x270 L5")
    hs = scenes.config4(n=500_000, w=480, h=270, frames=3)
    hs.views[0].image_index = 1
    ref = oracle_mod.forward(hs)
    scene, info, ctx, images, masks = run_hip_forward(hs)
    check_forward(hs, ref, ctx, images, masks, info)


def test_edge_cases(oracle_mod):
    """one point; points behind the camera; every point dropped; odd image sizes; one level."""
    from adop_amd import scenes

    announce("edge: single point")
    hs = scenes.config1(n=1, w=33, h=17, levels=3)
    hs.position[0, :3] = [0, 0, 0]
    hs.normal[0] = scenes.pack_normals(np.array([[0, 0, -1.0]]))[0]
    ref, _ = _fwd_bwd(hs, oracle_mod, needs=(True, True, True))
    assert ref.weight[0].sum() == 1
    announce("edge: all points behind the camera")
    hs = scenes.config1(n=1000, w=64, h=48, levels=2)
    hs.position[:, 2] = -10
    ref, _ = _fwd_bwd(hs, oracle_mod)
    assert all(w.sum() == 0 for w in ref.weight)
    announce("edge: everything dropped, ghost gradients on")
    hs = scenes.config1(n=5000, w=64, h=64, levels=5)
    hs.dropout = np.ones((1, 5000), np.float32)
    hs.params.ghost_gradients = 1
    _fwd_bwd(hs, oracle_mod)
    announce("edge: one level, 1x1 coarse sizes")
    hs = scenes.config1(n=3000, w=17, h=9, levels=4)
    _fwd_bwd(hs, oracle_mod)


def test_determinism_depth_index():
    """two runs give bit-identical packed depth|index buffers (the race on the early-z read is benign)."""
    from adop_amd import scenes

    announce("determinism")
    hs = scenes.config3(n=300_000, w=480, h=270)
    _, info1, _, _, _ = run_hip_forward(hs)
    a = [L.depth_index_tensor.clone() for L in info1.cache.layers_cuda]
    _, info2, _, _, _ = run_hip_forward(hs)
    for x, L in zip(a, info2.cache.layers_cuda):
        assert (x == L.depth_index_tensor).all()


def test_error_codes():
    import ctypes as C
    from adop_amd import _capi, render, scenes

    announce("error codes")
    hs = scenes.config1(n=100, w=32, h=32, levels=2)
    scene = render.NeuralScene.from_host(hs, "cuda")
    cache = render.PointRendererCache()
    info = render.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params, num_layers=2, cache=cache)
    cache.Build(info, True)
    s = scene.struct()
    fb = cache.forward_struct()
    fb.num_layers = 7
    rc = cache.lib.adop_forward(C.byref(s), cache.views_array(), 1, C.byref(hs.params), C.byref(fb),
                                C.c_void_p(cache.workspace.data_ptr()), cache.workspace.numel(), None, None)
    assert rc == _capi.ADOP_UNSUPPORTED_LAYERS
    assert b"layers" in cache.lib.adop_last_error_string()
    fb.num_layers = 2
    rc = cache.lib.adop_forward(C.byref(s), cache.views_array(), 1, C.byref(hs.params), C.byref(fb),
                                C.c_void_p(cache.workspace.data_ptr()), 16, None, None)
    assert rc == _capi.ADOP_WORKSPACE_TOO_SMALL
    s.normal = None
    rc = cache.lib.adop_forward(C.byref(s), cache.views_array(), 1, C.byref(hs.params), C.byref(fb),
                                C.c_void_p(cache.workspace.data_ptr()), cache.workspace.numel(), None, None)
    assert rc == _capi.ADOP_INVALID_ARG


def test_bad_texture_index_is_counted(oracle_mod):
    from adop_amd import scenes

    announce("texture index out of range is skipped and counted")
    hs = scenes.config1(n=2000, w=64, h=64, levels=2)
    hs.index[::7] = 10_000_000
    hs.index[3] = -5
    ref = oracle_mod.forward(hs)
    scene, info, ctx, images, masks = run_hip_forward(hs)
    check_forward(hs, ref, ctx, images, masks, info)
    assert info.cache.read_stats().bad_index == ref.stats.bad_index > 0


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
@pytest.mark.parametrize("forward_path", [1, 2], ids=["direct", "tiles"])
def test_runs_that_miss_a_view_are_marked_and_skipped(oracle_mod, forward_path, collect_stats):
    """A batch of crops: most runs of 64 points miss most views.  The forward marks them in the point cache (first
    record of the run: a NaN bit pattern in x, depth 0); without the counters (the production setting: wrappers and
    benchmark pass no counter buffer) it writes none of their other records and, on the tile path, none of their tile
    words; the blend and the backward of the batch skip them, and every result still equals the checker's.  No run with
    a point in the image is marked.  The plain runs start from a point cache and a workspace filled with a poison
    pattern: the records of marked runs still hold it afterwards (they really were not written), no record of an
    unmarked run does, and nothing computed from the buffers is off."""
    import torch
    from adop_amd import render, scenes

    from helpers import POISON_BITS

    n, w, h = 150_000, 256, 192
    hs = scenes.config2(n=n, w=w, h=h, levels=3, batch=1, seed=9)
    hs.params.forward_path = forward_path
    g = np.random.default_rng(2)
    poses = [hs.poses_se3[0], scenes.look_at_view((0.5, 2.5, -1.5)), scenes.look_at_view((9.0, 0.0, 0.0), (20.0, 0.0, 0.0))]
    hs.poses_se3 = np.stack(poses)  # the third camera looks away from the cloud
    hs.views = [scenes.make_view(64, 48, image_index=f, crop=(1.0, 1.0, -float(g.integers(0, w - 64)), -float(g.integers(0, h - 48)), 0.0))
                for f in (0, 0, 1, 1, 2)]
    hs.dropout = scenes.bernoulli_mask(4, len(hs.views), n, 0.25)
    announce(f"crops and a camera that looks away: N={n} B={len(hs.views)} 64x48 L=3 forward_path={forward_path}")
    ref, refb = _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats)
    # the marks in the cache of a second forward
    scene, info, ctx, images, masks = run_hip_forward(hs, collect_stats=collect_stats, poison=not collect_stats)
    cache = info.cache.point_cache.cpu().numpy()  # [B,N,4]
    bits = cache[:, ::64, 0].view(np.uint32)
    marked = (bits == 0x7FC0C011) & (cache[:, ::64, 2] == 0)
    assert marked[4].all()  # nothing of the cloud is in front of the third camera
    assert 0.3 < marked[:4].mean() < 0.99
    if not collect_stats:
        words = cache.view(np.uint32)  # [B,N,4]
        in_marked = np.repeat(marked, 64, axis=1)[:, :n]
        first = np.zeros((len(hs.views), n), bool)
        first[:, ::64] = True
        rest_of_marked = in_marked & ~first
        # the 63 other records of a marked run were left alone ...
        assert (words[rest_of_marked] == POISON_BITS).all()
        # ... and every record of an unmarked run was written
        assert not (words[~in_marked] == POISON_BITS).any()
    # The other records of a marked run are not written.  The records of the unmarked runs account for every point
    # the checker counts as visible at the finest level: no run with a point in the image was marked.
    z = cache[:, :, 2]
    ipx, ipy = cache[:, :, 0], cache[:, :, 1]
    with np.errstate(invalid="ignore"):
        inside = (z != 0) & ~np.isnan(ipx) & (np.rint(ipx) >= 0) & (np.rint(ipx) < 64) & (np.rint(ipy) >= 0) & (np.rint(ipy) < 48)
    inside &= ~np.repeat(marked, 64, axis=1)[:, :n]
    assert int(inside.sum()) == ref.stats.visible[0]


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
@pytest.mark.parametrize("forward_path", [1, 2], ids=["direct", "tiles"])
def test_runs_left_of_the_image_still_reach_the_coarse_levels(oracle_mod, forward_path, collect_stats):
    """Level l takes the pixel rint(ip * 0.5^l): a point up to half a coarse pixel left of (or above) the image is
    outside at level 0 and inside at a coarser level.  The cloud is ordered by image x here, so that whole runs of 64
    points lie in that band: a forward that drops runs by their level-0 position alone loses them."""
    from adop_amd import scenes

    n, w, h = 60_000, 250, 186
    hs = scenes.config2(n=n, w=w, h=h, levels=5, batch=1, seed=3)
    hs.params.forward_path = 1
    scene, info, ctx, images, masks = run_hip_forward(hs)
    cache = info.cache.point_cache.cpu().numpy()[0]  # one view: every record is written
    x_full = np.where(cache[:, 2] != 0, cache[:, 0], np.inf)
    order = np.argsort(x_full, kind="stable")
    hs.position, hs.index = hs.position[order], hs.index[order]
    if hs.normal is not None:
        hs.normal = hs.normal[order]
    x_full, y_full = x_full[order], cache[order, 1]
    # two windows of 128 x 96 whose left edges cut through the cloud
    offsets = [(-70.0, -40.0), (-101.0, -60.0)]
    hs.views = [scenes.make_view(128, 96, image_index=0, crop=(1.0, 1.0, cx, cy, 0.0)) for cx, cy in offsets]
    hs.dropout = scenes.bernoulli_mask(5, 2, n, 0.2)
    hs.params.forward_path = forward_path
    for cx, cy in offsets:
        band = (x_full + cx >= -7.9) & (x_full + cx < -0.6)
        runs = np.add.reduceat(band.astype(np.int64), np.arange(0, n, 64))
        whole = np.repeat(runs == 64, 64)[:n]
        assert (runs == 64).sum() >= 3, "the scene no longer puts whole runs into the band"
        assert (whole & (y_full + cy > 0) & (y_full + cy < 95)).sum() >= 64  # and those runs have points at image height
    announce(f"runs of 64 points in the band left of two windows: N={n} 128x96 L=5 forward_path={forward_path} "
             f"counters={collect_stats}")
    _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats)


def test_two_forwards_before_their_backwards(oracle_mod):
    """Gradient accumulation, or an evaluation render between a step's forward and backward: a second forward through
    the same cache must not touch what the first one saved for its backward pass."""
    import torch
    from adop_amd import render, scenes

    announce("two forwards through one cache, then both backwards")
    hs1 = scenes.config3(n=120_000, w=320, h=180, channels=4)
    hs2 = scenes.config3(n=120_000, w=320, h=180, channels=4)
    hs2.poses_se3 = np.stack([scenes.look_at_view((1.5, 1.0, -2.4))])
    hs2.dropout = scenes.bernoulli_mask(77, 1, hs2.num_points, 0.25)
    scene1 = render.NeuralScene.from_host(hs1, "cuda")
    scene2 = render.NeuralScene.from_host(hs2, "cuda")
    cache = render.PointRendererCache()

    class Ctx:
        def save_for_backward(self, *t):
            self.saved_tensors = t

    runs = []
    for hs, scene in ((hs1, scene1), (hs2, scene2)):
        hs.params.forward_path = 0
        info = render.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params, num_layers=hs.num_layers,
                                       cache=cache, train=True,
                                       dropout_points=None if hs.dropout is None else torch.from_numpy(hs.dropout))
        ctx = Ctx()
        images, masks = render.BlendPointCloudForward(ctx, info)
        runs.append((hs, info, ctx, images))
    torch.cuda.synchronize()
    for k, (hs, info, ctx, images) in enumerate(runs):
        ref = oracle_mod.forward(hs)
        for l in range(hs.num_layers):
            di = ctx.depth_index[l].cpu().numpy().view(np.uint64)
            assert np.array_equal(di, ref.depth_index[l]), f"forward {k}, level {l}: packed depth|index"
            assert np.array_equal(ctx.saved_tensors[2 * l + 1].cpu().numpy(), ref.weight[l])
        gout = scenes.upstream_grads(hs, 40 + k)
        grads = render.BlendPointCloudBackward(ctx, info, _torch_grads(gout))
        torch.cuda.synchronize()
        saved = oracle_mod.ForwardResult(hs)
        for l in range(hs.num_layers):
            saved.depth_index[l][...] = ctx.depth_index[l].cpu().numpy().view(np.uint64)
            saved.depth[l][...] = ctx.saved_tensors[2 * l].cpu().numpy()
            saved.weight[l][...] = ctx.saved_tensors[2 * l + 1].cpu().numpy()
            saved.out[l][...] = images[l].cpu().numpy()
        refb = oracle_mod.backward(hs, saved, gout)
        check_backward(hs, refb, grads, info, stats=False)


def test_tile_path_images_are_bit_identical_from_run_to_run():
    """The tile path sums a pixel's descriptors by walking a list that the entries of the tile were pushed on in
    whatever order the wavefronts ran: two runs may add in different orders.  Documented here as measured: the packed
    depth, depth, weight and mask are bit-identical from run to run, the images agree within the 1e-5 bar of the blend
    (and are bit-identical in most pixels)."""
    from adop_amd import scenes

    announce("tile path: run-to-run agreement of the images")
    hs = scenes.config3(n=400_000, w=480, h=270)
    runs = []
    for _ in range(3):
        _, info, _, images, _ = run_hip_forward(hs, collect_stats=False, forward_path=2)
        runs.append(([L.depth_index_tensor.clone() for L in info.cache.layers_cuda],
                     [L.weight.clone() for L in info.cache.layers_cuda], [im.clone() for im in images]))
    same = total = 0
    for di, wt, im in runs[1:]:
        for l in range(hs.num_layers):
            assert (di[l] == runs[0][0][l]).all() and (wt[l] == runs[0][1][l]).all()
            a, b = im[l].cpu().numpy(), runs[0][2][l].cpu().numpy()
            assert np.abs(a - b).max() <= 1e-5 * max(np.abs(b).max(), 1e-30)
            same += int((a.view(np.uint32) == b.view(np.uint32)).sum())
            total += a.size
    print(f"[info] tile path, 3 runs: {same} of {total} image values bit-identical", flush=True)
    assert same >= 0.9 * total


@pytest.mark.parametrize("slice_entries", ["64", "7", "1"], ids=["slices_of_64", "slices_of_7", "no_rows_left"])
@pytest.mark.parametrize("channels,collect_stats", [(8, True), (8, False), (4, False), (3, True)],
                         ids=["C8-counters", "C8-plain", "C4-plain", "C3-counters"])
def test_full_bins_are_split_between_workgroups(oracle_mod, forward_path, slice_entries, channels, collect_stats):
    """A cloud that covers a few tiles only (the camera far away) puts tens of thousands of entries into one bin; bins
    above four times adop_tuning.tile_slice_entries entries (8192 by default) are split in slices of that size that
    as many workgroups take, the last of which merges their rows.  Forced here on small scenes: with 64 and 7 entries
    per slice most bins are split (up to 1023 slices a bin), with 1 the rows run out and most bins stay whole.  Forward and backward
    through the tile path still equal the checker (packed depth bit for bit), with and without the counters, for the
    vectorised channel counts and the generic one."""
    from adop_amd import scenes

    if forward_path != 2:
        pytest.skip("the tile path only")
    from adop_amd import _capi

    announce(f"tile path with split bins: tile_slice_entries={slice_entries}, C={channels}, counters={collect_stats}")
    hs = scenes.config3(n=150_000, w=160, h=96, channels=channels)
    with _capi.tuning(tile_slice_entries=int(slice_entries)):
        _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats)
        # the camera ten times as far: the cloud lands in a handful of tiles
        el, az = np.deg2rad(20.0), np.deg2rad(30.0)
        hs.poses_se3 = scenes.look_at_view(30.0 * np.array([np.cos(el) * np.sin(az), np.sin(el), -np.cos(el) * np.cos(az)]))[None, :]
        _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=not collect_stats)


def test_smaller_workspaces(oracle_mod, forward_path):
    """adop_workspace_size_for + adop_render_params.workspace_flags: a workspace without the region of a forward pass
    that keeps no point cache, without the tile bins, with small bins, and the combinations.  Same results; without the
    bins the library renders through the direct path (and refuses forward_path = 2); without the other region it
    refuses a forward pass that passes no point cache."""
    import torch
    from adop_amd import _capi, render, scenes

    hs = scenes.config3(n=150_000, w=256, h=144, channels=4, seed=21)
    ref = oracle_mod.forward(hs)
    gout = scenes.upstream_grads(hs, 9)
    KEPT, NOBINS, SMALL = _capi.WORKSPACE_POINT_CACHE_KEPT, _capi.WORKSPACE_NO_TILE_PATH, _capi.WORKSPACE_SMALL_BINS
    lib = _capi.load_library()
    sizes = {}
    for flags in (0, KEPT, NOBINS, KEPT | NOBINS, SMALL, SMALL | KEPT):
        announce(f"workspace flags {flags}, forward_path={forward_path}")
        if (flags & NOBINS) and forward_path == 2:
            with pytest.raises(RuntimeError, match="tile bins"):
                run_hip_forward(hs, workspace_flags=flags)
            continue
        scene, info, ctx, images, masks = run_hip_forward(hs, workspace_flags=flags, poison=True)
        sizes[flags] = info.cache.workspace.numel()
        check_forward(hs, ref, ctx, images, masks, info)
        grads = render.BlendPointCloudBackward(ctx, info, _torch_grads(gout))
        torch.cuda.synchronize()
        refb = oracle_mod.backward(hs, download_forward(hs, info, images, masks), gout)
        check_backward(hs, refb, grads, info)
        if flags & KEPT:  # a forward pass that passes no point cache after all
            with pytest.raises(RuntimeError, match="point_cache"):
                run_hip_forward(hs, workspace_flags=flags, train=False)
        else:
            got = run_hip_forward(hs, workspace_flags=flags, train=False, poison=True)
            check_forward(hs, ref, got[2], got[3], got[4], got[1])
    if forward_path != 2:
        assert sizes[0] > sizes[KEPT] > sizes[NOBINS] > sizes[KEPT | NOBINS] and sizes[0] > sizes[SMALL] > sizes[SMALL | KEPT]
    s = _capi.Scene()
    s.num_points, s.num_channels, s.num_poses, s.num_cameras, s.intrinsics_cols = hs.num_points, 4, 1, 1, 13
    assert lib.adop_workspace_size_for(ctypes.byref(s), 1, 4, 256, 144, 8) == 0  # an unknown flag
    hs.params.workspace_flags = 0


@pytest.mark.parametrize("collect_stats", [True, False], ids=["counters", "plain"])
def test_small_bins_fall_back_to_the_direct_path_on_the_device(oracle_mod, forward_path, collect_stats):
    """ADOP_WORKSPACE_SMALL_BINS holds one bin entry per four points and view.  A view that sees the whole cloud has
    more (a cube in front of the camera: one entry per point and a few second entries): the prefix sum of the binning
    passes finds that out on the device, the tile kernels return at once and the direct path's kernels behind them
    render the call, counters included.  A batch of crops fits and runs through the tile kernels.  Both against the
    checker, forward (with and without a point cache) and backward."""
    import torch
    from adop_amd import _capi, render, scenes

    if forward_path != 2:
        pytest.skip("the tile path only")
    SMALL = _capi.WORKSPACE_SMALL_BINS
    # (a) overflow: every point of the cube is in the image
    hs = scenes.config1(n=120_000, w=320, h=320, levels=4, seed=3, point_order="morton")
    hs.params.ghost_gradients = 0
    announce(f"small bins, a view that overflows them: 120k pts 320x320, counters={collect_stats}")
    ref = oracle_mod.forward(hs)
    assert int(ref.stats.visible[0]) > hs.num_points // 4 + 1024  # more entries than the small bins hold
    for train in (True, False):
        scene, info, ctx, images, masks = run_hip_forward(hs, workspace_flags=SMALL, train=train, poison=True,
                                                          collect_stats=collect_stats)
        check_forward(hs, ref, ctx, images, masks, info, stats=collect_stats)
        if train:
            gout = scenes.upstream_grads(hs, 9)
            grads = render.BlendPointCloudBackward(ctx, info, _torch_grads(gout))
            torch.cuda.synchronize()
            refb = oracle_mod.backward(hs, download_forward(hs, info, images, masks), gout)
            check_backward(hs, refb, grads, info, stats=collect_stats)
    # (b) no overflow: four crops that see a part of the cloud each
    hs = scenes.config3(n=200_000, w=192, h=128, channels=4, seed=13)
    hs.views = [scenes.make_view(192, 128, crop=(3.0, 3.0, -float(x), -float(y), 0.0)) for (x, y) in
                ((100, 60), (300, 120), (150, 200), (20, 10))]
    hs.dropout = scenes.bernoulli_mask(5, 4, hs.num_points, 0.25)
    announce(f"small bins, four crops that fit: 200k pts, counters={collect_stats}")
    ref = oracle_mod.forward(hs)
    assert sum(int(v) for v in ref.stats.visible[:1]) < hs.num_points  # well inside 4 * N / 4
    _fwd_bwd(hs, oracle_mod, collect_stats=collect_stats, poison=True, workspace_flags=SMALL)
    hs.params.workspace_flags = 0


# Every kernel variant the tuning switches choose between, each on one small scene (forward without a point cache,
# training forward and backward) against the checker.
TUNING_VARIANTS = [dict(count_ppt=1), dict(count_ppt=2), dict(count_ppt=4), dict(scatter_ppt=1), dict(scatter_ppt=4), dict(tile_k=2),
                   dict(tile_k=4), dict(normalize_fused=0), dict(normalize_fused=0, normalize_by_queue=0),
                   dict(prepass_ppt=1), dict(prepass_ppt=2), dict(prepass_ppt=4), dict(direct_lists=0),
                   dict(prepass_group_from=0), dict(prepass_group_from=5), dict(blend_group_from=2),
                   dict(blend_group_from=5), dict(list_block=64), dict(list_block=256),
                   dict(bin_shard_shift=3, count_ppt=4, scatter_ppt=4), dict(forward_path=1), dict(forward_path=2)]


@pytest.mark.parametrize("variant", TUNING_VARIANTS, ids=lambda v: ",".join(f"{k}={x}" for k, x in v.items()))
def test_every_tuning_variant_gives_the_same_results(oracle_mod, variant, forward_path):
    from adop_amd import _capi, scenes

    tile_only = {"count_ppt", "scatter_ppt", "tile_k", "bin_shard_shift"}
    direct_only = {"prepass_ppt", "direct_lists", "prepass_group_from", "blend_group_from", "list_block"}
    if (forward_path == 1 and set(variant) & tile_only) or (forward_path == 2 and set(variant) & direct_only):
        pytest.skip("a switch of the other forward path")
    announce(f"tuning variant {variant}: 120k pts B=2 200x120 L4, forward_path={forward_path}")
    hs = scenes.config3(n=120_000, w=200, h=120, channels=4, seed=11)
    hs.views = [scenes.make_view(200, 120), scenes.make_view(200, 120, crop=(1.25, 1.25, -20.0, -10.0, 0.0))]
    hs.dropout = scenes.bernoulli_mask(4, 2, hs.num_points, 0.25)
    one = __import__("copy").copy(hs)  # (normalize_fused concerns calls with one view)
    one.views, one.dropout = hs.views[:1], np.ascontiguousarray(hs.dropout[:1])
    with _capi.tuning(**variant):
        if "forward_path" in variant:
            import helpers
            helpers.FORWARD_PATH = 0  # the library's own choice, through the switch
        for scene in (hs, one):
            ref = oracle_mod.forward(scene)
            got = run_hip_forward(scene, collect_stats=False, train=False)
            check_forward(scene, ref, got[2], got[3], got[4], got[1], stats=False)
            _fwd_bwd(scene, oracle_mod, collect_stats=False, poison=True)


def test_zz_report_end_to_end_misses():
    """Prints what the end-to-end element-wise check of every case above found (the asserts are in _fwd_bwd)."""
    for case, rec in end_to_end_misses.items():
        print("[end-to-end]", case, {k: (m, n, float(f"{w:.2e}")) for k, (m, n, w) in rec.items() if m}, flush=True)
