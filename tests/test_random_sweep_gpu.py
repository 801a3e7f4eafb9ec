"""GPU parity on randomly drawn small scenes: every seed picks the cloud size, image size, number of levels and views,
channel count, camera model, distortion, crop, LOD radii, dropout, gradient switches and descriptor storage, and the
HIP path (both forward implementations, with and without a point cache) is compared with the CPU checker to the
bars of tests/test_parity_gpu.py.  The named cases cover what the reference's configurations use; the sweep covers
the combinations nobody thought of."""
import os

import numpy as np
import pytest

from helpers import announce, assert_norm_close, check_backward, check_forward, download_forward, run_hip_forward

pytestmark = pytest.mark.gpu

# ADOP_SWEEP_SEEDS="first:count" draws other scenes than the 100 of a default run (a longer soak on a GPU box)
_first, _count = (int(x) for x in os.environ.get("ADOP_SWEEP_SEEDS", "0:100").split(":"))
SEEDS = list(range(_first, _first + _count))


def random_scene(seed):
    from adop_amd import scenes

    g = np.random.default_rng(7000 + seed)
    levels = int(g.integers(1, 6))
    w = int(g.integers(max(17, 1 << (levels - 1)), 150))
    h = int(g.integers(max(17, 1 << (levels - 1)), 150))
    batch = int(g.integers(1, 4))
    n = int(g.choice([1, 7, 63, 64, 65, 255, 257, 1000, 5000, 20000, 40000]))
    ghost = bool(g.integers(0, 2))
    ocam = g.random() < 0.25
    order = str(g.choice(["morton", "random", "generated"]))
    if ocam:
        hs = scenes.config5(n=n, w=w, h=h, levels=levels, batch=batch, patches=20, seed=seed, point_order=order)
        hs.env_texture = None
        hs.params.ghost_gradients = 1 if ghost else 0
    else:
        hs = scenes.config2(n=n, w=w, h=h, levels=levels, batch=batch, seed=seed, ghost=ghost, point_order=order)
        if g.random() < 0.5:
            hs.intrinsics[0, 5:] = g.uniform(-1.0, 1.0, 8) * [0.05, 0.02, 0.005, 0.02, 0.01, 0.002, 0.002, 0.002]
        if g.random() < 0.3:
            hs.intrinsics[0, 4] = g.uniform(-0.3, 0.3)  # shear
        hs.params.dist_cutoff = float(g.choice([1.0e6, 1.5, 0.8]))
    # descriptors: channel count, storage, texel index
    C = int(g.choice([1, 3, 4, 8, 1, 3, 4, 8, 2, 5, 7, 12, 16]))  # 4 and 8 have kernels of their own; 16 is the limit
    kind = str(g.choice(["identity", "permuted", "shared"]))
    ntex = n if kind != "shared" else max(1, n // 2)
    tex = g.random((C, ntex), dtype=np.float32)
    if g.random() < 0.25:
        tex = tex.astype(np.float16)
    hs.texture = tex
    if kind == "permuted":
        hs.index = g.permutation(n).astype(np.int32)
    elif kind == "shared":
        hs.index = (g.permutation(n) % ntex).astype(np.int32)
    hs.background = g.random(C, dtype=np.float32)
    # crop transform of every view
    if g.random() < 0.5:
        for v in hs.views:
            s = float(g.uniform(0.7, 1.4))
            v.crop_fx, v.crop_fy = s, s
            v.crop_cx, v.crop_cy = float(g.uniform(-0.3, 0.1) * w), float(g.uniform(-0.3, 0.1) * h)
    # LOD radii
    if g.random() < 0.4:
        hs.position[:, 3] = g.uniform(0.0005, 0.02, n).astype(np.float32)
        hs.params.drop_out_points_by_radius = 1
        hs.params.drop_out_radius_threshold = float(g.uniform(0.02, 0.3))  # radii are 0.02 .. 1 pixel at level 0
    # dropout mask (ghost points need one to exist)
    p = float(g.choice([0.0, 0.1, 0.3, 0.5, 0.5, 1.0]))
    hs.dropout = None if (p == 0.0 and g.random() < 0.5) else scenes.bernoulli_mask(seed + 3, batch, n, p)
    hs.params.check_normal = int(g.integers(0, 2)) if hs.normal is not None else 0
    hs.params.depth_accept = float(g.choice([0.01, 0.002, 0.05]))
    hs.params.output_background_mask = int(g.integers(0, 2))
    hs.params.output_background_mask_value = float(g.choice([0.0, 0.25]))
    hs.params.normalize_mode = int(g.integers(0, 2))
    hs.params.test_backward_mode = int(g.choice([0, 4]))
    needs = tuple(bool(x) for x in g.integers(0, 2, 3))
    what = (f"seed {seed}: N={n} {w}x{h} L={levels} B={batch} C={C} {tex.dtype} index={kind} "
            f"{'ocam' if ocam else 'pinhole'} order={order} ghost={ghost} dropout={p} needs={needs}")
    return hs, needs, what


@pytest.mark.parametrize("forward_path", [1, 2], ids=["direct", "tiles"])
@pytest.mark.parametrize("seed", SEEDS)
def test_random_scene(oracle_mod, seed, forward_path):
    import torch
    from adop_amd import render, scenes

    hs, needs, what = random_scene(seed)
    announce(f"{what} forward_path={forward_path}")
    ref = oracle_mod.forward(hs)
    # inference forward (no point cache), counters on even seeds
    scene, info, ctx, images, masks = run_hip_forward(hs, collect_stats=seed % 2 == 0, forward_path=forward_path,
                                                      train=False)
    check_forward(hs, ref, ctx, images, masks, info, stats=seed % 2 == 0)
    # training forward + backward; every third seed without the counters (the kernels' production variants), from a
    # poisoned point cache and workspace
    counters = seed % 3 != 0
    scene, info, ctx, images, masks = run_hip_forward(hs, collect_stats=counters, forward_path=forward_path,
                                                      poison=not counters, pixel_records=seed % 4 != 1)
    check_forward(hs, ref, ctx, images, masks, info, stats=counters)
    gout = scenes.upstream_grads(hs, seed + 11)
    grads = render.BlendPointCloudBackward(ctx, info, [torch.from_numpy(g).cuda() for g in gout], needs)
    torch.cuda.synchronize()
    saved = download_forward(hs, info, images, masks)
    refb = oracle_mod.backward(hs, saved, gout, *needs)
    check_backward(hs, refb, grads, info, stats=counters)
    refb2 = oracle_mod.backward(hs, ref, gout, *needs)
    names = ["grad_texture", "grad_background", "grad_points", "grad_pose", "grad_intrinsics"]
    for name, gr in zip(names, grads):
        if gr is not None:
            assert_norm_close(gr.float().cpu().numpy(), getattr(refb2, name), 1e-4, name + " (checker forward)")
