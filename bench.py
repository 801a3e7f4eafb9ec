#!/usr/bin/env python3
"""Benchmark of the point-rasterizer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config3|config1|config2|config4|config5|crops]

A step is one pass of the hot path over one batch of synthetic input that already sits in HBM:
``adop_forward`` + ``adop_backward`` through the C-ABI (forward only for configs 1 and 4; config 5 adds the
environment-map pass on its OCam views and its texture gradient).  Prints ONE JSON line.

Default workload: BASELINE config 3 (10 M points, 1920x1080, 4 levels, 8 channels, forward + backward with
descriptor / point / pose / intrinsics gradients) -> points/s.  The default run then also measures the second
headline figure, config 4 (100 M points, 5 levels, fp16 descriptors, forward over the 300-frame orbit -> frames/s),
and reports it under ``step.config4`` (``--no-config4`` leaves it out), and after it every other BASELINE
configuration and the reference's training shape under ``step.configs``: config 1, config 2, config 5 (with its
environment map), a training batch of 16 crops, and configs 3 and 4 once more with the cloud in random order and with
the reference's default LOD radius test (``--headline-only`` leaves these out).

``roofline`` describes the slowest kernel of the step: algorithmic bytes of that kernel (byte model below, with
the point-level counts V/A/G measured by the kernels' own counters in an untimed pass) divided by its average
duration measured with HIP events on the launch stream, against the 8 TB/s HBM peak.  ``roofline.traffic`` and
``step.hbm_frac_measured`` use HBM bytes per launch measured with rocprofv3 counters (MEASURED_TRAFFIC below: each
table names the profile it comes from and the kernel state it was measured on; for any other state they are null).
``cpu_baseline`` times the CPU checker (OpenMP build) on the host cores for the same workload (or a bounded
sample of it): one warm-up run, then the median of three; ``cpu_baseline.matches_gpu`` compares the buffers the
checker computed in those runs with the HIP path's on the same inputs.
"""
import argparse
import ctypes as C
import gc
import hashlib
import glob
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
KERNEL_OF_STAGE = {"BinCount": "bin_count_kernel", "BinScatter": "bin_scatter_kernel", "TileDepth": "tile_depth_kernel", "TileBlend": "tile_blend_kernel",
                   "DepthPrepass": "prepass_kernel", "RenderForward": "blend_kernel", "CombineAndFill": "resolve_kernel",
                   "CombineAndFillBackward": "interleave_kernel", "RenderBackward/descriptor": "backward_tex_kernel",
                   "RenderBackward/spatial": "backward_ghost_kernel", "EnvironmentMap": "env_sample_kernel",
                   "EnvironmentMapBackward": "env_backward_kernel"}

# HBM bytes per launch (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, KiB per dispatch; FETCH_SIZE x 2.0 and WRITE_SIZE
# x 1.0 after calibration with plain device copies of known size), per workload.  "sources" is kernel_sources_state() of
# the tree the profile was taken on (python bench.py --print-sources-state): the figures are quoted for that state only.
MEASURED_TRAFFIC = {
    "config3": {"sources": "78604d234635", "profile": "profiles/config3_tile_path_fwd_bwd_kernels_traffic_instructions.md",
                "bytes": {"RenderBackward/descriptor": 860.0e6, "RenderBackward/spatial": 572.1e6, "TileBlend": 529.0e6, "BinCount": 430.3e6, "BinScatter": 197.5e6, "CombineAndFillBackward": 220.8e6, "TileDepth": 101.5e6, "Post Process Gradient": 0.5e6, "CombineAndFill": 23.5e6, "Initialize": 11.8e6}},
    "config1": {"sources": "78604d234635", "profile": "profiles/config1_direct_path_forward_kernels_traffic_instructions.md",
                "bytes": {"DepthPrepass": 13.0e6, "RenderForward": 8.5e6, "Initialize": 3.5e6, "CombineAndFill": 5.6e6}},
    "config2": {"sources": "78604d234635", "profile": "profiles/config2_fwd_bwd_kernels_traffic_instructions.md",
                "bytes": {"RenderBackward/descriptor": 200.8e6, "TileBlend": 161.9e6, "RenderBackward/spatial": 146.7e6, "BinScatter": 67.5e6, "BinCount": 64.5e6, "CombineAndFillBackward": 67.2e6, "TileDepth": 37.9e6, "Post Process Gradient": 15.1e6, "Initialize": 3.4e6, "CombineAndFill": 6.6e6}},
    "config4": {"sources": "78604d234635", "profile": "profiles/config4_direct_path_forward_kernels_traffic_instructions.md",
                "bytes": {"DepthPrepass": 5080.7e6, "RenderForward": 1545.8e6, "CombineAndFill": 176.8e6, "Initialize": 110.5e6}},
    "config5": {"sources": "78604d234635", "profile": "profiles/config5_ocam_envmap_fwd_bwd_kernels_traffic_instructions.md",
                "bytes": {"RenderBackward/spatial": 5753.6e6, "TileBlend": 5064.9e6, "EnvironmentMapBackward": 2242.8e6, "BinCount": 2189.5e6, "RenderBackward/descriptor": 4091.9e6, "EnvironmentMap": 3081.4e6, "BinScatter": 3331.6e6, "TileDepth": 1622.9e6, "CombineAndFillBackward": 1872.4e6, "Post Process Gradient": 484.7e6, "CombineAndFill": 177.1e6, "Initialize": 91.5e6}},
    "crops": {"sources": "78604d234635", "profile": "profiles/training_batch_16_crops_fwd_bwd_kernels_traffic_instructions.md",
                "bytes": {"RenderBackward/descriptor": 1579.8e6, "RenderBackward/spatial": 1242.0e6, "BinCount": 587.1e6, "TileBlend": 1211.8e6, "BinScatter": 764.6e6, "CombineAndFillBackward": 446.2e6, "TileDepth": 249.2e6, "Post Process Gradient": 120.3e6, "CombineAndFill": 47.8e6, "Initialize": 23.7e6}},
}


def byte_model(N, B, C_, S_d, P, V, A, G, has_mask, has_dropout):
    """Algorithmic bytes per kernel for one step (per-unit figures of the hot-path byte model)."""
    sv, sa, sg = sum(V), sum(A), sum(G)
    drop = 4 if has_dropout else 0
    k = {}
    k["DepthPrepass"] = B * N * 20 + sv * 8
    k["RenderForward"] = B * N * (24 + drop) + sa * (C_ * S_d + C_ * 4 + 4)
    k["CombineAndFill"] = B * P * (8 + 4 + 2 * C_ * 4) + (B * P * 4 if has_mask else 0)
    # RenderBackward runs as two kernels: descriptor gradient (+ work queue) and ghost / spatial gradient
    k["RenderBackward/descriptor"] = B * N * (24 + drop) + sa * (4 + 4 + C_ * 4 + C_ * 4)
    k["RenderBackward/spatial"] = sg * (4 * (8 + 8 * C_) + C_ * S_d + 16)
    k["CombineAndFillBackward"] = B * P * (4 + 4 * C_)
    return k


def tile_path_model(k, N, B, C_, P_levels, V, has_dropout, lt=2):
    """The same forward bytes attributed to the kernels of the tile-bin path: bin_kernel<0> reads the points,
    bin_kernel<1> re-reads them (the blend's read), tile_depth_kernel does the depth prepass, tile_blend_kernel
    the blend and the resolve of the fine levels, resolve_kernel the coarse levels."""
    drop = 4 if has_dropout else 0
    lt = min(lt, len(V))
    frac_coarse = sum(P_levels[lt:]) / float(sum(P_levels))
    prepass, blend, caf = k.pop("DepthPrepass"), k.pop("RenderForward"), k.pop("CombineAndFill")
    k["BinCount"] = B * N * 20
    k["BinScatter"] = B * N * (24 + drop)
    k["TileDepth"] = sum(V) * 8
    k["TileBlend"] = (blend - B * N * (24 + drop)) + caf * (1 - frac_coarse)
    k["CombineAndFill"] = caf * frac_coarse
    assert abs(sum((k[n] for n in ("BinCount", "BinScatter", "TileDepth", "TileBlend", "CombineAndFill"))) - (prepass + blend + caf)) < 1
    return k


def kernel_sources_state():
    """First 12 hex digits of the SHA-256 over the code of the sources the library is built from (adop_amd/csrc/*.hip,
    *.h and the C header; comments and white space left out): the state of the kernels a traffic profile was taken on.
    A table of MEASURED_TRAFFIC is quoted only while this matches its "sources" entry, so an edited kernel can never be
    reported with stale measured bytes."""
    import re

    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(ROOT, "adop_amd", "csrc", "*.hip")) +
                   glob.glob(os.path.join(ROOT, "adop_amd", "csrc", "*.h")) +
                   [os.path.join(ROOT, "include", "adop_raster.h")])
    for f in files:
        text = open(f, encoding="utf-8").read()
        text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)   # block comments
        text = re.sub(r"//[^\n]*", " ", text)                # line comments (no string of these sources holds "//")
        text = " ".join(text.split())
        h.update(os.path.basename(f).encode())
        h.update(text.encode())
    return h.hexdigest()[:12]


def host_threads():
    """Threads of the CPU baseline: the share of the host this process is given (OMP_NUM_THREADS where the
    environment sets it, as the GPU boxes do for their one-GPU share; otherwise every core the OS shows)."""
    env = os.environ.get("OMP_NUM_THREADS", "")
    n = int(env) if env.isdigit() and int(env) > 0 else (os.cpu_count() or 1)
    os.environ["OMP_NUM_THREADS"] = str(n)
    return n


def bench_preprocess(args):
    """Point-cloud preprocessing (the caller side of the path): 4th-nearest-neighbour distance and Morton codes of the
    config-3 cloud in random order.  One step = both kernels' chains on all points."""
    import numpy as np
    import torch
    from adop_amd import preprocess, scenes

    t0 = time.time()
    hs = scenes.config3(point_order="random", **({"n": args.points} if args.points else {}))
    gen_s = time.time() - t0
    N = hs.num_points
    pos = torch.from_numpy(hs.position).cuda()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    for _ in range(max(args.warmup, 1)):
        preprocess.KNearestNeighbourDistance(pos, 4)
        preprocess.MortonCodes(pos)
    torch.cuda.synchronize()
    t_knn = t_mor = 0.0
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ev[0].record()
        preprocess.KNearestNeighbourDistance(pos, 4)
        ev[1].record()
        preprocess.MortonCodes(pos)
        ev[2].record()
        torch.cuda.synchronize()
        t_knn += ev[0].elapsed_time(ev[1])
        t_mor += ev[1].elapsed_time(ev[2])
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    t_knn /= args.steps
    t_mor /= args.steps
    # The point filters of a new scene (outside the timed steps): camera distance over 100 frames on an orbit, lonely
    # points (5th neighbour), close points (0.00005 / camera distance).
    frames = 100
    poses = torch.from_numpy(np.stack([scenes.orbit_pose(f, radius=3.0, deg_per_frame=3.6) for f in range(frames)])).cuda()
    intr = torch.from_numpy(hs.intrinsics).cuda()
    fviews = [scenes.make_view(hs.views[0].w, hs.views[0].h, image_index=f) for f in range(frames)]
    filt = {}
    for name, fn in (("camera_distance_100_frames", lambda: preprocess.PointDistanceToCamera(pos, poses, intr, fviews)),
                     ("lonely_points", lambda: preprocess.RemoveLonelyPoints(pos, cam, 5, 0.02)),
                     ("close_points", lambda: preprocess.RemoveClosePoints(pos, cam, 0.00005))):
        ts = []
        for _ in range(3):
            torch.cuda.synchronize()
            tf = time.perf_counter()
            r = fn()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - tf) * 1e3)
        if name == "camera_distance_100_frames":
            cam = r
        filt[name] = round(sorted(ts)[1], 3)
    # algorithmic bytes of the neighbour search: the cloud is read twice and written once in cell order (binning),
    # read once more by the search, 4 bytes per point out; neighbours are read through the caches (the library bins
    # twice, for its first and second grid: its choice, not the algorithm's)
    knn_bytes = N * (16 + 16 + 16 + 16 + 4)
    cpu = None
    if not args.no_cpu_baseline:
        import oracle.preprocess as op
        m = args.cpu_points or 20000
        tc0 = time.perf_counter()
        op.knn_distance(hs.position[:m], 4)
        op.morton_codes(hs.position[:m])
        sec = time.perf_counter() - tc0
        cpu = {"value": m / sec, "unit": "points/s", "cores": 1, "kind": "port",
               "sample": f"brute-force neighbour search among the first {m} of {N} points + their Morton codes",
               "seconds": round(sec, 3)}
    return {
        "metric": "preprocess points/s", "value": N / (ms_per_step * 1e-3), "unit": "points/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"preprocess: 4th-nearest-neighbour distance + Morton codes, {N} points of config3 in "
                               "random order"},
        "roofline": {"bound": "hbm", "kernel": "knn_search_kernel", "stage": "knn_distance",
                     "achieved": round(knn_bytes / (t_knn * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(knn_bytes / (t_knn * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel_ms": round(t_knn, 4), "algorithmic_bytes": int(knn_bytes)},
        "cpu_baseline": cpu,
        "step": {"stage_ms": {"knn_distance": round(t_knn, 4), "morton_codes": round(t_mor, 4)},
                 "filters_ms": filt,
                 "scene_gen_s": round(gen_s, 1)},
    }


def make_scene(args, workload, point_order, lod):
    """The host scene of a workload.  point_order: "morton" = the reference's stored order (Morton curve + shuffled
    256-point blocks, SceneData.cpp:101-102), "random" = a random permutation.  lod: position.w gets the drop-out radius
    of a new scene (4th-neighbour distance x sqrt(1/u), blocks sorted by it: SceneData.cpp:103-104; computed on the
    device) and the LOD radius test is switched on (the reference's default, Settings.h:36-37)."""
    from adop_amd import preprocess, scenes

    import copy

    kw = {"n": args.points} if args.points else {}
    key = (workload, point_order, args.points)
    if key in _scene_cache:  # (config 4 takes half a minute to generate: its LOD variant starts from the same cloud)
        base = _scene_cache[key]
        hs = copy.copy(base)
        hs.params, hs.meta, hs.views = copy.copy(base.params), dict(base.meta), [copy.copy(v) for v in base.views]
    else:
        if workload == "config3":
            hs = scenes.config3(point_order=point_order, **kw)
        elif workload == "config1":
            hs = scenes.config1(**kw)
        elif workload == "config2":
            hs = scenes.config2(point_order=point_order, **kw)
        elif workload == "config4":
            hs = scenes.config4(point_order=point_order, **kw)
        elif workload == "crops":
            hs = scenes.training_batch(point_order=point_order, **kw)
        else:
            hs = scenes.config5(point_order=point_order, **kw)
        if workload == "config4" and point_order == "morton":
            _scene_cache[key] = hs
            return make_scene(args, workload, point_order, lod)
    if lod:
        preprocess.AttachDropOutRadii(hs)
    return hs


_scene_cache = {}


def compare_with_checker(lib, scene, chs, ref, refb, cgout, full):
    """cpu_baseline.matches_gpu: the HIP path on the CPU sample's inputs (the views of ``chs`` of the resident scene)
    against the buffers the checker computed while it was timed.  Packed depth|index, depth and weight bit for bit;
    blended descriptors within 1e-5 relative (x sqrt(n / 1024) on a pixel of n > 1024 points, 1e-7 absolute floor: the
    bars of tests/helpers.py).  ``full`` (the sample is the whole workload): the descriptor gradient element-wise within
    1e-4 / 1e-6, the other gradients within 1e-4 of the tensor's largest magnitude (the checker's backward pass ran on
    its own forward images here, whose sums differ by the order of the additions)."""
    import numpy as np
    import torch
    from adop_amd import render

    cache = render.PointRendererCache()
    info = render.NeuralRenderInfo(scene=scene, images=list(chs.views), params=chs.params, num_layers=chs.num_layers,
                                   cache=cache, train=refb is not None,
                                   dropout_points=None if chs.dropout is None else torch.from_numpy(chs.dropout))

    class Ctx:
        def save_for_backward(self, *t):
            self.saved_tensors = t

    ctx = Ctx()
    images, _ = render.BlendPointCloudForward(ctx, info)
    torch.cuda.synchronize()
    m = {"depth_index_bit_exact": True, "depth_bit_exact": True, "weight_bit_exact": True, "out_within_1e-5": True,
         "out_max_rel_err": 0.0}
    for l, L in enumerate(cache.layers_cuda):
        m["depth_index_bit_exact"] &= bool(np.array_equal(L.depth_index_tensor.cpu().numpy().view(np.uint64), ref.depth_index[l]))
        m["depth_bit_exact"] &= bool(np.array_equal(L.depth.cpu().numpy().view(np.uint32), ref.depth[l].view(np.uint32)))
        w = L.weight.cpu().numpy()
        m["weight_bit_exact"] &= bool(np.array_equal(w, ref.weight[l]))
        got, want = images[l].cpu().numpy().astype(np.float64), ref.out[l].astype(np.float64)
        err = np.abs(got - want)
        bar = np.maximum(1e-5 * np.sqrt(np.maximum(w.astype(np.float64) / 1024.0, 1.0)) * np.abs(want), 1e-7)
        m["out_within_1e-5"] &= bool((err <= bar).all())
        m["out_max_rel_err"] = max(m["out_max_rel_err"], float((err / np.maximum(np.abs(want), 1e-3)).max()))
    if refb is not None and full:
        grads = render.BlendPointCloudBackward(ctx, info, [torch.from_numpy(g).cuda() for g in cgout])
        torch.cuda.synchronize()
        g_tex = grads[0].cpu().numpy().astype(np.float64)
        want = refb.grad_texture.astype(np.float64)
        m["grad_texture_within_1e-4"] = bool((np.abs(g_tex - want) <= np.maximum(1e-4 * np.abs(want), 1e-6)).all())
        for name, g in zip(("grad_background", "grad_points", "grad_pose", "grad_intrinsics"), grads[1:]):
            want = getattr(refb, name)
            if g is not None and want is not None:
                e = float(np.abs(g.cpu().numpy().astype(np.float64) - want).max() / max(float(np.abs(want).max()), 1e-30))
                m[name + "_norm_err"] = e
                m[name + "_within_1e-4"] = e <= 1e-4
        del grads
    m["all"] = all(v for k, v in m.items() if isinstance(v, bool))
    del cache, info, ctx, images
    torch.cuda.empty_cache()
    return m


def run_workload(args, workload, steps, warmup, lib, point_order=None, lod=False, cpu_leg=True, graph=True):
    """Measures one render workload; returns the JSON object of its bench line."""
    import numpy as np
    import torch
    from adop_amd import _capi, render, scenes

    dev = "cuda:0"
    t0 = time.time()
    point_order = point_order or args.point_order
    hs = make_scene(args, workload, point_order, lod)
    backward = workload not in ("config1", "config4")
    with_env = workload == "config5" and hs.env_texture is not None and not args.no_env
    gen_s = time.time() - t0

    scene = render.NeuralScene.from_host(hs, dev)
    cache = render.PointRendererCache()
    info = render.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params, num_layers=hs.num_layers,
                                   cache=cache, train=backward and not args.no_point_cache,
                                   workspace_flags=args.workspace_flags,
                                   dropout_points=None if hs.dropout is None else torch.from_numpy(hs.dropout))
    hs.params.workspace_flags = args.workspace_flags
    cache.Build(info, True)
    s = scene.struct()
    fb = cache.forward_struct()
    views = cache.views_array()
    B, N, Cn, L = hs.batch, hs.num_points, hs.num_channels, hs.num_layers
    ws = C.c_void_p(cache.workspace.data_ptr())
    ws_n = cache.workspace.numel()
    stream_of = [C.c_void_p(torch.cuda.current_stream().cuda_stream)]

    gb = None
    keep = []
    if backward:
        gout = [torch.from_numpy(g).to(dev) for g in scenes.upstream_grads(hs)]
        gb = _capi.BackwardBuffers()
        for l in range(L):
            gb.grad_out[l] = gout[l].data_ptr()
        g_tex = torch.empty(scene.texture.shape, dtype=torch.float32, device=dev)
        g_bg = torch.empty(Cn, dtype=torch.float32, device=dev)
        g_pts = torch.empty(N, 4, dtype=torch.float32, device=dev)
        g_pts_c = torch.empty(N, dtype=torch.float32, device=dev)
        g_pose = torch.empty(scene.poses_se3.shape[0], 6, dtype=torch.float64, device=dev)
        g_pose_c = torch.empty(scene.poses_se3.shape[0], dtype=torch.float32, device=dev)
        g_intr = torch.empty_like(scene.intrinsics)
        g_intr_c = torch.empty(scene.intrinsics.shape[0], dtype=torch.float32, device=dev)
        keep = [gout, g_tex, g_bg, g_pts, g_pts_c, g_pose, g_pose_c, g_intr, g_intr_c]
        gb.grad_texture, gb.grad_background = g_tex.data_ptr(), g_bg.data_ptr()
        gb.grad_points, gb.grad_points_count = g_pts.data_ptr(), g_pts_c.data_ptr()
        if workload in ("config3", "crops"):
            gb.grad_pose, gb.grad_pose_count = g_pose.data_ptr(), g_pose_c.data_ptr()
            gb.grad_intrinsics, gb.grad_intrinsics_count = g_intr.data_ptr(), g_intr_c.data_ptr()
    env_args = None
    if with_env:
        env = scene.environment_map
        g_env = torch.empty_like(env)
        gout_arr = (C.c_void_p * L)(*[g.data_ptr() for g in gout])
        # the texture coordinates travel from the forward to the backward call (the reference's autograd saves them too)
        uvs = [torch.empty(B, h, w, 2, dtype=torch.float32, device=dev) for (w, h) in hs.level_sizes()]
        uv_arr = (C.c_void_p * L)(*[t.data_ptr() for t in uvs])
        # the composed images go to buffers of their own (the reference composes out of place, RenderModule.cpp:121-125):
        # the backward pass sees the rasterizer's own output
        composed = [torch.empty_like(o) for o in cache.output_forward]
        comp_arr = (C.c_void_p * L)(*[t.data_ptr() for t in composed])
        env_args = (C.c_void_p(env.data_ptr()), int(env.shape[1]), int(env.shape[2]), gout_arr, C.c_void_p(g_env.data_ptr()),
                    uv_arr, comp_arr)
        keep += [g_env, uvs, composed]

    frame = [0]
    env_events = []  # (name, start, stop) torch events around the environment-map calls while profiling

    def fail():
        raise RuntimeError(lib.adop_last_error_string().decode())

    def step(stats=None, timed_env=False):
        if workload == "config4":
            views[0].image_index = frame[0] % scene.poses_se3.shape[0]  # the orbit: 1.2 degrees per frame
            frame[0] += 1
        if lib.adop_forward(C.byref(s), views, B, C.byref(hs.params), C.byref(fb), ws, ws_n, stats, stream_of[0]) != 0:
            fail()
        if with_env:
            # spherical environment map sampled at the empty pixels of the OCam views, added to the images
            if timed_env:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            if lib.adop_env_sample(C.byref(s), views, B, env_args[0], env_args[1], env_args[2], C.byref(fb), env_args[5],
                                   env_args[6], 2, stream_of[0]) != 0:
                fail()
            if timed_env:
                e1.record()
                env_events.append(("EnvironmentMap", e0, e1))
        if backward:
            if lib.adop_backward(C.byref(s), views, B, C.byref(hs.params), C.byref(fb), C.byref(gb), ws, ws_n, stats,
                                 stream_of[0]) != 0:
                fail()
        if with_env:
            if timed_env:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            if lib.adop_env_sample_backward(C.byref(s), views, B, env_args[1], env_args[2], C.byref(fb), env_args[3],
                                            env_args[5], env_args[4], stream_of[0]) != 0:
                fail()
            if timed_env:
                e1.record()
                env_events.append(("EnvironmentMapBackward", e0, e1))

    copy_gbs = None
    if args.calibrate_copy:
        # plain device copy of 1 GiB (2 GiB of traffic): what the memory system delivers to the simplest kernel
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        copy_gbs = 10 * 2 * src.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9
        del src, dst

    # untimed pass with counters: V_l, A_l, G_l of the byte model
    step(C.c_void_p(cache.stats.data_ptr()))
    torch.cuda.synchronize()
    st = cache.read_stats()
    V, A, G = list(st.visible)[:L], list(st.accepted)[:L], list(st.spatial)[:L]
    empty_pixels = 0
    if with_env:
        empty_pixels = int(sum(int((m == 0).sum().item()) for m in cache.output_forward_background_mask))

    frame[0] = 0
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    ms_per_step = (t2 - t1) * 1e3 / steps

    # per-stage durations from HIP events on the launch stream
    lib.adop_profile_enable(1)
    prof_steps = min(steps, 50)
    for _ in range(prof_steps):
        step(timed_env=True)
    torch.cuda.synchronize()
    arr = (_capi.StageTime * 16)()
    n = lib.adop_profile_read(arr, 16)
    lib.adop_profile_enable(0)
    stages = {arr[i].name.decode(): arr[i].total_ms / prof_steps for i in range(n)}  # ms per step
    for name, e0, e1 in env_events:
        stages[name] = stages.get(name, 0.0) + e0.elapsed_time(e1) / prof_steps

    # the same step recorded once into a HIP graph and replayed (outside the timed region above: what the host-side
    # launches cost); configuration 4 changes a host-side argument every frame and is not recorded
    graph_ms = None
    if workload != "config4" and not args.no_graph and graph:
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        eager_stream = stream_of[0]
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                stream_of[0] = C.c_void_p(side.cuda_stream)
                step()
        stream_of[0] = eager_stream
        for _ in range(max(warmup, 1)):
            graph.replay()
        torch.cuda.synchronize()
        tg = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - tg) * 1e3 / steps
        del graph

    P_levels = [w * h for (w, h) in hs.level_sizes()]
    P = sum(P_levels)
    S_d = 2 if hs.texture.dtype == np.float16 else 4
    model = byte_model(N, B, Cn, S_d, P, V, A, G, bool(hs.params.output_background_mask), hs.dropout is not None)
    if "TileBlend" in stages:
        model = tile_path_model(model, N, B, Cn, P_levels, V, hs.dropout is not None)
    if not backward:
        model = {k: v for k, v in model.items() if k in ("DepthPrepass", "RenderForward", "CombineAndFill", "BinCount",
                                                         "BinScatter", "TileDepth", "TileBlend")}
    if with_env:
        # every pixel reads its mask and the image and writes the composed image, an empty one also stores its uv and
        # reads its four taps per channel; backward: mask, uv, upstream gradient and the read-modify-write of the taps
        model["EnvironmentMap"] = B * P * (4 + 8 * Cn) + empty_pixels * (8 + 16 * Cn)
        model["EnvironmentMapBackward"] = B * P * 4 + empty_pixels * (8 + 4 * Cn + 2 * 16 * Cn)
    total_bytes = sum(model.values())
    dom = max((k for k in model if k in stages), key=lambda k: stages[k])
    dom_gbs = model[dom] / (stages[dom] * 1e-3) / 1e9

    # measured HBM traffic (rocprofv3 counters), for the exact workload and kernel state the profile was taken on
    measured, measured_from = {}, None
    tab = MEASURED_TRAFFIC.get(workload)
    if (tab and not args.points and point_order == "morton" and not args.no_point_cache
            and not lod and tab.get("sources") == kernel_sources_state()):
        measured = {k: v for k, v in tab["bytes"].items() if k in stages}
        measured_from = {"profile": tab["profile"], "sources": tab["sources"]}
    step_measured = None  # every stage of the step that moves memory has a figure
    if measured and all(k in measured for k in stages if k != "Prepare Backward"):
        step_measured = sum(measured.values())
    roofline = {"bound": "hbm", "kernel": KERNEL_OF_STAGE.get(dom, dom), "stage": dom, "achieved": round(dom_gbs, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                "traffic": measured.get(dom), "traffic_from": measured_from if dom in measured else None,
                "kernel_ms": round(stages[dom], 4), "algorithmic_bytes": int(model[dom])}
    step_gbs = total_bytes / (ms_per_step * 1e-3) / 1e9
    # a stage whose algorithmic bytes exceed what it moves (neighbouring points share lines through the L2) is charged
    # its measured bytes in hbm_frac_dedup, so that no stage is credited with more than it moves
    dedup_bytes = sum(min(model[k], measured.get(k, model[k])) for k in model) if measured else None

    if workload in ("config4", "config1"):
        what = "100M" if workload == "config4" else str(N)
        metric, unit, value = f"forward frames/s at {what} points {hs.views[0].w}x{hs.views[0].h} x{L} levels", "frames/s", 1e3 / ms_per_step
    else:
        metric, unit = "fwd+bwd points/s", "points/s"
        value = N * B / (ms_per_step * 1e-3)

    cpu = None
    if cpu_leg and not args.no_cpu_baseline:
        import copy
        import oracle
        nthreads = host_threads()
        chs, sample, full = hs, "the full workload", True
        cpu_n = args.cpu_points or 0
        if workload == "config5":
            # one of the 8 views (the others cost the same per view: stated, not measured)
            chs = copy.copy(hs)
            chs.views, chs.dropout = hs.views[:1], None if hs.dropout is None else np.ascontiguousarray(hs.dropout[:1])
            sample, full = f"view 0 of {B} at the full point count and resolution, forward + backward (points/s counts that one view)", False
        if workload == "crops":
            chs = copy.copy(hs)
            chs.views, chs.dropout = hs.views[:4], np.ascontiguousarray(hs.dropout[:4])
            sample, full = f"the 4 crops of frame 0 (of {B}) at the full point count, forward + backward", False
        if cpu_n and cpu_n < N:
            chs = copy.copy(chs)
            chs.position, chs.index = hs.position[:cpu_n], hs.index[:cpu_n]
            chs.normal = None if hs.normal is None else hs.normal[:cpu_n]
            chs.dropout = None if chs.dropout is None else np.ascontiguousarray(chs.dropout[:, :cpu_n])
            sample, full = f"first {cpu_n} of {N} points; " + sample, False
        # one untimed warm-up run, then three timed ones: the median is the figure (config 4: the three runs are the
        # orbit frames 0, 100 and 200, the warm-up is frame 50)
        frames_cpu = [50, 0, 100, 200] if workload == "config4" else [0, 0, 0, 0]
        if workload == "config4":
            sample = "the full cloud, forward; warm-up on orbit frame 50, then frames 0, 100 and 200"
        cgout = scenes.upstream_grads(chs) if backward else None
        oracle.lib(True)  # load outside the timed region
        runs, matches = [], None
        for k, f in enumerate(frames_cpu):
            if workload == "config4":
                chs.views[0].image_index = f
            tc0 = time.perf_counter()
            ref = oracle.forward(chs, omp=True)
            refb = oracle.backward(chs, ref, cgout, omp=True) if backward else None
            if k > 0:
                runs.append(time.perf_counter() - tc0)
            if k == len(frames_cpu) - 1 and not cpu_n:
                matches = compare_with_checker(lib, scene, chs, ref, refb, cgout, full)
                matches["sample"] = "the buffers of the last timed run" + (f" (orbit frame {f})" if workload == "config4" else "")
            del ref, refb
        tc = sorted(runs)[len(runs) // 2]
        if workload == "config4":
            chs.views[0].image_index = 0
        used = oracle.lib(True).oracle_num_threads()
        if workload in ("config4", "config1"):
            cpu_val, cpu_unit = (chs.num_points / N) / tc, "frames/s"
        else:
            cpu_val, cpu_unit = chs.num_points * chs.batch / tc, "points/s"
        cpu = {"value": cpu_val, "unit": cpu_unit, "cores": used, "kind": "port",
               "sample": sample + "; one warm-up run, median of three timed runs",
               "seconds": round(tc, 4), "seconds_runs": [round(r, 4) for r in runs], "host_cpus": os.cpu_count(),
               "threads_from": "OMP_NUM_THREADS" if os.environ.get("OMP_NUM_THREADS") else "os.cpu_count()",
               "matches_gpu": matches}
        assert used == nthreads or used >= 1

    out = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if S_d == 4 else "f16-stored/f32-accumulated", "data": "synthetic",
        "config": {"workload": (f"BASELINE {hs.name}" if hs.name.startswith("config") else "training batch of 4 frames x 4 crops of config3") +
                               f": {N} points, B={B}, {hs.views[0].w}x{hs.views[0].h}, "
                               f"{L} levels, C={Cn}, " + ("forward+backward" if backward else "forward only") +
                               (", spherical environment map on the OCam views with its gradient" if with_env else "") +
                               (", 300-pose orbit of radius 12, 1.2 degrees per frame" if workload == "config4" else ""),
                   "point_order": hs.meta.get("point_order", "as generated"),
                   "lod_radius_test": bool(hs.params.drop_out_points_by_radius),
                   "dropout": 0.25 if hs.dropout is not None else 0.0,
                   "ghost_gradients": bool(hs.params.ghost_gradients)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "step": {"algorithmic_bytes": int(total_bytes), "achieved_GBps": round(step_gbs, 1),
                 "hbm_frac": round(step_gbs / HBM_PEAK_GBS, 4),
                 "measured_bytes": None if step_measured is None else int(step_measured),
                 "hbm_frac_measured": None if step_measured is None else round(step_measured / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                 "hbm_frac_dedup": None if dedup_bytes is None else round(dedup_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                 "measured_from": measured_from,
                 "workspace_bytes": int(ws_n),
                 "saved_for_backward_bytes": int((0 if cache.point_cache is None else cache.point_cache.numel() * 4) +
                                                 (0 if cache.pixel_cache is None else cache.pixel_cache.numel() * 4)),
                 "stage_ms": {k: round(v, 4) for k, v in stages.items()},
                 "stage_GBps": {k: round(model[k] / (stages[k] * 1e-3) / 1e9, 1) for k in model if k in stages},
                 "stage_GBps_measured": {k: round(measured[k] / (stages[k] * 1e-3) / 1e9, 1) for k in measured} or None,
                 "stages_model_above_peak": [k for k in model if k in stages and model[k] / (stages[k] * 1e-3) / 1e9 > HBM_PEAK_GBS],
                 "visible": V, "accepted": A, "spatial": G, "scene_gen_s": round(gen_s, 1),
                 "graph_replay_ms_per_step": None if graph_ms is None else round(graph_ms, 4),
                 "device_copy_GBps": None if copy_gbs is None else round(copy_gbs, 1)},
    }
    if with_env:
        out["step"]["empty_pixels"] = empty_pixels
    del keep, cache, scene, info, hs
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0, help="timed steps (default 20; 300 = the whole orbit for config4)")
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="config3",
                    choices=["config1", "config2", "config3", "config4", "config5", "crops", "preprocess"])
    ap.add_argument("--points", type=int, default=0, help="override the point count (0 = the configuration's)")
    ap.add_argument("--point-order", default="morton", choices=["morton", "random"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-config4", action="store_true",
                    help="default workload only: do not measure the 100 M-point orbit after config3")
    ap.add_argument("--headline-only", action="store_true",
                    help="default workload only: leave out the other configurations (step.configs)")
    ap.add_argument("--print-sources-state", action="store_true",
                    help="print kernel_sources_state() (what a MEASURED_TRAFFIC table is keyed on) and exit")
    ap.add_argument("--workspace-flags", type=int, default=0,
                    help="adop_workspace_size_for flags: 1 point cache kept, 2 no tile path, 4 small bins")
    ap.add_argument("--tuning", default="",
                    help="adop_tuning fields for the whole run, e.g. tile_k=2,count_ppt=4 (A/B runs of the library's switches)")
    ap.add_argument("--no-env", action="store_true", help="config5 without the environment-map passes")
    ap.add_argument("--no-graph", action="store_true", help="do not replay the step from a HIP graph as well")
    ap.add_argument("--no-point-cache", action="store_true",
                    help="do not keep the projected points for the backward pass (it projects again)")
    ap.add_argument("--cpu-points", type=int, default=0, help="point count of the CPU sample (0 = the full cloud)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.print_sources_state:
        print(kernel_sources_state())
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (one process, one MI355X); "
              "a figure at several GPUs is not produced. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    from adop_amd import _capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    lib = _capi.load_library()
    torch.cuda.set_device(0)
    if args.tuning:
        t = _capi.Tuning()
        lib.adop_get_tuning(C.byref(t))
        for kv in args.tuning.split(","):
            k, v = kv.split("=")
            if not hasattr(t, k):
                sys.exit(f"bench.py: unknown tuning field {k}")
            setattr(t, k, int(v))
        if lib.adop_set_tuning(C.byref(t)) != 0:
            sys.exit("bench.py: " + lib.adop_last_error_string().decode())
    if args.workload == "preprocess":
        args.steps = args.steps or 20
        print(json.dumps(bench_preprocess(args)))
        return

    steps = args.steps or (300 if args.workload == "config4" else 20)
    out = run_workload(args, args.workload, steps, args.warmup, lib)

    def brief(r):
        """The figures of a further workload that go into step.configs of the default line."""
        st = r["step"]
        return {"metric": r["metric"], "value": round(r["value"], 2), "unit": r["unit"], "steps": r["steps"],
                "ms_per_step": round(r["ms_per_step"], 4), "workload": r["config"]["workload"],
                "point_order": r["config"]["point_order"], "lod_radius_test": r["config"]["lod_radius_test"],
                "dtype": r["dtype"], "roofline": r["roofline"], "cpu_baseline": r["cpu_baseline"],
                "hbm_frac": st["hbm_frac"], "hbm_frac_measured": st["hbm_frac_measured"],
                "achieved_GBps": st["achieved_GBps"], "algorithmic_bytes": st["algorithmic_bytes"],
                "measured_bytes": st["measured_bytes"], "workspace_bytes": st["workspace_bytes"],
                "saved_for_backward_bytes": st["saved_for_backward_bytes"], "stage_ms": st["stage_ms"],
                "stage_GBps": st["stage_GBps"], "scene_gen_s": st["scene_gen_s"]}

    default_run = args.workload == "config3" and not args.points and args.point_order == "morton"
    if default_run and not args.no_config4:
        # the second headline figure: forward frames/s at 100 M points over the whole 300-frame orbit
        c4 = run_workload(args, "config4", 300, args.warmup, lib)
        out["step"]["config4"] = dict(brief(c4), frames=c4["steps"], ms_per_frame=round(c4["ms_per_step"], 4),
                                      target_frames_per_s=60)
    if default_run and not args.headline_only:
        # Every other BASELINE configuration and the reference's training shape, and the two headline configurations
        # once more in random point order and with the reference's default LOD radius test.  Fewer steps each, no graph
        # replay; the CPU leg only where the work differs from a configuration already timed on the CPU.
        cf = {}
        few = max(5, min(steps, 10))
        cf["config3_random_order"] = brief(run_workload(args, "config3", few, args.warmup, lib, point_order="random",
                                                        cpu_leg=False, graph=False))
        cf["config3_lod_radius_test"] = brief(run_workload(args, "config3", few, args.warmup, lib, lod=True, graph=False))
        if not args.no_config4:
            cf["config4_random_order"] = brief(run_workload(args, "config4", 100, args.warmup, lib, point_order="random",
                                                            cpu_leg=False))
            cf["config4_lod_radius_test"] = brief(run_workload(args, "config4", 300, args.warmup, lib, lod=True, cpu_leg=False))
        cf["config1"] = brief(run_workload(args, "config1", 100, args.warmup, lib, graph=False))
        cf["config2"] = brief(run_workload(args, "config2", 50, args.warmup, lib, graph=False))
        cf["config5"] = brief(run_workload(args, "config5", few, args.warmup, lib, graph=False))
        cf["crops"] = brief(run_workload(args, "crops", few, args.warmup, lib, graph=False))
        out["step"]["configs"] = cf
        # the pass line of the headline workload: bytes really moved / step time against the 8 TB/s peak, next to the
        # fraction by algorithmic bytes
        out["step"]["pass_line"] = {"hbm_frac_algorithmic": out["step"]["hbm_frac"],
                                    "hbm_frac_measured": out["step"]["hbm_frac_measured"], "target": 0.60}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
