#!/usr/bin/env python3
"""Benchmark of the point-rasterizer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config3|config2|config4|config5]

A step is one pass of the hot path over one batch of synthetic input that already sits in HBM:
``adop_forward`` + ``adop_backward`` through the C-ABI (forward only for the viewer workload config4).
Prints ONE JSON line.  Default workload: BASELINE config 3 (10 M points, 1920x1080, 4 levels, 8 channels,
forward + backward with descriptor / point / pose / intrinsics gradients) -> points/s.

``roofline`` describes the slowest kernel of the step: algorithmic bytes of that kernel (byte model below, with
the point-level counts V/A/G measured by the kernels' own counters in an untimed pass) divided by its average
duration measured with HIP events on the launch stream, against the 8 TB/s HBM peak.
``cpu_baseline`` times the CPU checker (OpenMP build) on the host cores for the same workload (or a bounded
sample of it).
"""
import argparse
import ctypes as C
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
                   "RenderBackward/spatial": "backward_ghost_kernel"}


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
    print(json.dumps({
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
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="config3", choices=["config2", "config3", "config4", "config5", "preprocess"])
    ap.add_argument("--points", type=int, default=0, help="override the point count (0 = the configuration's)")
    ap.add_argument("--point-order", default="morton", choices=["morton", "random"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-point-cache", action="store_true",
                    help="do not keep the projected points for the backward pass (it projects again)")
    ap.add_argument("--cpu-points", type=int, default=0, help="point count of the CPU sample (0 = automatic)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (one process, one MI355X); "
              "a figure at several GPUs is not produced. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from adop_amd import _capi, render, scenes

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    lib = _capi.load_library()
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.workload == "preprocess":
        bench_preprocess(args)
        return

    t0 = time.time()
    kw = {"n": args.points} if args.points else {}
    if args.workload == "config3":
        hs = scenes.config3(point_order=args.point_order, **kw)
    elif args.workload == "config2":
        hs = scenes.config2(point_order=args.point_order, **kw)
    elif args.workload == "config4":
        hs = scenes.config4(point_order=args.point_order, **kw)
    else:
        hs = scenes.config5(point_order=args.point_order, **kw)
    backward = args.workload != "config4"
    gen_s = time.time() - t0

    scene = render.NeuralScene.from_host(hs, dev)
    cache = render.PointRendererCache()
    info = render.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params, num_layers=hs.num_layers,
                                   cache=cache, train=backward and not args.no_point_cache,
                                   dropout_points=None if hs.dropout is None else torch.from_numpy(hs.dropout))
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
        if args.workload in ("config3",):
            gb.grad_pose, gb.grad_pose_count = g_pose.data_ptr(), g_pose_c.data_ptr()
            gb.grad_intrinsics, gb.grad_intrinsics_count = g_intr.data_ptr(), g_intr_c.data_ptr()

    frame = [0]

    def step(stats=None):
        if args.workload == "config4":
            views[0].image_index = frame[0] % scene.poses_se3.shape[0]  # orbit
            frame[0] += 1
        rc = lib.adop_forward(C.byref(s), views, B, C.byref(hs.params), C.byref(fb), ws, ws_n, stats, stream_of[0])
        if rc != 0:
            raise RuntimeError(lib.adop_last_error_string().decode())
        if backward:
            rc = lib.adop_backward(C.byref(s), views, B, C.byref(hs.params), C.byref(fb), C.byref(gb), ws, ws_n,
                                   stats, stream_of[0])
            if rc != 0:
                raise RuntimeError(lib.adop_last_error_string().decode())

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

    frame[0] = 0
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    ms_per_step = (t2 - t1) * 1e3 / args.steps

    # per-stage durations from HIP events on the launch stream
    lib.adop_profile_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    arr = (_capi.StageTime * 16)()
    n = lib.adop_profile_read(arr, 16)
    lib.adop_profile_enable(0)
    stages = {arr[i].name.decode(): arr[i].total_ms / args.steps for i in range(n)}  # ms per step

    # the same step recorded once into a HIP graph and replayed (outside the timed region above: what the host-side
    # launches cost); configuration 4 changes a host-side argument every frame and is not recorded
    graph_ms = None
    if args.workload != "config4":
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        eager_stream = stream_of[0]
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                stream_of[0] = C.c_void_p(side.cuda_stream)
                step()
        stream_of[0] = eager_stream
        for _ in range(max(args.warmup, 1)):
            graph.replay()
        torch.cuda.synchronize()
        tg = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - tg) * 1e3 / args.steps

    P = sum(w * h for (w, h) in hs.level_sizes())
    S_d = 2 if hs.texture.dtype == np.float16 else 4
    model = byte_model(N, B, Cn, S_d, P, V, A, G, bool(hs.params.output_background_mask), hs.dropout is not None)
    if "TileBlend" in stages:
        model = tile_path_model(model, N, B, Cn, [w * h for (w, h) in hs.level_sizes()], V, hs.dropout is not None)
    if not backward:
        model = {k: v for k, v in model.items() if k in ("DepthPrepass", "RenderForward", "CombineAndFill", "BinCount",
                                                         "BinScatter", "TileDepth", "TileBlend")}
    total_bytes = sum(model.values())
    dom = max((k for k in model if k in stages), key=lambda k: stages[k])
    dom_gbs = model[dom] / (stages[dom] * 1e-3) / 1e9
    # HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch,
    # FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0 after calibration with plain device copies); measured for the default
    # workload only
    measured_traffic = {}
    if args.workload == "config3" and not args.points and args.point_order == "morton" and not args.no_point_cache:
        # profiles/config3_tile_path_fwd_bwd_kernels_traffic_instructions.md, profiles/config3_direct_path_fwd_bwd_kernels_traffic_instructions.md
        measured_traffic = {"RenderBackward/descriptor": 912.7e6, "RenderBackward/spatial": 486.2e6, "TileBlend": 438.1e6,
                            "BinCount": 436.4e6, "BinScatter": 196.9e6, "TileDepth": 101.0e6,
                            "CombineAndFillBackward": 397.3e6, "RenderForward": 611.0e6, "DepthPrepass": 578.9e6}
    if args.workload == "config4" and not args.points and args.point_order == "morton":
        # profiles/config4_direct_path_forward_kernels_traffic_instructions.md
        measured_traffic = {"DepthPrepass": 5053.5e6, "RenderForward": 1548.3e6}
    roofline = {"bound": "hbm", "kernel": KERNEL_OF_STAGE.get(dom, dom), "stage": dom, "achieved": round(dom_gbs, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom_gbs / HBM_PEAK_GBS, 4),
                "traffic": measured_traffic.get(dom),
                "kernel_ms": round(stages[dom], 4), "algorithmic_bytes": int(model[dom])}
    step_gbs = total_bytes / (ms_per_step * 1e-3) / 1e9

    if args.workload == "config4":
        metric, unit, value = "forward frames/s at 100M points 1920x1080 x5 levels", "frames/s", 1e3 / ms_per_step
    else:
        metric, unit = "fwd+bwd points/s", "points/s"
        value = N * B / (ms_per_step * 1e-3)

    cpu = None
    if not args.no_cpu_baseline:
        import oracle
        cores = min(os.cpu_count() or 1, 16)
        os.environ["OMP_NUM_THREADS"] = str(cores)
        chs, sample = hs, "the full workload, one step"
        cpu_n = args.cpu_points or (20_000_000 if N > 20_000_000 else 0)
        if cpu_n and cpu_n < N:
            # bounded sample: the first cpu_n points of the same cloud at the same resolution
            import copy
            chs = copy.copy(hs)
            chs.position, chs.index = hs.position[:cpu_n], hs.index[:cpu_n]
            chs.normal = None if hs.normal is None else hs.normal[:cpu_n]
            chs.dropout = None if hs.dropout is None else np.ascontiguousarray(hs.dropout[:, :cpu_n])
            sample = f"first {cpu_n} of {N} points, same resolution, one step"
        tc0 = time.perf_counter()
        ref = oracle.forward(chs, omp=True)
        if backward:
            oracle.backward(chs, ref, scenes.upstream_grads(chs), omp=True)
        tc = time.perf_counter() - tc0
        nthreads = oracle.lib(True).oracle_num_threads()
        if args.workload == "config4":
            cpu_val, cpu_unit = (chs.num_points / N) / tc, "frames/s"
            sample += " (frames/s scaled linearly to the full point count)"
        else:
            cpu_val, cpu_unit = chs.num_points * B / tc, "points/s"
        cpu = {"value": cpu_val, "unit": cpu_unit, "cores": nthreads, "kind": "port", "sample": sample,
               "seconds": round(tc, 3)}

    out = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if S_d == 4 else "f16-stored/f32-accumulated", "data": "synthetic",
        "config": {"workload": f"BASELINE {hs.name}: {N} points, B={B}, {hs.views[0].w}x{hs.views[0].h}, "
                               f"{L} levels, C={Cn}, " + ("forward+backward" if backward else "forward only"),
                   "point_order": hs.meta.get("point_order", "as generated"), "lod_radius_test": False,
                   "dropout": 0.25 if hs.dropout is not None else 0.0,
                   "ghost_gradients": bool(hs.params.ghost_gradients)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "step": {"algorithmic_bytes": int(total_bytes), "achieved_GBps": round(step_gbs, 1),
                 "hbm_frac": round(step_gbs / HBM_PEAK_GBS, 4),
                 "stage_ms": {k: round(v, 4) for k, v in stages.items()},
                 "stage_GBps": {k: round(model[k] / (stages[k] * 1e-3) / 1e9, 1) for k in model if k in stages},
                 "visible": V, "accepted": A, "spatial": G, "scene_gen_s": round(gen_s, 1),
                 "graph_replay_ms_per_step": None if graph_ms is None else round(graph_ms, 4),
                 "device_copy_GBps": None if copy_gbs is None else round(copy_gbs, 1)},
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
