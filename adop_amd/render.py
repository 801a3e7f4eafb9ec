"""Host-side mirror of the reference's render interface on top of the C-ABI (``include/adop_raster.h``).

Names, argument order and return order follow the reference so that its callers map one to one:

==============================  ===================================================================
here                            reference
==============================  ===================================================================
``NeuralPointCloud``            ``NeuralPointCloudCudaImpl`` (rendering/NeuralPointCloudCuda.h:19-45)
``NeuralScene``                 the tensors ``NeuralScene`` owns that the render stage reads
                                (texture/background, point cloud, poses, intrinsics; data/NeuralScene.h)
``NeuralRenderInfo``            rendering/PointRenderer.h:25-34
``PointRendererCache``          rendering/PointRenderer.h:96-157 (Build/Allocate, realloc key {C,N,L,B,h,w})
``PointRender``                 ``torch::autograd::PointRender`` (PointRenderer.h:39-46, RenderInfo.cpp:34-59)
``BlendPointCloud``             RenderInfo.cpp:19-30
``ApplyTangentToPose``          PointRenderer.cu:1659-1665
==============================  ===================================================================

torch is used for device memory and the current stream only; all arithmetic happens in the HIP library.
"""
import ctypes as C
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import _capi


def _ptr(t):
    return None if t is None else t.data_ptr()


def _check(rc, lib):
    if rc != _capi.ADOP_OK:
        raise RuntimeError(f"adop_raster error {rc}: {lib.adop_last_error_string().decode()}")


class NeuralPointCloud:
    """``t_position [N,4] f32``, ``t_normal [N,1] i32`` (10-bit packed) or None, ``t_index [N,1] i32``."""

    def __init__(self, position, normal, index, device="cuda"):
        self.t_position = torch.as_tensor(position, dtype=torch.float32).to(device).contiguous()
        self.t_normal = None if normal is None else torch.as_tensor(normal, dtype=torch.int32).to(device).reshape(-1, 1).contiguous()
        self.t_index = torch.as_tensor(index, dtype=torch.int32).to(device).reshape(-1, 1).contiguous()
        assert self.t_position.dim() == 2 and self.t_position.shape[1] == 4
        assert self.t_index.shape[0] == self.t_position.shape[0]
        self._index_is_identity = None

    def index_is_identity(self):
        """True if t_index[i] == i for all i (how the reference builds it); evaluated once and cached."""
        if self._index_is_identity is None:
            n = self.Size()
            ar = torch.arange(n, dtype=torch.int32, device=self.t_index.device)
            self._index_is_identity = bool((self.t_index.view(-1) == ar).all().item())
        return self._index_is_identity

    def Size(self):
        return int(self.t_position.shape[0])


class NeuralScene:
    """The per-scene tensors the render stage consumes."""

    def __init__(self, point_cloud, texture, background_color, poses_se3, intrinsics, tangent_poses=None,
                 environment_map=None):
        dev = point_cloud.t_position.device
        self.point_cloud_cuda = point_cloud
        self.texture = texture.to(dev).contiguous()  # [C,N] f32 | f16
        self.background_color = background_color.to(dev, torch.float32).contiguous()
        self.poses_se3 = poses_se3.to(dev, torch.float64).contiguous()  # [F,8]
        self.tangent_poses = (torch.zeros(self.poses_se3.shape[0], 6, dtype=torch.float64, device=dev)
                              if tangent_poses is None else tangent_poses)
        self.intrinsics = intrinsics.to(dev, torch.float32).contiguous()  # [K,13] | [K,5+P]
        self.environment_map = None if environment_map is None else environment_map.to(dev, torch.float32).contiguous()

    @classmethod
    def from_host(cls, hs, device="cuda"):
        pc = NeuralPointCloud(hs.position, hs.normal, hs.index, device)
        return cls(pc, torch.from_numpy(hs.texture), torch.from_numpy(hs.background),
                   torch.from_numpy(hs.poses_se3), torch.from_numpy(hs.intrinsics),
                   environment_map=None if hs.env_texture is None else torch.from_numpy(hs.env_texture))

    def struct(self):
        s = _capi.Scene()
        pc = self.point_cloud_cuda
        s.position = _ptr(pc.t_position)
        s.normal = _ptr(pc.t_normal)
        s.index = _ptr(pc.t_index)
        s.num_points = pc.Size()
        s.texture = _ptr(self.texture)
        s.texture_dtype = _capi.TEXTURE_F16 if self.texture.dtype == torch.float16 else _capi.TEXTURE_F32
        s.num_channels = int(self.texture.shape[0])
        s.num_texels = int(self.texture.shape[1])
        s.background_color = _ptr(self.background_color)
        s.poses_se3 = _ptr(self.poses_se3)
        s.num_poses = int(self.poses_se3.shape[0])
        s.intrinsics = _ptr(self.intrinsics)
        s.num_cameras = int(self.intrinsics.shape[0])
        s.intrinsics_cols = int(self.intrinsics.shape[1])
        s.index_is_identity = 1 if (pc.index_is_identity() and s.num_texels == s.num_points) else 0
        return s


@dataclass
class LayerCuda:
    """rendering/PointRenderer.h:65-94"""
    size: tuple = (0, 0)  # (w, h)
    scale: float = 1.0
    depth: Optional[torch.Tensor] = None
    weight: Optional[torch.Tensor] = None
    depth_index_tensor: Optional[torch.Tensor] = None  # int64 storage of the packed u64


@dataclass
class NeuralRenderInfo:
    scene: NeuralScene = None
    images: List[_capi.View] = field(default_factory=list)
    params: _capi.RenderParams = None
    num_layers: int = 0
    cache: "PointRendererCache" = None
    # The reference draws the dropout mask inside the cache (bernoulli_, PointRenderer.cu:1083).  Passing it here
    # makes a run reproducible; None + dropout>0 draws it with torch.  A host tensor is copied to the device by every
    # forward pass (4 bytes per point and view): hand in a device tensor where that matters.
    dropout_points: Optional[torch.Tensor] = None
    dropout: float = 0.0
    collect_stats: bool = False
    # RenderParams::debug_print_num_rendered_points (Settings.h:43): the sum of the weights after a forward pass
    debug_print_num_rendered_points: bool = False
    # NeuralRenderInfo::train (RenderInfo.h): a backward pass may follow, so the forward pass leaves the projected
    # points in a tensor of its own (saved like depth / weight) instead of the workspace
    train: bool = True
    # with train: the forward pass also leaves the resolved images pixel by pixel for the backward pass (one more
    # saved tensor of the size of the images); False: the backward pass builds those records from the images itself
    keep_pixel_records: bool = True
    # adop_workspace_size_for flags (_capi.WORKSPACE_*): a smaller workspace for a caller that always keeps the point
    # cache (train) and / or can do without the tile-bin forward path
    workspace_flags: int = 0


class PointRendererCache:
    """Buffer lifecycle of the render stage; reallocates only when {C,N,L,B,h,w} changes
    (PointRenderer.cu:952-1037)."""

    def __init__(self):
        self.lib = _capi.load_library()
        self.layers_cuda: List[LayerCuda] = []
        self.cache_size = None
        self.dropout_points = None
        self.point_cache = None
        self.pixel_cache = None
        self.output_forward = []
        self.output_forward_background_mask = []
        self.workspace = None
        self.stats = None
        self.info = None
        self.num_batches = 0

    # -- Allocate / InitializeData -------------------------------------------------------------
    def Build(self, info, forward):
        self.info = info
        self.num_batches = len(info.images)
        assert self.num_batches > 0
        self.Allocate(info, forward)
        if forward:
            self.InitializeData(forward)

    def Allocate(self, info, forward):
        fd = info.images[0]
        scene = info.scene
        dev = scene.texture.device
        new_size = (int(scene.texture.shape[0]), scene.point_cloud_cuda.Size(), info.num_layers, self.num_batches,
                    fd.h, fd.w, int(info.workspace_flags))
        if new_size == self.cache_size:
            return
        B = self.num_batches
        self.layers_cuda = []
        w, h, scale = fd.w, fd.h, 1.0
        for _ in range(info.num_layers):
            assert w > 0 and h > 0
            L = LayerCuda(size=(w, h), scale=scale)
            L.depth = torch.empty(B, 1, h, w, dtype=torch.float32, device=dev)
            L.weight = torch.empty(B, 1, h, w, dtype=torch.float32, device=dev)
            L.depth_index_tensor = torch.empty(B, 1, h, w, dtype=torch.int64, device=dev)
            self.layers_cuda.append(L)
            w //= 2
            h //= 2
            scale *= 0.5
        s = scene.struct()
        nbytes = self.lib.adop_workspace_size_for(C.byref(s), B, info.num_layers, fd.w, fd.h, int(info.workspace_flags))
        self.workspace = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=dev)
        self.stats = torch.zeros(C.sizeof(_capi.Stats) // 8, dtype=torch.int64, device=dev)
        self.cache_size = new_size

    def InitializeData(self, forward):
        info = self.info
        scene = info.scene
        dev = scene.texture.device
        B, Cn = self.num_batches, int(scene.texture.shape[0])
        # created every frame because it is moved to the caller (PointRenderer.cu:1050-1059); the HIP path clears
        # depth / weight / out itself, so plain empty() is enough here
        self.output_forward = [torch.empty(B, Cn, L.size[1], L.size[0], dtype=torch.float32, device=dev)
                               for L in self.layers_cuda]
        self.output_forward_background_mask = []
        if info.params.output_background_mask:
            self.output_forward_background_mask = [
                torch.empty(B, 1, L.size[1], L.size[0], dtype=torch.float32, device=dev) for L in self.layers_cuda]
        N = scene.point_cloud_cuda.Size()
        if info.dropout_points is not None:
            self.dropout_points = info.dropout_points.to(dev, torch.float32).contiguous()
            assert tuple(self.dropout_points.shape) == (B, N)
        elif info.dropout > 0:
            self.dropout_points = torch.empty(B, N, dtype=torch.float32, device=dev).bernoulli_(info.dropout)
        else:
            self.dropout_points = None  # zero_() in the reference; nothing is dropped
        # projected points, saved for the backward pass (handed to the autograd context like the outputs);
        # without a backward pass the library keeps them in its workspace
        self.point_cache = (torch.empty(B, N, 4, dtype=torch.float32, device=dev)
                            if (forward and info.train) else None)
        # the resolved images pixel by pixel, for the spatial gradients of the backward pass (saved like the outputs)
        pixels = B * sum(L.size[0] * L.size[1] for L in self.layers_cuda)
        self.pixel_cache = (torch.empty(pixels, Cn, dtype=torch.float32, device=dev)
                            if (forward and info.train and info.keep_pixel_records) else None)

    # -- C-ABI structs -----------------------------------------------------------------------
    def forward_struct(self):
        fb = _capi.ForwardBuffers()
        fb.num_layers = len(self.layers_cuda)
        for l, L in enumerate(self.layers_cuda):
            S = fb.layers[l]
            S.w, S.h = L.size
            S.depth_index = _ptr(L.depth_index_tensor)
            S.depth = _ptr(L.depth)
            S.weight = _ptr(L.weight)
            S.out = _ptr(self.output_forward[l])
            S.mask = _ptr(self.output_forward_background_mask[l]) if self.output_forward_background_mask else None
        fb.dropout_points = _ptr(self.dropout_points)
        fb.point_cache = _ptr(self.point_cache)
        fb.pixel_cache = _ptr(self.pixel_cache)
        return fb

    def views_array(self):
        arr = (_capi.View * self.num_batches)()
        for i, v in enumerate(self.info.images):
            arr[i] = v
        return arr

    def read_stats(self):
        host = self.stats.cpu().numpy().tobytes()
        return _capi.Stats.from_buffer_copy(host)


def _stream_ptr():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def BlendPointCloudForward(ctx, info, build=True):
    """PointRenderer.cu:1389-1531.  Returns (images per level, masks per level).  ``build=False``: the caller has
    already run ``cache.Build(info, True)`` (the reference calls it first thing, :1407)."""
    cache = info.cache
    if build:
        cache.Build(info, True)
    s = info.scene.struct()
    fb = cache.forward_struct()
    stats = C.c_void_p(cache.stats.data_ptr()) if info.collect_stats else None
    info.params.workspace_flags = int(info.workspace_flags)  # (how the cache sized the workspace)
    rc = cache.lib.adop_forward(C.byref(s), cache.views_array(), cache.num_batches, C.byref(info.params), C.byref(fb),
                                C.c_void_p(cache.workspace.data_ptr()), cache.workspace.numel(), stats, _stream_ptr())
    _check(rc, cache.lib)
    if info.debug_print_num_rendered_points:  # PointRenderer.cu:1502-1512
        weight_sum = 0.0
        for L in cache.layers_cuda:
            weight_sum += float(L.weight.sum().item())
        print(f"# Rasterized Points = {int(weight_sum)}", flush=True)
    if ctx is not None:
        save = []
        for L in cache.layers_cuda:
            save += [L.depth, L.weight]
        save += list(cache.output_forward)
        ctx.save_for_backward(*save)
        ctx.dropout_points = cache.dropout_points
        ctx.point_cache = cache.point_cache
        ctx.pixel_cache = cache.pixel_cache
        ctx.depth_index = [L.depth_index_tensor for L in cache.layers_cuda]
        ctx.masks = list(cache.output_forward_background_mask)
        # depth / weight / packed depth now belong to the graph (the kernels write them through raw pointers, autograd
        # would not notice a later forward overwriting them): the next forward allocates fresh ones
        cache.cache_size = None
    return list(cache.output_forward), list(cache.output_forward_background_mask)


def BlendPointCloudBackward(ctx, info, image_gradients, needs=(True, True, True)):
    """PointRenderer.cu:1549-1644.  Returns [g_texture, g_background, g_points, g_pose_tangent, g_intrinsics]
    (None where the input does not require a gradient)."""
    cache = info.cache
    scene = info.scene
    L = info.num_layers
    dev = scene.texture.device
    saved = ctx.saved_tensors
    assert len(saved) == 3 * L
    image_gradients = [g.contiguous() for g in image_gradients[:L]]  # mask gradients are ignored (:1568-1571)
    for g in image_gradients:
        assert g.dtype == torch.float32

    fb = _capi.ForwardBuffers()
    fb.num_layers = L
    for l in range(L):
        S = fb.layers[l]
        S.w, S.h = int(saved[2 * l].shape[3]), int(saved[2 * l].shape[2])
        S.depth = _ptr(saved[2 * l])
        S.weight = _ptr(saved[2 * l + 1])
        S.out = _ptr(saved[2 * L + l])
        S.depth_index = _ptr(ctx.depth_index[l])
        S.mask = _ptr(ctx.masks[l]) if ctx.masks else None
    fb.dropout_points = _ptr(ctx.dropout_points)
    fb.point_cache = _ptr(getattr(ctx, "point_cache", None))
    fb.pixel_cache = _ptr(getattr(ctx, "pixel_cache", None))

    need_points, need_pose, need_intr = needs
    N = scene.point_cloud_cuda.Size()
    # gradient of a half texture is still accumulated in fp32
    g_texture = torch.empty(scene.texture.shape, dtype=torch.float32, device=dev)
    g_background = torch.empty_like(scene.background_color)
    g_points = torch.empty(N, 4, dtype=torch.float32, device=dev) if need_points else None
    g_points_count = torch.empty(N, dtype=torch.float32, device=dev) if need_points else None
    g_pose = torch.empty_like(scene.tangent_poses) if need_pose else None
    g_pose_count = torch.empty(scene.tangent_poses.shape[0], dtype=torch.float32, device=dev) if need_pose else None
    g_intr = torch.empty_like(scene.intrinsics) if need_intr else None
    g_intr_count = torch.empty(scene.intrinsics.shape[0], dtype=torch.float32, device=dev) if need_intr else None

    gb = _capi.BackwardBuffers()
    for l in range(L):
        gb.grad_out[l] = _ptr(image_gradients[l])
    gb.grad_texture = _ptr(g_texture)
    gb.grad_background = _ptr(g_background)
    gb.grad_points, gb.grad_points_count = _ptr(g_points), _ptr(g_points_count)
    gb.grad_pose, gb.grad_pose_count = _ptr(g_pose), _ptr(g_pose_count)
    gb.grad_intrinsics, gb.grad_intrinsics_count = _ptr(g_intr), _ptr(g_intr_count)

    cache.num_batches = len(info.images)
    cache.info = info
    s = scene.struct()
    stats = C.c_void_p(cache.stats.data_ptr()) if info.collect_stats else None
    info.params.workspace_flags = int(info.workspace_flags)
    rc = cache.lib.adop_backward(C.byref(s), cache.views_array(), cache.num_batches, C.byref(info.params),
                                 C.byref(fb), C.byref(gb), C.c_void_p(cache.workspace.data_ptr()),
                                 cache.workspace.numel(), stats, _stream_ptr())
    _check(rc, cache.lib)
    cache.output_gradient_point_count = g_points_count
    cache.output_gradient_pose_tangent_count = g_pose_count
    cache.output_gradient_intrinsics_count = g_intr_count
    return [g_texture, g_background, g_points, g_pose, g_intr]


class PointRender(torch.autograd.Function):
    """forward(texture, background_color, points, pose_tangents, intrinsics, info) -> L images (+ L masks);
    backward returns five gradients and None for ``info`` (RenderInfo.cpp:34-59)."""

    @staticmethod
    def forward(ctx, texture, background_color, points, pose_tangents, intrinsics, info):
        ctx.render_info = info
        color, mask = BlendPointCloudForward(ctx, info)
        ctx.num_masks = len(mask)
        for m in mask:
            ctx.mark_non_differentiable(m)
        return tuple(color) + tuple(mask)

    @staticmethod
    def backward(ctx, *grad_output):
        info = ctx.render_info
        needs = (ctx.needs_input_grad[2], ctx.needs_input_grad[3], ctx.needs_input_grad[4])
        g_tex, g_bg, g_pts, g_pose, g_intr = BlendPointCloudBackward(ctx, info, list(grad_output), needs)
        if info.scene.texture.dtype != torch.float32:
            g_tex = g_tex.to(info.scene.texture.dtype)
        return g_tex, g_bg, g_pts, g_pose, g_intr, None


def BlendPointCloud(info):
    """Render the scene into a batch of image pyramids (RenderInfo.cpp:19-30)."""
    sc = info.scene
    return list(PointRender.apply(sc.texture, sc.background_color, sc.point_cloud_cuda.t_position, sc.tangent_poses,
                                  sc.intrinsics, info))


def ApplyTangentToPose(tangent, pose):
    """pose = se3_exp(tangent) * pose; tangent = 0 (PointRenderer.cu:1646-1665)."""
    assert tangent.is_contiguous() and pose.is_contiguous()
    assert tangent.dtype == torch.float64 and pose.dtype == torch.float64
    lib = _capi.load_library()
    rc = lib.adop_apply_tangent(C.c_void_p(tangent.data_ptr()), C.c_void_p(pose.data_ptr()), int(tangent.shape[0]),
                                _stream_ptr())
    _check(rc, lib)


def EnvironmentMapSample(info, fb_struct=None, add_to_out=True, want_uv=False, want_env=False):
    """EnvironmentMapImpl::Sample (EnvironmentMap.cu:107-157) fused with ``images += (1-mask)*env``
    (RenderModule.cpp:121-125).  Operates on the cache's current forward outputs.  ``add_to_out``: False / 0 = sample
    only, True / 1 = add in place, 2 = the second return value holds the composed images and the rasterizer's outputs
    stay untouched (what the backward pass should see, as in the reference)."""
    want_env = want_env or add_to_out == 2
    cache = info.cache
    scene = info.scene
    env = scene.environment_map
    assert env is not None and env.dim() == 3
    dev = env.device
    B, Cn = cache.num_batches, int(scene.texture.shape[0])
    fb = fb_struct or cache.forward_struct()
    L = info.num_layers
    uv = [torch.empty(B, l.size[1], l.size[0], 2, dtype=torch.float32, device=dev) for l in cache.layers_cuda] if want_uv else None
    ev = [torch.empty(B, Cn, l.size[1], l.size[0], dtype=torch.float32, device=dev) for l in cache.layers_cuda] if want_env else None
    uv_arr = (C.c_void_p * L)(*[t.data_ptr() for t in uv]) if uv else None
    ev_arr = (C.c_void_p * L)(*[t.data_ptr() for t in ev]) if ev else None
    s = scene.struct()
    rc = cache.lib.adop_env_sample(C.byref(s), cache.views_array(), B, C.c_void_p(env.data_ptr()), int(env.shape[1]),
                                   int(env.shape[2]), C.byref(fb), uv_arr, ev_arr, int(add_to_out),
                                   _stream_ptr())
    _check(rc, cache.lib)
    return uv, ev


def EnvironmentMapSampleBackward(info, grad_out, fb_struct=None, uv=None):
    """Gradient of the fused sample-and-add w.r.t. the environment texture.  ``uv``: the per-level texture coordinates
    ``EnvironmentMapSample(..., want_uv=True)`` returned for the same views (the kernel then reads them instead of
    computing every pixel's ray again)."""
    cache = info.cache
    scene = info.scene
    env = scene.environment_map
    L = info.num_layers
    fb = fb_struct or cache.forward_struct()
    grad_out = [g.contiguous() for g in grad_out[:L]]
    g_arr = (C.c_void_p * L)(*[g.data_ptr() for g in grad_out])
    g_env = torch.empty_like(env)
    s = scene.struct()
    uv_arr = None if uv is None else (C.c_void_p * L)(*[t.data_ptr() for t in uv[:L]])
    rc = cache.lib.adop_env_sample_backward(C.byref(s), cache.views_array(), cache.num_batches, int(env.shape[1]),
                                            int(env.shape[2]), C.byref(fb), g_arr, uv_arr, C.c_void_p(g_env.data_ptr()),
                                            _stream_ptr())
    _check(rc, cache.lib)
    return g_env
