"""Point-cloud preprocessing of SceneData (data/SceneData.cpp:96-118) on the device: the filters for lonely and
close points, Morton order, shuffled 256-point blocks, the radius of every point from its 4th nearest neighbour,
blocks sorted by radius.

The order of the cloud and the radii decide how the rasterizer runs (coherent wavefronts, the LOD early exit), so the
steps sit next to it.  The distance search and the Morton codes are HIP kernels behind the C-ABI
(``adop_knn_distance``, ``adop_morton_codes``, ``adop_point_distance_to_camera``, ``adop_close_points``); sorting and permuting go through torch.
"""
import ctypes as C

import torch

from . import _capi
from .render import _check, _stream_ptr


def _bbox(position):
    lo, hi = torch.aminmax(position, dim=0)  # one pass over the contiguous [N,4] array
    both = torch.stack([lo[:3], hi[:3]]).cpu()
    return (C.c_float * 3)(*both[0].tolist()), (C.c_float * 3)(*both[1].tolist())


def KNearestNeighbourDistance(position, rank=4):
    """Distance of every point to its ``rank``-th nearest other point: ``data[i](0)`` of ComputeRadius
    (SceneData.cpp:441-463).  position: [N,4] f32 on the device."""
    assert position.is_cuda and position.dtype == torch.float32 and position.dim() == 2 and position.shape[1] == 4
    position = position.contiguous()
    n = int(position.shape[0])
    lib = _capi.load_library()
    out = torch.empty(n, dtype=torch.float32, device=position.device)
    ws = torch.empty(int(lib.adop_knn_workspace_size(n)), dtype=torch.uint8, device=position.device)
    mn, mx = _bbox(position)
    rc = lib.adop_knn_distance(C.c_void_p(position.data_ptr()), n, int(rank), mn, mx, C.c_void_p(out.data_ptr()),
                               C.c_void_p(ws.data_ptr()), int(ws.numel()), _stream_ptr())
    _check(rc, lib)
    return out


def MortonCodes(position):
    """63-bit Morton code of every point inside the cloud's bounding box (the key of ReorderMorton64)."""
    assert position.is_cuda and position.dtype == torch.float32 and position.dim() == 2 and position.shape[1] == 4
    position = position.contiguous()
    n = int(position.shape[0])
    lib = _capi.load_library()
    codes = torch.empty(n, dtype=torch.int64, device=position.device)
    mn, mx = _bbox(position)
    rc = lib.adop_morton_codes(C.c_void_p(position.data_ptr()), n, mn, mx, C.c_void_p(codes.data_ptr()), _stream_ptr())
    _check(rc, lib)
    return codes


def PointDistanceToCamera(position, poses_se3, intrinsics, frames):
    """SceneData::PointDistanceToCamera (SceneData.cpp:645-669): distance of every point to the nearest camera that
    sees it.  position [N,4] f32, poses_se3 [F,8] f64 (view transforms), intrinsics [K,13] f32 on the device;
    ``frames``: one adop view per frame (w, h, image_index, camera_index)."""
    assert position.is_cuda and position.dtype == torch.float32 and position.dim() == 2 and position.shape[1] == 4
    assert poses_se3.is_cuda and poses_se3.dtype == torch.float64 and poses_se3.shape[1] == 8
    assert intrinsics.is_cuda and intrinsics.dtype == torch.float32 and intrinsics.shape[1] == 13
    position, poses_se3, intrinsics = position.contiguous(), poses_se3.contiguous(), intrinsics.contiguous()
    lib = _capi.load_library()
    s = _capi.Scene()
    s.position, s.num_points = position.data_ptr(), int(position.shape[0])
    s.poses_se3, s.num_poses = poses_se3.data_ptr(), int(poses_se3.shape[0])
    s.intrinsics, s.num_cameras, s.intrinsics_cols = intrinsics.data_ptr(), int(intrinsics.shape[0]), 13
    views = (_capi.View * len(frames))(*frames)
    out = torch.empty(s.num_points, dtype=torch.float32, device=position.device)
    ws = torch.empty(int(lib.adop_frames_workspace_size(len(frames))), dtype=torch.uint8, device=position.device)
    rc = lib.adop_point_distance_to_camera(C.byref(s), views, len(frames), C.c_void_p(out.data_ptr()),
                                           C.c_void_p(ws.data_ptr()), int(ws.numel()), _stream_ptr())
    _check(rc, lib)
    return out


def RemoveLonelyPoints(position, camera_distance, n=5, dis_th=0.02):
    """Keep mask of SceneData::RemoveLonelyPoints (SceneData.cpp:550-595): a point goes when the distance to its
    n-th nearest neighbour, relative to its camera distance, exceeds ``dis_th``."""
    d = KNearestNeighbourDistance(position, n)
    return ~(d / camera_distance > dis_th)


def RemoveClosePoints(position, camera_distance, dis_th=0.00005, rounds_per_call=8):
    """Keep mask of SceneData::RemoveClosePoints (SceneData.cpp:598-642): in index order, a point goes when a point
    kept before it lies within dis_th / camera_distance of it."""
    assert position.is_cuda and position.dtype == torch.float32 and position.dim() == 2 and position.shape[1] == 4
    position = position.contiguous()
    n = int(position.shape[0])
    radius = (dis_th / camera_distance).to(torch.float32).contiguous()
    lib = _capi.load_library()
    state = torch.empty(n, dtype=torch.int32, device=position.device)
    undecided = torch.empty(rounds_per_call, dtype=torch.int32, device=position.device)
    ws = torch.empty(int(lib.adop_knn_workspace_size(n)), dtype=torch.uint8, device=position.device)
    mn, mx = _bbox(position)
    resume = 0
    while True:
        rc = lib.adop_close_points(C.c_void_p(position.data_ptr()), n, C.c_void_p(radius.data_ptr()), mn, mx,
                                   C.c_void_p(state.data_ptr()), C.c_void_p(undecided.data_ptr()), rounds_per_call,
                                   resume, C.c_void_p(ws.data_ptr()), int(ws.numel()), _stream_ptr())
        _check(rc, lib)
        if int(undecided[-1].item()) == 0:
            return state == 1
        resume = 1


def FilterPointCloud(position, poses_se3, intrinsics, frames, lonely=(5, 0.02), close=0.00005):
    """The two filters of a new scene in the reference's order (SceneData.cpp:98-99): RemoveLonelyPoints(5, 0.02), then
    RemoveClosePoints(0.00005) on what is left.  Returns the ids of the surviving points, ascending."""
    ids = torch.arange(int(position.shape[0]), device=position.device)
    cam = PointDistanceToCamera(position, poses_se3, intrinsics, frames)  # per point: erasing others does not change it
    keep = RemoveLonelyPoints(position, cam, *lonely)
    position, cam, ids = position[keep].contiguous(), cam[keep], ids[keep]
    keep = RemoveClosePoints(position, cam, close)
    return ids[keep]


def ReorderMorton64(position):
    """Permutation that sorts the cloud along the Morton curve (stable: equal codes keep their order)."""
    return torch.sort(MortonCodes(position), stable=True).indices


def RandomBlockShuffle(num_points, block_size=256, generator=None):
    """Permutation that shuffles whole blocks of ``block_size`` consecutive points (a last, shorter block stays
    last)."""
    nb = num_points // block_size
    dev = "cuda"
    perm = torch.randperm(nb, generator=generator, device="cpu").to(dev)
    idx = (perm[:, None] * block_size + torch.arange(block_size, device=dev)[None, :]).reshape(-1)
    tail = torch.arange(nb * block_size, num_points, device=dev)
    return torch.cat([idx, tail])


def ComputeRadius(position, rank=4, generator=None):
    """SceneData::ComputeRadius (SceneData.cpp:441-484): returns ``data`` [N,4] with data[:,0] = distance to the
    rank-th neighbour, data[:,2] = sqrt(1 / u), u ~ U(0,1), data[:,3] = data[:,0] * data[:,2] (the drop-out radius the
    rasterizer reads as position.w, NeuralPointCloudCuda.cpp:21-35)."""
    n = int(position.shape[0])
    data = torch.zeros(n, 4, dtype=torch.float32, device=position.device)
    data[:, 0] = KNearestNeighbourDistance(position, rank)
    if generator is not None and generator.device.type == "cpu":  # a host generator: draw there
        u = torch.rand(n, generator=generator, dtype=torch.float64, device="cpu").to(position.device)
    else:
        u = torch.rand(n, generator=generator, dtype=torch.float64, device=position.device)
    data[:, 2] = torch.sqrt(1.0 / u.clamp_min_(1e-300)).to(torch.float32)
    data[:, 3] = data[:, 0] * data[:, 2]
    return data


def SortBlocksByRadius(radius, block_size=256):
    """Permutation that sorts every full block of ``block_size`` points by ascending radius
    (SceneData.cpp:671-684; the last, shorter block keeps its order)."""
    n = int(radius.shape[0])
    nb = n // block_size
    head = radius[: nb * block_size].reshape(nb, block_size)
    order = torch.sort(head, dim=1, stable=True).indices + (torch.arange(nb, device=radius.device) * block_size)[:, None]
    return torch.cat([order.reshape(-1), torch.arange(nb * block_size, n, device=radius.device)])


def PreprocessPointCloud(position, normal=None, rank=4, block_size=256, seed=0):
    """The initial processing of a new scene in the reference's order (SceneData.cpp:101-104): ReorderMorton64,
    RandomBlockShuffle(256), ComputeRadius, SortBlocksByRadius(256).  Returns (position [N,4] with the drop-out radius in
    w, normal, data [N,4], order) where ``order`` maps new to original point ids."""
    gen = torch.Generator(device="cpu").manual_seed(int(seed))
    gen_dev = torch.Generator(device=position.device).manual_seed(int(seed))  # the per-point numbers are drawn on the device
    position = position.contiguous()
    order = ReorderMorton64(position)
    order = order[RandomBlockShuffle(int(position.shape[0]), block_size, gen)]
    position = position[order].contiguous()
    data = ComputeRadius(position, rank, gen_dev)
    by_radius = SortBlocksByRadius(data[:, 3], block_size)
    order = order[by_radius]
    position = position[by_radius].clone()
    data = data[by_radius].contiguous()
    position[:, 3] = data[:, 3]
    return position, (None if normal is None else normal[order].contiguous()), data, order


def AttachDropOutRadii(hs, rank=4, block_size=256, seed=0):
    """Gives a host scene (``scenes.HostScene`` in the reference's point order) what the rasterizer's LOD test reads,
    as a new scene gets it (SceneData.cpp:103-104): ``position.w`` = ComputeRadius' drop-out radius, every 256-point
    block sorted by it; switches ``drop_out_points_by_radius`` on (the reference's default, Settings.h:36-37).  The
    descriptors and the dropout mask of the synthetic scenes are independent random numbers per point and stay."""
    pos = torch.from_numpy(hs.position).cuda()
    gen = torch.Generator(device=pos.device).manual_seed(int(seed))
    data = ComputeRadius(pos, rank, gen)
    order = SortBlocksByRadius(data[:, 3], block_size)
    pos = pos[order].contiguous()
    pos[:, 3] = data[order, 3]
    hs.position = pos.cpu().numpy()
    if hs.normal is not None:
        hs.normal = torch.from_numpy(hs.normal).cuda()[order].cpu().numpy()
    hs.params.drop_out_points_by_radius = 1
    hs.meta["lod_radius_test"] = True
    return hs
