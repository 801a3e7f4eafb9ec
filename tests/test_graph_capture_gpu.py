"""The forward and backward calls recorded into a HIP graph (stream capture through torch.cuda.graph): the library
launches kernels only (no allocation, no memset node, no synchronisation), so a replay must give what an eager call
gives for the inputs then in place.  Replayed several times with changed inputs and eager work in between."""
import numpy as np
import pytest

from helpers import announce

pytestmark = pytest.mark.gpu


class Ctx:
    def save_for_backward(self, *t):
        self.saved_tensors = t


@pytest.mark.parametrize("forward_path", [1, 2], ids=["direct", "tiles"])
def test_forward_backward_replayed_from_a_graph(forward_path):
    import torch
    from adop_amd import render, scenes

    hs = scenes.config3(n=300_000, w=480, h=270)
    hs.params.forward_path = forward_path
    announce(f"graph capture: config3 N=300000 480x270, forward_path={forward_path}")
    scene = render.NeuralScene.from_host(hs, "cuda")
    drop = torch.from_numpy(hs.dropout).cuda()
    info = render.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params, num_layers=hs.num_layers,
                                   cache=render.PointRendererCache(), collect_stats=False, train=True,
                                   dropout_points=drop)
    gen = torch.Generator(device="cuda").manual_seed(3)
    tex0 = scene.texture.clone()

    def eager():
        ctx = Ctx()
        images, _ = render.BlendPointCloudForward(ctx, info)
        gout = [torch.ones_like(im) * (l + 1) for l, im in enumerate(images)]
        grads = render.BlendPointCloudBackward(ctx, info, gout)
        packed = [L.depth_index_tensor.clone() for L in info.cache.layers_cuda]
        return [im.clone() for im in images], [g.clone() for g in grads], packed

    eager()  # first call: lazy initialisation outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ctx = Ctx()
            g_images, _ = render.BlendPointCloudForward(ctx, info)
            g_gout = [torch.ones_like(im) * (l + 1) for l, im in enumerate(g_images)]
            g_grads = render.BlendPointCloudBackward(ctx, info, g_gout)
            g_layers = list(info.cache.layers_cuda)  # the buffers the recorded kernels write (a later forward takes new ones)
    torch.cuda.synchronize()
    for rep in range(4):
        # new inputs in place: descriptors, and the camera pose (the view constants are computed on the device)
        scene.texture.copy_(tex0 * (1.0 + 0.25 * rep) + 0.125 * rep)
        scene.poses_se3[0, 4:7] += 0.01 * rep
        want_images, want_grads, want_packed = eager()
        for L in g_layers:  # scribble over what the replay must rewrite
            L.depth_index_tensor.fill_(7)
            L.weight.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for l, L in enumerate(g_layers):
            assert bool((L.depth_index_tensor == want_packed[l]).all()), (rep, l)
            a, b = g_images[l], want_images[l]
            assert float((a - b).abs().max()) <= 1e-5 * float(b.abs().max()), (rep, l)
        for name, a, b in zip(["texture", "background", "points", "pose", "intrinsics"], g_grads, want_grads):
            assert float((a.double() - b.double()).abs().max()) <= 1e-4 * float(b.double().abs().max()) + 1e-12, (rep, name)
