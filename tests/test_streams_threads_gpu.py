"""The calls of the C-ABI keep no state between them but what the caller hands in (scene, buffers, workspace), queue
their work on the stream they are given and never wait for the device (the reference's render stage works on the
legacy default stream through `__constant__` parameter blocks and is not re-entrant, PointRenderer.cu:139-141,
1096-1143).  Two host threads, each with a scene, a workspace and a stream of its own, run forward + backward side by
side without waiting in between; every thread's last results must be the checker's."""
import threading

import numpy as np
import pytest

from helpers import announce, check_backward, check_forward, download_forward

pytestmark = pytest.mark.gpu


def _worker(hs, forward_path, rounds, out, key, start):
    import torch
    from adop_amd import render, scenes

    try:
        hs.params.forward_path = forward_path
        stream = torch.cuda.Stream()  # default priority
        with torch.cuda.stream(stream):
            scene = render.NeuralScene.from_host(hs, "cuda")
            info = render.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params,
                                           num_layers=hs.num_layers, cache=render.PointRendererCache(),
                                           collect_stats=False, train=True,
                                           dropout_points=None if hs.dropout is None else torch.from_numpy(hs.dropout))
            gout_host = scenes.upstream_grads(hs, 5)
            gout = [torch.from_numpy(g).cuda() for g in gout_host]
            stream.synchronize()
            start.wait()  # both threads queue their work at the same time

            class Ctx:
                def save_for_backward(self, *t):
                    self.saved_tensors = t

            for _ in range(rounds):
                ctx = Ctx()
                images, masks = render.BlendPointCloudForward(ctx, info)
                grads = render.BlendPointCloudBackward(ctx, info, gout, (True, True, True))
            stream.synchronize()
            out[key] = (info, ctx, images, masks, grads, gout_host)
    except BaseException as e:  # noqa: BLE001 - handed to the test's thread
        out[key] = e
        start.abort()


@pytest.mark.parametrize("forward_path", [1, 2], ids=["direct", "tiles"])
def test_two_host_threads_on_streams_of_their_own(oracle_mod, forward_path):
    from adop_amd import scenes

    announce(f"two host threads, two streams, two workspaces, forward_path={forward_path}: 20 forward + backward each")
    cases = {"a": scenes.config3(n=400_000, w=480, h=270),
             "b": scenes.config2(n=150_000, w=200, h=160, levels=3, batch=3, seed=4)}
    out = {}
    start = threading.Barrier(2)
    threads = [threading.Thread(target=_worker, args=(hs, forward_path, 20, out, key, start))
               for key, hs in cases.items()]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
        assert not t.is_alive()
    for key, hs in cases.items():
        assert not isinstance(out[key], BaseException), out[key]
        info, ctx, images, masks, grads, gout_host = out[key]
        ref = oracle_mod.forward(hs)
        check_forward(hs, ref, ctx, images, masks, info, stats=False)
        refb = oracle_mod.backward(hs, download_forward(hs, info, images, masks), gout_host, True, True, True)
        check_backward(hs, refb, grads, info, stats=False)
        assert np.isfinite(grads[0].cpu().numpy()).all()
