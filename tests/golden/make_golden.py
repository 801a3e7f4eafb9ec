"""Writes tests/golden/*.npz with the CPU checker (run from the repository root: python tests/golden/make_golden.py).

The reference ships no test vectors for this path (it has no tests), so these fixtures are produced by this
repository's own checker after it has been pinned by tests/test_oracle_math.py and tests/test_oracle_render.py.
They freeze its behaviour: a later change of the checker or of the HIP path that alters a result shows up here.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from adop_amd import scenes  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def golden_scenes():
    """name -> HostScene; small enough to commit (a few hundred KB)."""
    a = scenes.config1(n=2000, w=32, h=32, levels=3, seed=0)
    b = scenes.config3(n=3000, w=48, h=27, levels=3, channels=4, seed=1)
    b.intrinsics[0, 5:] = [0.05, -0.02, 0.003, 0.01, 0.002, -0.001, 0.001, -0.0015]
    b.params.dist_cutoff = 1.5
    c = scenes.config5(n=3000, w=44, h=30, levels=3, batch=2, patches=40, seed=2)
    c.params.ghost_gradients = 0
    return {"config1_2k_32x32": a, "config3_3k_48x27_distortion": b, "config5_ocam_3k_44x30": c}


def run(hs):
    fwd = oracle.forward(hs)
    gout = scenes.upstream_grads(hs, 77)
    bwd = oracle.backward(hs, fwd, gout)
    out = {}
    for l in range(hs.num_layers):
        out[f"depth_index_{l}"] = fwd.depth_index[l]
        out[f"weight_{l}"] = fwd.weight[l]
        out[f"out_{l}"] = fwd.out[l]
    for name in ("grad_texture", "grad_background", "grad_points", "grad_points_count", "grad_pose", "grad_pose_count",
                 "grad_intrinsics", "grad_intrinsics_count"):
        out[name] = getattr(bwd, name)
    return out


if __name__ == "__main__":
    for name, hs in golden_scenes().items():
        res = run(hs)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **res)
        print(name, {k: v.shape for k, v in list(res.items())[:3]})
