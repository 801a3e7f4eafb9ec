"""The render stage inside an optimisation loop, as the reference's training uses it (PointRender autograd function,
optimiser step on the descriptors / on the pose tangent, ApplyTangent): the image loss falls, and a perturbed camera
pose moves back towards the pose the target images were rendered from."""
import numpy as np
import pytest

from helpers import announce

pytestmark = pytest.mark.gpu


def smooth_scene(seed=0):
    from adop_amd import scenes

    hs = scenes.config3(n=400_000, w=320, h=180, channels=4, levels=3, seed=seed)
    xyz = hs.position[:, :3].astype(np.float64)
    k = np.array([[1.3, 0.4, -0.7], [-0.5, 1.1, 0.9], [0.8, -1.2, 0.3], [0.2, 0.7, 1.4]])
    hs.texture = (0.5 + 0.5 * np.sin(2.0 * xyz @ k.T)).T.astype(np.float32).copy()  # smooth in space
    hs.dropout = None
    hs.params.ghost_gradients = 0  # every rendered point receives a spatial gradient (:487-488)
    hs.params.normalize_mode = 1
    return hs


def render(scene, info):
    from adop_amd import render as R

    return R.BlendPointCloud(info)[: info.num_layers]


def make(hs):
    import torch
    from adop_amd import render as R

    scene = R.NeuralScene.from_host(hs, "cuda")
    info = R.NeuralRenderInfo(scene=scene, images=list(hs.views), params=hs.params, num_layers=hs.num_layers,
                              cache=R.PointRendererCache(), train=True)
    return scene, info


def loss_of(images, target):
    return sum(((a - b) ** 2).mean() for a, b in zip(images, target))


def test_descriptors_converge_to_the_target_images():
    import torch

    hs = smooth_scene()
    announce("optimise descriptors: N=400000 320x180 L=3 C=4")
    scene, info = make(hs)
    with torch.no_grad():
        target = [t.clone() for t in render(scene, info)]
    scene.texture = torch.full_like(scene.texture, 0.5).requires_grad_(True)
    opt = torch.optim.Adam([scene.texture], lr=0.05)
    losses = []
    for it in range(40):
        opt.zero_grad()
        loss = loss_of(render(scene, info), target)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < 0.05 * losses[0], losses[::8]


def test_perturbed_pose_moves_back():
    import torch
    from adop_amd import render as R

    hs = smooth_scene(1)
    announce("optimise the pose tangent: N=400000 320x180 L=3 C=4")
    scene, info = make(hs)
    with torch.no_grad():
        target = [t.clone() for t in render(scene, info)]
    true_pose = scene.poses_se3.clone()
    # left perturbation of the view transform: 2 cm sideways and up, 0.2 degrees about y
    delta = torch.tensor([[0.02, -0.015, 0.0, 0.0, 0.0035, 0.0]], dtype=torch.float64, device="cuda")
    R.ApplyTangentToPose(delta.clone(), scene.poses_se3)
    scene.tangent_poses.requires_grad_(True)

    def pose_error():
        return float((scene.poses_se3[0, :7] - true_pose[0, :7]).norm())

    e0 = pose_error()
    with torch.no_grad():
        l0 = float(loss_of(render(scene, info), target))
    opt = torch.optim.Adam([scene.tangent_poses], lr=1e-3)
    for it in range(80):
        opt.zero_grad()
        loss = loss_of(render(scene, info), target)
        loss.backward()
        opt.step()
        with torch.no_grad():
            R.ApplyTangentToPose(scene.tangent_poses, scene.poses_se3)  # folds the step into the pose, tangent = 0
    with torch.no_grad():
        l1 = float(loss_of(render(scene, info), target))
    e1 = pose_error()
    print("pose error", e0, "->", e1, "loss", l0, "->", l1)
    assert e1 < 0.5 * e0 and l1 < 0.5 * l0, (e0, e1, l0, l1)
