"""Training through the anchor decode (Scaffold-GS / Octree-GS): with gradients enabled the decoder evaluates the
reference module's statements as torch operations (as the reference trains: its fused decoder is an inference
component), the rasterizer behind it differentiates in HIP.  Checked: the differentiable path gives the kernels'
Gaussians; its gradients equal those of the oracle's statements evaluated in float64; a short optimisation of a
perturbed Scaffold-GS model against its own rendering reduces the loss."""
import numpy as np
import pytest
import torch

from landmarksystem_amd import scenes
from landmarksystem_amd.models import ScaffoldGS
from oracle import anchor_oracle as ao
from tests.test_gpu_decode import TOL, build_decoder

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("add_dist", [(True, True, True), (True, False, True)])
def test_differentiable_decode_matches_kernels_and_float64_gradients(gpu_device, add_dist):
    A = 3000
    sc = scenes.config5(A=A)
    if not add_dist[1]:
        w0, b0, w1, b1 = sc.mlp["cov"]
        sc.mlp = dict(sc.mlp, cov=(w0[:, :35].contiguous(), b0, w1, b1))
    g = torch.Generator().manual_seed(3)
    vis = torch.rand(A, generator=g) < 0.7
    dec = build_decoder(sc, gpu_device, add_dist=add_dist).train()
    dev = lambda t: t.to(gpu_device)  # noqa: E731
    inputs = dict(anchor=dev(sc.anchor), anchor_feat=dev(sc.anchor_feat), offset=dev(sc.offset), scaling=dev(sc.scaling))
    cam = dev(sc.camera.camera_center)
    with torch.no_grad():
        kernels = dec(cam, visible_mask=dev(vis), **inputs)
    for p in dec.parameters():
        p.requires_grad_(True)
    leaves = {k: v.clone().requires_grad_(True) for k, v in inputs.items() if k != "anchor"}
    got = dec(cam, anchor=inputs["anchor"], visible_mask=dev(vis), **leaves)
    assert got[0].requires_grad and got[5].shape == (int(vis.sum()) * sc.n_offsets, 1)
    # same Gaussians as the kernels (away from the mask threshold the two paths keep the same offsets)
    raw = got[5].detach().view(-1)
    if float(raw.abs().min()) > 1e-5:
        for a, b in zip(got[:5], kernels[:5]):
            assert a.shape == b.shape
            assert float((a.detach() - b).abs().max()) <= TOL * max(1.0, float(b.abs().max()))
        assert torch.equal(got[6], kernels[6])
    # gradients of a weighted sum of every output against float64 autograd through the oracle's statements
    weights = [torch.randn(t.shape, generator=g) for t in got[:5]]
    loss = sum((t * dev(w)).sum() for t, w in zip(got[:5], weights))
    loss.backward()
    ref_mlp = {h: tuple(t.double().requires_grad_(True) for t in sc.mlp[h]) for h in ao.HEADS}
    ref_in = {k: v.double().requires_grad_(True) for k, v in (("anchor_feat", sc.anchor_feat), ("offset", sc.offset),
                                                               ("scaling", sc.scaling))}
    ref = ao.decode(sc.camera.camera_center, sc.anchor, ref_in["anchor_feat"], ref_in["offset"], ref_in["scaling"], vis,
                    ref_mlp, sc.n_offsets, add_dist=add_dist, keep_override=got[6].cpu(), dtype=torch.float64)
    ref_loss = sum((ref[k] * w.double()).sum() for k, w in zip(("xyz", "color", "opacity", "scaling", "rot"), weights))
    ref_loss.backward()
    assert abs(float(loss.detach()) - float(ref_loss.detach())) <= 1e-4 * abs(float(ref_loss.detach())) + 1e-3

    def close(name, a, b):
        scale = float(b.abs().max())
        assert scale > 0, name
        assert float((a.cpu().double() - b).abs().max()) <= 2e-4 * scale, name

    for name in leaves:
        close(name, leaves[name].grad, ref_in[name].grad)
    for head, module in (("opacity", dec.mlp_opacity), ("cov", dec.mlp_cov), ("color", dec.mlp_color)):
        for k, prm in enumerate((module[0].weight, module[0].bias, module[2].weight, module[2].bias)):
            close("%s[%d]" % (head, k), prm.grad, ref_mlp[head][k].grad)


def test_scaffold_training_reduces_the_loss(gpu_device):
    """scaffold_gs/gs_trainer.py's step in miniature: forward in training mode returns (image, scaling), the loss
    back-propagates through the HIP rasterizer and the decode into anchors' parameters and MLPs, Adam steps."""
    scene = scenes.config5(A=4000, width=160, height=96)
    target_model = ScaffoldGS.from_scene(scene).to(gpu_device).eval()
    with torch.no_grad():
        target = target_model(scene.camera).clone()
    assert float(target.max()) > 0.05
    g = torch.Generator().manual_seed(9)
    model = ScaffoldGS.from_scene(scene).to(gpu_device)
    with torch.no_grad():
        model._anchor_feat.add_(0.2 * torch.randn(model._anchor_feat.shape, generator=g).to(gpu_device))
        model._offset.add_(0.05 * torch.randn(model._offset.shape, generator=g).to(gpu_device))
        for p in model.anchor_decoder.parameters():
            p.add_(0.02 * torch.randn(p.shape, generator=g).to(gpu_device))
    model.train()
    train = [model._anchor_feat, model._offset, model._scaling] + list(model.anchor_decoder.parameters())
    for p in train:
        p.requires_grad_(True)
    opt = torch.optim.Adam(train, lr=2e-3)
    losses = []
    for _ in range(40):
        image, scaling = model(scene.camera, retain_grad=True)
        assert image.requires_grad and scaling.shape[1] == 3
        loss = (image - target).abs().mean()
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(np.isfinite(losses)) and losses[-1] < 0.6 * losses[0], (losses[0], losses[-1])
    assert model.viewspace_points.grad is not None and model.viewspace_points.grad.shape == model.viewspace_points.shape
    assert model.offset_selection_mask.dtype == torch.bool and model.opacity.shape[1] == 1
    assert model.visibility_filter.shape[0] == int(model.offset_selection_mask.sum())
    for p in train:
        assert p.grad is not None and torch.isfinite(p.grad).all()
    # training mode without gradients: the same pair, from the kernels
    with torch.no_grad():
        image2, scaling2 = model(scene.camera)
    assert not image2.requires_grad and scaling2.shape[1] == 3 and model.opacity.shape[1] == 1
    with torch.no_grad():
        image3, _ = model(scene.camera)
    assert torch.equal(image2, image3)
    # eval mode afterwards is the kernels' frame again (no graph)
    model.eval()
    frame = model(scene.camera)
    assert not frame.requires_grad and frame.shape == target.shape
    assert float((frame - image2).abs().max()) <= 2e-3  # (same parameters; offsets at the opacity threshold may differ)


def test_octree_training_step_with_level_input_and_feature_bank(gpu_device):
    """Octree-GS in training mode (octree_gs/gs_trainer.py sets the level-of-detail mask itself before the forward
    call): the differentiable decode with the level input and the feature bank gives the kernels' frame, and one
    backward pass leaves finite gradients on every parameter, the feature bank's included."""
    from landmarksystem_amd.models import OctreeGS
    scene = scenes.config5(A=6000, width=160, height=96)
    level = torch.randint(0, 4, (6000,), generator=torch.Generator().manual_seed(2))
    model = OctreeGS(scene.anchor, scene.anchor_feat, scene.offset, torch.log(scene.scaling), scene.rotation, level,
                     voxel_size=0.5, standard_dist=250.0, fork=2, n_offsets=scene.n_offsets, use_feat_bank=True,
                     add_level=True, add_opacity_dist=False, add_cov_dist=False, add_color_dist=False).to(gpu_device)
    cam = scene.camera
    model.eval()
    frame = model(cam)
    mask = model._anchor_mask.clone()
    assert 0 < int(mask.sum()) < 6000
    model.train()
    model.set_anchor_mask(cam.camera_center, 0, cam.resolution_scale)
    assert torch.equal(model._anchor_mask, mask)
    train = [model._anchor_feat, model._offset, model._scaling] + list(model.anchor_decoder.parameters())
    for p in train:
        p.requires_grad_(True)
    image, scaling = model(cam, retain_grad=True)
    assert image.requires_grad
    assert not bool((model.voxel_visible_mask & ~mask).any())
    diff = (image.detach() - frame).abs()
    assert float(diff.max()) <= 2e-3 and float(diff.mean()) <= 1e-5  # same frame up to offsets at the opacity threshold
    (image.square().mean() + 1e-3 * scaling.prod(dim=1).mean()).backward()
    for p in train:
        assert p.grad is not None and torch.isfinite(p.grad).all()
    assert float(model.anchor_decoder.mlp_feature_bank[0].weight.grad.abs().max()) > 0
    assert float(model._anchor_feat.grad.abs().max()) > 0 and float(model._offset.grad.abs().max()) > 0
