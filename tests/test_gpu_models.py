"""GPU tests of the model-side callers (landmarksystem_amd/models.py): the
vanilla / Scaffold / Octree forward sequences of the reference, end to end,
with the rasterizer checked against the oracle on the Gaussians it was given."""
import math

import numpy as np
import pytest
import torch

from landmarksystem_amd import scenes
from landmarksystem_amd.models import GaussianModel, OctreeGS, ScaffoldGS
from oracle import anchor_oracle as ao
from oracle import c_oracle as co
from tests.helpers import (check_anchor_model_frame, check_images, oracle_frame, oracle_gaussians, psnr,
                           vanilla_model_reference)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fuse", [False, True], ids=["reference-sequence", "fused-prefilter"])
def test_vanilla_model_forward(gpu_device, fuse):
    """Both forward sequences of the vanilla model: the reference's (prefilter, gather of the visible rows, render:
    fuse_prefilter=False) and the single pass that is the default."""
    scene = scenes.config2(P=50_000, width=640, height=360)
    model = GaussianModel.from_activated(scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs,
                                         sh_degree=3, act_cache=True, fuse_prefilter=fuse).to(gpu_device).eval()
    assert GaussianModel(dict(sh_degree=3)).fuse_prefilter is True  # the default
    image = model(scene.camera)
    # activations round-trip (log/exp, logit/sigmoid) perturb the inputs by an ulp: feed the oracle the
    # model's own activated tensors
    act = scenes.GaussianScene("act", model.get_xyz.cpu(), model.get_scaling.cpu(), model.get_rotation.cpu(),
                               model.get_opacity.cpu(), model.get_features.cpu(), 3, scene.cameras, scene.bg)
    ref = co.render(oracle_frame(act), oracle_gaussians(act))
    check_images(dict(image=image.cpu().numpy()), ref, "vanilla model forward" + (", fused" if fuse else ""))
    vis = ref["radii"] > 0
    assert torch.equal(model.visibility_filter.cpu(), torch.from_numpy(vis))
    assert model.radii.shape[0] == int(vis.sum())  # eval mode renders the prefiltered subset
    np.testing.assert_array_equal(model.radii.cpu().numpy(), ref["radii"][vis])
    assert "scaling" in model._cache  # act_cache: activations computed once
    again = model(scene.camera)
    assert torch.equal(image, again)


@pytest.mark.parametrize("A,width,height,fuse", [(30_000, 640, 360, False), (30_000, 640, 360, True),
                                                 (500_000, 1920, 1080, False), (500_000, 1920, 1080, True)])
def test_scaffold_model_forward(gpu_device, A, width, height, fuse):
    """Scaffold-GS forward, scaled down and at the full size of the 500k-anchor workload, through the reference's
    sequence of calls (fuse_prefilter=False) and through the default one-kernel prefilter."""
    scene = scenes.config5(A=A, width=width, height=height)
    model = ScaffoldGS.from_scene(scene, fuse_prefilter=fuse).to(gpu_device).eval()
    assert ScaffoldGS.from_scene(scenes.config5(A=10)).fuse_prefilter is True  # the default
    cam = scene.camera
    image = model(cam)
    assert image.shape == (3, height, width)
    # anchor-level visibility equals the oracle's visible filter on the anchors
    vis_ref = co.visible_filter(oracle_frame(scenes.GaussianScene("a", scene.anchor, scene.scaling[:, :3],
                                scene.rotation, torch.zeros(1), torch.zeros(1, 1, 3), 1, [cam], scene.bg),
                                sh_degree=1), scene.anchor.numpy(), scales=model.get_scaling[:, :3].cpu().numpy(),
                                rotations=model.get_rotation.cpu().numpy()) > 0
    assert torch.equal(model.voxel_visible_mask.cpu(), torch.from_numpy(vis_ref))
    dec = check_anchor_model_frame(model, cam, image, "Scaffold-GS %d anchors%s" % (A, ", fused" if fuse else ""))
    assert dec["xyz"].shape[0] > A // 10


def test_compute_cov3D_python_path(gpu_device):
    """compute_cov3D_python=True (origin_gs/gs_model.py:173-174): the model hands the rasterizer covariances it
    computed with torch statements instead of scales and rotations.  Against the oracle fed the same covariances:
    radii bit for bit, image to the frame bars; against the default path: the same frame up to the fp32 rounding of
    two ways of forming R diag(s^2) R^T; in training mode the gradients of both paths agree."""
    scene = scenes.config2(P=50_000, width=640, height=360)
    args = (scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs)
    default = GaussianModel.from_activated(*args, sh_degree=3, act_cache=True).to(gpu_device).eval()
    python_cov = GaussianModel.from_activated(*args, sh_degree=3, act_cache=True,
                                              compute_cov3D_python=True).to(gpu_device).eval()
    a, b = default(scene.camera), python_cov(scene.camera)
    cov = python_cov.get_covariance(1.0).cpu()
    want_cov = np.stack([co.cov3d(python_cov.get_scaling[i].cpu().numpy(), 1.0, python_cov.get_rotation[i].cpu().numpy())
                         for i in range(0, scene.P, 97)])
    np.testing.assert_allclose(cov.numpy()[::97], want_cov, rtol=0, atol=2e-6 * float(np.abs(want_cov).max()))
    act = scenes.GaussianScene("act", python_cov.get_xyz.cpu(), python_cov.get_scaling.cpu(),
                               python_cov.get_rotation.cpu(), python_cov.get_opacity.cpu(),
                               python_cov.get_features.cpu(), 3, scene.cameras, scene.bg)
    ref = co.render(oracle_frame(act), oracle_gaussians(act, cov3D_precomp=cov.numpy()))
    check_images(dict(image=b.cpu().numpy()), ref, "compute_cov3D_python")
    np.testing.assert_array_equal(python_cov.visibility_filter.cpu().numpy(), ref["radii"] > 0)
    np.testing.assert_array_equal(python_cov.radii.cpu().numpy(), ref["radii"][ref["radii"] > 0])
    assert psnr(a.cpu().numpy(), b.cpu().numpy()) >= 60.0
    assert int((default.visibility_filter != python_cov.visibility_filter).sum()) <= 5

    # training mode: gradients reach scales and rotations through the torch covariance and cov3D_precomp's gradient
    small = scenes.tiny_scene(P=500, width=96, height=64, sh_degree=2, seed=31)
    grads = []
    target = torch.rand(3, 64, 96, generator=torch.Generator().manual_seed(1)).to(gpu_device)
    for flag in (False, True):
        m = GaussianModel.from_activated(small.means3D, small.scales, small.rotations, small.opacities, small.shs,
                                         sh_degree=2, compute_cov3D_python=flag).to(gpu_device).train()
        for p in m.parameters():
            p.requires_grad_(True)
        ((m(small.camera) - target) ** 2).mean().backward()
        grads.append({n: p.grad.clone() for n, p in m.named_parameters()})
    for name in grads[0]:
        g0, g1 = grads[0][name], grads[1][name]
        assert torch.isfinite(g1).all() and float(g0.abs().max()) > 0, name
        assert float((g0 - g1).abs().max()) <= 2e-3 * float(g0.abs().max()), name


def test_octree_lod_mask_and_forward(gpu_device):
    scene = scenes.config5(A=20_000, width=480, height=270)
    g = torch.Generator().manual_seed(5)
    level = torch.randint(0, 5, (20_000,), generator=g)
    common = dict(n_offsets=scene.n_offsets)
    model = OctreeGS(scene.anchor, scene.anchor_feat, scene.offset, torch.log(scene.scaling), scene.rotation, level,
                     voxel_size=0.5, standard_dist=250.0, fork=2, fuse_prefilter=False, **common)
    scaffold = ScaffoldGS.from_scene(scene, fuse_prefilter=False)
    model.anchor_decoder.load_state_dict(scaffold.anchor_decoder.state_dict())
    model = model.to(gpu_device).eval()
    cam = scene.camera
    image = model(cam)
    # level-of-detail mask against the closed form level <= round(log2(standard_dist / dist)) clamped to [0, L-1]
    pos = scene.anchor.double() + (0.5 / 2) / (2.0 ** level.double())[:, None]
    dist = (pos - cam.camera_center.double()).norm(dim=1)
    want_level = torch.clamp(torch.round(torch.log2(250.0 / dist)), 0, 4)
    want = level.double() <= want_level
    got = model._anchor_mask.cpu()
    near_half = (torch.log2(250.0 / dist) % 1 - 0.5).abs() < 1e-4  # fp32 vs fp64 rounding at .5 boundaries
    assert torch.equal(got[~near_half], want[~near_half])
    assert 0 < int(got.sum()) < 20_000
    # anchors outside the mask never become visible
    assert not bool((model.voxel_visible_mask.cpu() & ~got).any())
    # the frame equals a Scaffold-GS render with the masked-out anchors excluded
    scaffold = scaffold.to(gpu_device).eval()
    image2 = scaffold(cam, render_exclude_filter=model._anchor_mask)
    assert torch.equal(image, image2)
    model.enable_lod = False
    assert torch.equal(model(cam), scaffold(cam))


def test_fused_prefilter_gives_the_same_frame(gpu_device):
    scene = scenes.config3(P=200_000, width=960, height=540)
    args = (scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs)
    plain = GaussianModel.from_activated(*args, sh_degree=3, act_cache=True, fuse_prefilter=False).to(gpu_device).eval()
    fused = GaussianModel.from_activated(*args, sh_degree=3, act_cache=True, fuse_prefilter=True).to(gpu_device).eval()
    a, b = plain(scene.camera), fused(scene.camera)
    assert torch.equal(a, b)
    assert torch.equal(plain.visibility_filter, fused.visibility_filter)
    assert torch.equal(plain.radii, fused.radii)
    assert 0 < int(fused.visibility_filter.sum()) < scene.P
    # a render_exclude_filter or a scale modifier falls back to the reference's two-pass sequence
    keep = torch.ones(scene.P, dtype=torch.bool, device=gpu_device)
    keep[::2] = False
    assert torch.equal(plain(scene.camera, render_exclude_filter=keep), fused(scene.camera, render_exclude_filter=keep))
    assert torch.equal(plain(scene.camera, scaling_modifier=0.7), fused(scene.camera, scaling_modifier=0.7))


def test_checkpoint_round_trip_renders_the_same_frame(gpu_device, tmp_path):
    """point_cloud.ply + state_dict.th written in the reference's layout, read back, rendered: identical frames."""
    from landmarksystem_amd import checkpoints as ck
    scene = scenes.config2(P=30_000, width=480, height=270)
    vanilla = GaussianModel.from_activated(scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs,
                                           sh_degree=3, fuse_prefilter=False).to(gpu_device).eval()
    ck.save_model(vanilla, tmp_path / "v")
    loaded = ck.load_gaussian_model(tmp_path / "v", device=gpu_device, fuse_prefilter=False).eval()
    frame = loaded(scene.camera)
    assert torch.equal(vanilla(scene.camera), frame) and float(frame.max()) > 0.0
    ref = vanilla_model_reference(loaded, scene.camera)  # the loaded tensors through the oracle
    check_images(dict(image=frame.cpu().numpy()), ref, "vanilla model from a checkpoint")
    np.testing.assert_array_equal(loaded.visibility_filter.cpu().numpy(), ref["radii"] > 0)

    anchors = scenes.config5(A=20_000, width=480, height=270)
    scaffold = ScaffoldGS.from_scene(anchors).to(gpu_device).eval()
    ck.save_model(scaffold, tmp_path / "s")
    loaded = ck.load_scaffold_gs(tmp_path / "s", device=gpu_device).eval()
    frame = loaded(anchors.camera)
    assert torch.equal(scaffold(anchors.camera), frame)
    check_anchor_model_frame(loaded, anchors.camera, frame, "Scaffold-GS from a checkpoint")

    level = torch.randint(0, 5, (20_000,), generator=torch.Generator().manual_seed(5))
    octree = OctreeGS(anchors.anchor, anchors.anchor_feat, anchors.offset, torch.log(anchors.scaling),
                      anchors.rotation, level, voxel_size=0.5, standard_dist=250.0, n_offsets=anchors.n_offsets)
    octree.anchor_decoder.load_state_dict(scaffold.anchor_decoder.state_dict())
    octree = octree.to(gpu_device).eval()
    ck.save_model(octree, tmp_path / "o")
    loaded = ck.load_octree_gs(tmp_path / "o", device=gpu_device).eval()
    frame = loaded(anchors.camera)
    assert torch.equal(octree(anchors.camera), frame)
    check_anchor_model_frame(loaded, anchors.camera, frame, "Octree-GS from a checkpoint")
    assert torch.equal(octree._anchor_mask, loaded._anchor_mask) and 0 < int(loaded._anchor_mask.sum()) < 20_000


def test_spatial_order_renders_the_same_frame(gpu_device, tmp_path):
    """Storing the scene along a Morton curve changes memory order only: the frame is the same."""
    from landmarksystem_amd import checkpoints as ck
    scene = scenes.config3(P=150_000, width=640, height=360)
    model = GaussianModel.from_activated(scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs,
                                         sh_degree=3, fuse_prefilter=True).to(gpu_device).eval()
    ck.save_model(model, tmp_path / "v")
    plain = ck.load_gaussian_model(tmp_path / "v", device=gpu_device, fuse_prefilter=True).eval()
    ordered = ck.load_gaussian_model(tmp_path / "v", device=gpu_device, fuse_prefilter=True, spatial_order=True).eval()
    a, b = plain(scene.camera), ordered(scene.camera)
    assert int(plain.visibility_filter.sum()) == int(ordered.visibility_filter.sum()) > 0
    # Gaussians of exactly equal fp32 depth blend in index order, as in the reference, and among 1e5 depths there
    # are hundreds of exact ties; where two of them share a pixel the swap moves it by ~alpha1 * alpha2 * |c1 - c2|
    diff = (a - b).abs()
    assert float(diff.max()) <= 2e-3 and float((diff > 1e-6).float().mean()) < 0.01
    assert psnr(a.cpu().numpy(), b.cpu().numpy()) >= 80.0


def _octree_pair(scene, gpu_device, **kw):
    level = torch.randint(0, 5, (scene.anchor.shape[0],), generator=torch.Generator().manual_seed(5))
    extra = torch.randn(scene.anchor.shape[0], generator=torch.Generator().manual_seed(6)) * 0.3
    models = []
    for fuse in (False, True):
        m = OctreeGS(scene.anchor, scene.anchor_feat, scene.offset, torch.log(scene.scaling), scene.rotation, level,
                     voxel_size=0.5, standard_dist=250.0, fork=2, extra_level=extra, n_offsets=scene.n_offsets,
                     fuse_prefilter=fuse, **kw)
        m.anchor_decoder.load_state_dict(ScaffoldGS.from_scene(scene).anchor_decoder.state_dict())
        models.append(m.to(gpu_device).eval())
    return models


@pytest.mark.parametrize("dist2level", ["round", "floor", "ceil"])
def test_fused_anchor_prefilter_matches_the_reference_sequence(gpu_device, dist2level):
    """One-kernel anchor prefilter (level-of-detail mask + visibility) against the models' own sequence of torch
    operations, gathers and visible_filter call."""
    scene = scenes.config5(A=40_000, width=640, height=360)
    cam = scene.camera
    plain = ScaffoldGS.from_scene(scene, fuse_prefilter=False).to(gpu_device).eval()
    fused = ScaffoldGS.from_scene(scene, fuse_prefilter=True).to(gpu_device).eval()
    a, b = plain(cam), fused(cam)
    assert torch.equal(plain.voxel_visible_mask, fused.voxel_visible_mask)
    assert 0 < int(fused.voxel_visible_mask.sum()) < 40_000
    assert torch.equal(a, b)

    ref, one = _octree_pair(scene, gpu_device, dist2level=dist2level)
    a, b = ref(cam), one(cam)
    # the predicted level is the same fp32 formula evaluated by different code: anchors within rounding of a
    # decision boundary of floor / round / ceil may differ
    anchor_pos = scene.anchor.double() + 0.25 / (2.0 ** ref._level.cpu().double())
    dist = (anchor_pos - cam.camera_center.double()).norm(dim=1)
    pred = torch.log2(250.0 / dist) + ref._extra_level.cpu().double()
    frac = pred - torch.floor(pred)
    edge = (frac - 0.5).abs() < 1e-4 if dist2level == "round" else (frac < 1e-4) | (frac > 1 - 1e-4)
    same = ref._anchor_mask.cpu() == one._anchor_mask.cpu()
    assert bool(same[~edge].all()) and int((~same).sum()) <= int(edge.sum())
    assert 0 < int(one._anchor_mask.sum()) < 40_000
    assert not bool((one.voxel_visible_mask & ~one._anchor_mask).any())
    if bool(same.all()):
        assert torch.equal(ref.voxel_visible_mask, one.voxel_visible_mask) and torch.equal(a, b)
    # closed form in float64 away from the boundaries
    R = {"round": torch.round, "floor": torch.floor, "ceil": torch.ceil}[dist2level]
    want = ref._level.cpu().double().squeeze(1) <= torch.clamp(R(pred), 0, 4)
    assert torch.equal(one._anchor_mask.cpu()[~edge], want[~edge])
    one.enable_lod = ref.enable_lod = False
    assert torch.equal(ref(cam), one(cam)) and bool(one._anchor_mask.all())
