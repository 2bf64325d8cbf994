"""GPU tests of the drop-in Python API (GaussianRasterizer.forward and
.visible_filter as the reference's models call them) against the CPU oracle."""
import numpy as np
import pytest
import torch

from landmarksystem_amd import GaussianRasterizer, scenes
from oracle import c_oracle as co
from tests.helpers import check_images, oracle_frame, oracle_gaussians, settings_for

pytestmark = pytest.mark.gpu


def test_forward_as_the_vanilla_model_calls_it(gpu_device):
    scene = scenes.config2(P=60_000, width=640, height=360)
    rast = GaussianRasterizer(raster_settings=settings_for(scene, gpu_device))
    d = scene.to(gpu_device)
    means2D = torch.zeros_like(d.means3D)
    with torch.no_grad():
        image, radii, extra = rast(means3D=d.means3D, means2D=means2D, shs=d.shs, colors_precomp=None,
                                   opacities=d.opacities, scales=d.scales, rotations=d.rotations, cov3D_precomp=None)
    ref = co.render(oracle_frame(scene), oracle_gaussians(scene))
    assert image.shape == (3, 360, 640) and image.dtype == torch.float32 and not image.requires_grad
    assert radii.shape == (scene.P,) and radii.dtype == torch.int32
    np.testing.assert_array_equal(radii.cpu().numpy(), ref["radii"])
    assert rast.last_num_keys == ref["num_keys"]
    check_images(dict(image=image.cpu().numpy(), depth=extra.cpu().numpy(), alpha=rast.last_alpha.cpu().numpy()), ref,
                 "forward as the vanilla model calls it")
    assert extra.shape == (1, 360, 640)
    # callers permute and clamp the image (tests/test_inference_framework/test_inference.py:195-197)
    assert image.permute(1, 2, 0).clamp(0, 1).shape == (360, 640, 3)


def test_visible_filter_with_strided_slices(gpu_device):
    """Callers pass `scales[:, :3]` of a wider tensor (origin_gs/gs_model.py:327-329;
    Scaffold-GS anchors carry 6 scale columns)."""
    scene = scenes.config3(P=50_000)
    s = settings_for(scene, gpu_device, sh_degree=1)
    rast = GaussianRasterizer(raster_settings=s)
    wide = torch.cat([scene.scales, scene.scales * 2], dim=1).to(gpu_device)  # [P,6]
    radii = rast.visible_filter(means3D=scene.means3D.to(gpu_device), scales=wide[:, :3],
                                rotations=scene.rotations.to(gpu_device), cov3D_precomp=None)
    ref = co.visible_filter(oracle_frame(scene), scene.means3D.numpy(), scales=scene.scales.numpy(),
                            rotations=scene.rotations.numpy())
    assert radii.dtype == torch.int32
    np.testing.assert_array_equal(radii.cpu().numpy(), ref)
    assert 0 < int((radii > 0).sum()) < scene.P


def test_prefilter_then_gather_is_result_neutral(gpu_device):
    """The reference renders only the Gaussians its visibility prefilter keeps
    (origin_gs/gs_model.py:199-208); the image must not depend on that gather."""
    scene = scenes.config2(P=40_000, width=480, height=270)
    s = settings_for(scene, gpu_device)
    d = scene.to(gpu_device)
    rast = GaussianRasterizer(s)
    full, radii_full, _ = rast(means3D=d.means3D, means2D=None, shs=d.shs, colors_precomp=None, opacities=d.opacities,
                               scales=d.scales, rotations=d.rotations, cov3D_precomp=None)
    pre = GaussianRasterizer(s._replace(sh_degree=1))
    mask = (pre.visible_filter(means3D=d.means3D, scales=d.scales[:, :3], rotations=d.rotations,
                               cov3D_precomp=None) > 0).nonzero().squeeze(-1)
    assert 0 < mask.numel() < scene.P
    sub, radii_sub, _ = rast(means3D=d.means3D[mask], means2D=None, shs=d.shs[mask], colors_precomp=None,
                             opacities=d.opacities[mask], scales=d.scales[mask], rotations=d.rotations[mask],
                             cov3D_precomp=None)
    assert torch.equal(full, sub)
    assert torch.equal(radii_full[mask], radii_sub) and int((radii_full > 0).sum()) == mask.numel()


def test_settings_on_host_and_scale_modifier(gpu_device):
    """Matrices given as CPU tensors are uploaded; scale_modifier reaches the covariance."""
    scene = scenes.tiny_scene(P=400, width=96, height=64, sh_degree=2, seed=12)
    s = settings_for(scene, torch.device("cpu"), scale_modifier=1.7)
    rast = GaussianRasterizer(s)
    d = scene.to(gpu_device)
    image, radii, _ = rast(means3D=d.means3D, means2D=None, shs=d.shs, colors_precomp=None, opacities=d.opacities,
                           scales=d.scales, rotations=d.rotations, cov3D_precomp=None)
    ref = co.render(oracle_frame(scene, scale_modifier=1.7), oracle_gaussians(scene))
    np.testing.assert_array_equal(radii.cpu().numpy(), ref["radii"])
    check_images(dict(image=image.cpu().numpy()), ref, "host-side settings, scale modifier 1.7")


def test_frames_in_flight_on_two_streams_are_independent(gpu_device):
    """Each stream gets its own workspace, so frames of different scenes can be in flight at once (the next
    frame's preprocess overlapping the current frame's blend) and still come out as when rendered alone."""
    from landmarksystem_amd import GaussianRasterizer
    a = scenes.config2(P=120_000, width=640, height=360).to(gpu_device)
    b = scenes.config3(P=150_000, width=512, height=288).to(gpu_device)

    def render(scene):
        rast = GaussianRasterizer(settings_for(scene, gpu_device))
        return rast(means3D=scene.means3D, means2D=None, shs=scene.shs, colors_precomp=None, opacities=scene.opacities,
                    scales=scene.scales, rotations=scene.rotations, cov3D_precomp=None)

    alone = [render(a), render(b)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=gpu_device), torch.cuda.Stream(device=gpu_device)]
    outs = []
    for k in range(8):
        with torch.cuda.stream(streams[k % 2]):
            outs.append(render(a if k % 2 == 0 else b))
    torch.cuda.synchronize()
    for k, (image, radii, depth) in enumerate(outs):
        want = alone[k % 2]
        assert torch.equal(image, want[0]) and torch.equal(radii, want[1]) and torch.equal(depth, want[2])


@pytest.mark.parametrize("P,keep", [(0, 0.5), (1, 1.0), (777, 0.0), (5000, 0.3), (300_001, 0.88), (70_000, 1.0)])
def test_gather_rows_equals_boolean_indexing(gpu_device, P, keep):
    """gs355_gather_rows (the eval-mode gather of origin_gs/gs_model.py:199-208 as one pass) against torch's
    boolean indexing, bit for bit: rows of 4, 12, 16, 24 and 192 bytes, a None entry, a strided source."""
    from landmarksystem_amd import pipeline
    g = torch.Generator().manual_seed(P)
    mask = (torch.rand(P, generator=g) < keep).to(gpu_device)
    wide = torch.randn(P, 6, generator=g).to(gpu_device)
    tensors = [torch.randn(P, 3, generator=g).to(gpu_device), torch.randn(P, 16, 3, generator=g).to(gpu_device), None,
               torch.randn(P, 1, generator=g).to(gpu_device), wide[:, :3], torch.randn(P, 4, generator=g).to(gpu_device),
               wide]
    got = pipeline.gather_rows(mask, tensors)
    assert got[2] is None
    for t, out in zip(tensors, got):
        if t is not None:
            want = t[mask]
            assert out.shape == want.shape and out.is_contiguous()
            assert torch.equal(out, want)
    with pytest.raises(ValueError):
        pipeline.gather_rows(mask, [torch.zeros(P + 1, 3, device=gpu_device)])
