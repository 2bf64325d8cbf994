"""GPU test of the inference-engine shim: the reference's usage pattern
(tests/test_inference_framework/test_inference.py:255-285, tests/utils.py:172-201) —
`engine = init_inference(ModelClass, InferModuleOrNone, model_config, inference_config)` then
`engine(viewpoint_cam, 1.0, None, None)` — against the same model built directly from tensors."""
import numpy as np
import pytest
import torch

from landmarksystem_amd import checkpoints as ck
from landmarksystem_amd import scenes
from landmarksystem_amd.engine import InferenceModule, init_inference
from landmarksystem_amd.models import GaussianModel, OctreeGS, ScaffoldGS

from tests.helpers import check_anchor_model_frame, check_images, vanilla_model_reference

pytestmark = pytest.mark.gpu


class InferenceOctreeGSModule(InferenceModule):
    """A user-side module in the reference's style: builds the model itself, reshapes the arguments."""

    def __init__(self, *args, **kwargs):
        super().__init__(model=OctreeGS(*args, **kwargs))

    def preprocess(self, viewpoint_cam, scaling_modifier, retain_grad, render_exclude_filter):
        return (viewpoint_cam, scaling_modifier, retain_grad, render_exclude_filter, -1), {}

    def forward(self, *args, **kwargs):
        return self.model(*args, **kwargs)

    def postprocess(self, out):
        return out


def test_engine_renders_checkpoints_like_the_direct_models(gpu_device, tmp_path):
    scene = scenes.config2(P=30_000, width=480, height=270)
    vanilla = GaussianModel.from_activated(scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs,
                                           sh_degree=3).to(gpu_device).eval()
    ck.save_model(vanilla, tmp_path / "v")
    engine = init_inference(GaussianModel, None, dict(ckpt=str(tmp_path / "v" / "point_cloud.ply"), sh_degree=3,
                                                      act_cache=True), dict(runtime="Kernel", kernel_fusion=True))
    out = engine(scene.camera, 1.0, None, None)
    assert out.shape == (3, 270, 480) and not out.requires_grad
    assert torch.equal(out, vanilla(scene.camera))
    assert "scaling" in engine.base_model._cache  # act_cache from the model config
    ref = vanilla_model_reference(engine.base_model, scene.camera)  # the engine's tensors through the oracle
    check_images(dict(image=out.cpu().numpy()), ref, "engine, vanilla checkpoint")
    np.testing.assert_array_equal(engine.base_model.visibility_filter.cpu().numpy(), ref["radii"] > 0)

    anchors = scenes.config5(A=20_000, width=480, height=270)
    scaffold = ScaffoldGS.from_scene(anchors).to(gpu_device).eval()
    ck.save_model(scaffold, tmp_path / "s")
    engine = init_inference(ScaffoldGS, None, dict(ckpt=str(tmp_path / "s" / "point_cloud.ply"), n_offsets=10,
                                                   feat_dim=32, add_opacity_dist=True, add_cov_dist=True,
                                                   add_color_dist=True), dict(runtime="Torch"))
    out = engine(anchors.camera, 1.0, None, None)
    assert torch.equal(out, scaffold(anchors.camera))
    check_anchor_model_frame(engine.base_model, anchors.camera, out, "engine, Scaffold-GS checkpoint")

    level = torch.randint(0, 5, (20_000,), generator=torch.Generator().manual_seed(5))
    octree = OctreeGS(anchors.anchor, anchors.anchor_feat, anchors.offset, torch.log(anchors.scaling),
                      anchors.rotation, level, voxel_size=0.5, standard_dist=250.0, n_offsets=anchors.n_offsets)
    octree.anchor_decoder.load_state_dict(scaffold.anchor_decoder.state_dict())
    octree = octree.to(gpu_device).eval()
    ck.save_model(octree, tmp_path / "o")
    config = dict(ckpt=str(tmp_path / "o" / "point_cloud.ply"), n_offsets=10, feat_dim=32, fork=2, dist2level="round",
                  appearance_dim=0, add_opacity_dist=True, add_cov_dist=True, add_color_dist=True, enable_lod=True)
    engine = init_inference(OctreeGS, InferenceOctreeGSModule, config, dict(runtime="Kernel"))
    assert engine.base_model.voxel_size == 0.5 and engine.base_model.standard_dist == 250.0
    out = engine(anchors.camera, 1.0, None, None)
    assert torch.equal(out, octree(anchors.camera))
    check_anchor_model_frame(engine.base_model, anchors.camera, out, "engine, Octree-GS checkpoint")


def test_render_trajectory_equals_frame_by_frame(gpu_device):
    from landmarksystem_amd.engine import render_trajectory
    scene = scenes.config4(P=200_000, width=640, height=360, n_poses=6)
    model = GaussianModel.from_activated(scene.means3D, scene.scales, scene.rotations, scene.opacities, scene.shs,
                                         sh_degree=3, act_cache=True, fuse_prefilter=True).to(gpu_device).eval()
    want = [model(cam).clone() for cam in scene.cameras]
    for in_flight in (1, 2, 3):
        got = list(render_trajectory(model, scene.cameras, in_flight=in_flight))
        torch.cuda.synchronize()
        assert len(got) == len(want)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
    assert len({float(w.sum()) for w in want}) == len(want)  # the poses really differ
