"""Host-side checks of the inference-engine shim and the models' checkpoint protocol (no GPU): config
handling, the reference's sanity assertions (landmark/__init__.py:47-58), the one-rank rule, and
`get_state_dict_from_ckpt` -> `load_from_state_dict` filling a config-built (empty) model."""
import pytest
import torch

from landmarksystem_amd import checkpoints as ck
from landmarksystem_amd import engine as eng
from landmarksystem_amd.models import GaussianModel, OctreeGS, ScaffoldGS


def test_config_is_attribute_addressable(tmp_path):
    c = eng.Config({"runtime": "Kernel", "parallel_config": {"tp_size": 1}})
    assert c.runtime == "Kernel" and c.parallel_config.tp_size == 1
    assert not hasattr(c, "offload_config")
    c.ckpt_path = "x"
    assert c["ckpt_path"] == "x"
    f = tmp_path / "conf.py"
    f.write_text("runtime = 'Torch'\nkernel_fusion = False\n_private = 1\n")
    c = eng.Config.from_file(f)
    assert c.runtime == "Torch" and c.kernel_fusion is False and "_private" not in c


def test_postprocess_default_returns_single_result_bare():
    assert eng._plain_postprocess(5) == 5
    assert eng._plain_postprocess(1, 2) == (1, 2)
    assert eng._plain_preprocess(1, a=2) == ((1,), {"a": 2})


@pytest.mark.parametrize("bad", [dict(half_precision=True), dict(static_allocation=True)])
def test_sanity_assertions(bad):
    with pytest.raises(AssertionError, match="not supportted yet"):
        eng.init_inference(GaussianModel, None, dict(ckpt="unused.ply"), dict(runtime="Kernel", **bad))


def test_act_cache_with_offload_is_refused():
    with pytest.raises(AssertionError, match="Offload is not supportted when act_cache is True"):
        eng.init_inference(GaussianModel, None, dict(ckpt="unused.ply", act_cache=True),
                           dict(runtime="Torch", offload_config=dict(local_plane_split=[1, 1])))


def test_more_than_one_rank_is_refused():
    with pytest.raises(NotImplementedError, match="one GPU"):
        eng.init_inference(GaussianModel, None, dict(ckpt="unused.ply"),
                           dict(runtime="Kernel", parallel_config=dict(tp_size=4)))


def test_checkpoint_is_required_with_a_model_config():
    with pytest.raises(AssertionError, match="should set the checkpoint file path"):
        eng.init_inference(GaussianModel, None, dict(sh_degree=3), dict(runtime="Kernel"))


def test_unknown_runtime(tmp_path):
    g = torch.Generator().manual_seed(0)
    m = GaussianModel(torch.randn(4, 3, generator=g), torch.randn(4, 1, 3, generator=g), torch.randn(4, 15, 3, generator=g),
                      torch.randn(4, 3, generator=g), torch.randn(4, 4, generator=g), torch.randn(4, 1, generator=g))
    ck.save_model(m, tmp_path)
    with pytest.raises(ValueError, match="Jit"):
        eng.init_inference(GaussianModel, None, dict(ckpt=str(tmp_path / "point_cloud.ply")), dict(runtime="Jit"))


def _anchor_model(cls, g, **kw):
    r = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    m = cls(r(6, 3), r(6, 32), r(6, 10, 3), r(6, 6), r(6, 4), opacity=r(6, 1), **kw)
    for p in m.anchor_decoder.parameters():
        p.data = torch.randn(p.shape, generator=g)
    return m


def test_config_built_models_load_their_checkpoints(tmp_path):
    g = torch.Generator().manual_seed(2)
    v = GaussianModel(torch.randn(5, 3, generator=g), torch.randn(5, 1, 3, generator=g), torch.randn(5, 15, 3, generator=g),
                      torch.randn(5, 3, generator=g), torch.randn(5, 4, generator=g), torch.randn(5, 1, generator=g))
    ck.save_model(v, tmp_path / "v")
    empty = GaussianModel(dict(sh_degree=3, act_cache=True, white_bkgd=True))  # the reference's (config, ...) call
    assert empty._xyz.shape == (0, 3) and empty.act_cache and empty.background.tolist() == [1.0, 1.0, 1.0]
    state = empty.get_state_dict_from_ckpt(tmp_path / "v" / "point_cloud.ply", "cpu")
    assert set(state) == {"gaussian_encoding." + k for k in
                          ("_xyz", "_features_dc", "_features_rest", "_opacity", "_scaling", "_rotation")}
    empty.load_from_state_dict(state)
    assert all(torch.equal(a, b) for a, b in zip(v.parameters(), empty.parameters()))
    with pytest.raises(ValueError, match="only found keys"):
        GaussianModel(dict(sh_degree=3)).load_from_state_dict({"gaussian_encoding._opacity": torch.zeros(2, 1)})
    with pytest.raises(ValueError, match="not found any param keys"):
        GaussianModel(dict(sh_degree=3)).load_from_state_dict({})

    s = _anchor_model(ScaffoldGS, g)
    ck.save_model(s, tmp_path / "s")
    empty = ScaffoldGS(config=dict(n_offsets=10, feat_dim=32), scene_manager=None)
    empty.load_from_state_dict(empty.get_state_dict_from_ckpt(tmp_path / "s" / "point_cloud.ply", "cpu"))
    assert [n for n, _ in s.named_parameters()] == [n for n, _ in empty.named_parameters()]
    assert all(torch.equal(a, b) for a, b in zip(s.parameters(), empty.parameters()))
    with pytest.raises(ValueError, match="only found keys"):
        ScaffoldGS(config={}).load_from_state_dict({"gaussian_encoding._anchor": torch.zeros(2, 3)})
    banked = ScaffoldGS(config=dict(use_feat_bank=True))  # the feature bank is a fourth MLP of the decoder
    assert banked.anchor_decoder.mlp_feature_bank[0].weight.shape == (32, 3)
    assert banked.anchor_decoder.mlp_feature_bank[2].weight.shape == (3, 32)

    o = _anchor_model(OctreeGS, g, level=torch.tensor([0, 1, 2, 0, 1, 2]), voxel_size=0.25, standard_dist=40.0,
                      extra_level=torch.randn(6, generator=g), add_opacity_dist=False, add_cov_dist=False,
                      add_color_dist=False)
    ck.save_model(o, tmp_path / "o")
    empty = OctreeGS(dict(n_offsets=10, feat_dim=32, fork=2, dist2level="round", appearance_dim=0))
    assert empty.anchor_decoder.mlp_opacity[0].weight.shape == (32, 35)  # Octree-GS default: no distance inputs
    empty.load_from_state_dict(empty.get_state_dict_from_ckpt(tmp_path / "o" / "point_cloud.ply", "cpu"))
    assert empty.voxel_size == 0.25 and empty.standard_dist == 40.0
    assert torch.equal(o._level, empty._level) and torch.equal(o._extra_level, empty._extra_level)
    assert all(torch.equal(a, b) for a, b in zip(o.parameters(), empty.parameters()))
    with pytest.raises(NotImplementedError, match="appearance_dim"):
        OctreeGS(dict(appearance_dim=32))
    # the Scaffold-GS model never hands add_level / appearance_dim to its decoder (scaffold_gs/gs_model.py:126-134),
    # so its config's add_level=True default (:33) must be accepted
    plain = ScaffoldGS(dict(n_offsets=10, feat_dim=32, add_level=True, appearance_dim=32))
    assert plain.anchor_decoder.mlp_opacity[0].weight.shape == (32, 36) and not plain.anchor_decoder.add_level
    # Octree-GS does hand them over (octree_gs/gs_model.py:165-176): the level widens every head and the bank's input
    levelled = OctreeGS(dict(n_offsets=10, feat_dim=32, add_level=True, use_feat_bank=True))
    assert levelled.anchor_decoder.add_level and levelled.anchor_decoder.mlp_opacity[0].weight.shape == (32, 36)
    assert levelled.anchor_decoder.mlp_feature_bank[0].weight.shape == (32, 4)
    # a checkpoint with a feature bank and a level input loads into a decoder of the same shape
    ob = _anchor_model(OctreeGS, g, level=torch.tensor([0, 1, 2, 0, 1, 2]), voxel_size=0.25, standard_dist=40.0,
                       add_opacity_dist=False, add_cov_dist=False, add_color_dist=False, use_feat_bank=True,
                       add_level=True)
    ck.save_model(ob, tmp_path / "ob")
    back = ck.load_octree_gs(tmp_path / "ob", device="cpu")
    assert back.anchor_decoder.use_feat_bank and back.anchor_decoder.add_level
    assert not back.anchor_decoder.add_opacity_dist
    assert all(torch.equal(a, b) for a, b in zip(ob.anchor_decoder.parameters(), back.anchor_decoder.parameters()))


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU error")
def test_engine_needs_a_gpu(tmp_path):
    g = torch.Generator().manual_seed(0)
    ck.save_model(_anchor_model(ScaffoldGS, g), tmp_path)
    with pytest.raises(RuntimeError, match="needs a GPU"):
        eng.init_inference(ScaffoldGS, None, dict(ckpt=str(tmp_path / "point_cloud.ply")), dict(runtime="Kernel"))
