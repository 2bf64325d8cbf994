"""Pins for the anchor-decode oracle (oracle/anchor_oracle.py) against what the
reference's module computes (landmark/nerf_components/model_components/fields/
anchor_decoder.py:79-104, 147-242): the MLPs as torch.nn.Sequential modules
built the way the reference builds them, and the reference's
"concatenate, repeat, mask, split" data flow restated with einops."""
import torch
from einops import repeat
from torch import nn

from landmarksystem_amd import scenes
from oracle import anchor_oracle as ao


def reference_style(camera_center, anchor, feat, offset, scaling, visible_mask, mlps, n_offsets):
    """The module's own formulation: nn.Sequential MLPs, einops repeat, one big cat / mask / split."""
    seq = {}
    for name, act in (("opacity", nn.Tanh()), ("cov", None), ("color", nn.Sigmoid())):
        w0, b0, w1, b1 = mlps[name]
        l0, l1 = nn.Linear(w0.shape[1], w0.shape[0]), nn.Linear(w1.shape[1], w1.shape[0])
        with torch.no_grad():
            l0.weight.copy_(w0), l0.bias.copy_(b0), l1.weight.copy_(w1), l1.bias.copy_(b1)
        layers = [l0, nn.ReLU(True), l1] + ([act] if act is not None else [])
        seq[name] = nn.Sequential(*layers)
    with torch.no_grad():
        anchor, feat = anchor[visible_mask], feat[visible_mask]
        grid_offsets, grid_scaling = offset[visible_mask], scaling[visible_mask]
        ob_view = anchor - camera_center
        ob_dist = ob_view.norm(dim=1, keepdim=True)
        ob_view = ob_view / ob_dist
        cat_local_view = torch.cat([feat, ob_view, ob_dist], dim=1)
        neural_opacity = seq["opacity"](cat_local_view).reshape([-1, 1])
        mask = (neural_opacity > 0.0).view(-1)
        opacity = neural_opacity[mask]
        color = seq["color"](cat_local_view).reshape([anchor.shape[0] * n_offsets, 3])
        scale_rot = seq["cov"](cat_local_view).reshape([anchor.shape[0] * n_offsets, 7])
        offsets = grid_offsets.view([-1, 3])
        concatenated = torch.cat([grid_scaling, anchor], dim=-1)
        concatenated_repeated = repeat(concatenated, "n (c) -> (n k) (c)", k=n_offsets)
        concatenated_all = torch.cat([concatenated_repeated, color, scale_rot, offsets], dim=-1)
        masked = concatenated_all[mask]
        scaling_repeat, repeat_anchor, color, scale_rot, offsets = masked.split([6, 3, 3, 7, 3], dim=-1)
        scaling_out = scaling_repeat[:, 3:] * torch.sigmoid(scale_rot[:, :3])
        rot = torch.nn.functional.normalize(scale_rot[:, 3:7])
        xyz = repeat_anchor + offsets * scaling_repeat[:, :3]
    return xyz, color, opacity, scaling_out, rot, mask


def test_decode_equals_the_modules_formulation():
    sc = scenes.config5(A=3000)
    g = torch.Generator().manual_seed(1)
    vis = torch.rand(sc.anchor.shape[0], generator=g) < 0.6
    cam = sc.camera.camera_center
    got = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, sc.n_offsets)
    xyz, color, opacity, scaling, rot, mask = reference_style(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling,
                                                              vis, sc.mlp, sc.n_offsets)
    assert torch.equal(got["keep"], mask)
    for name, want in (("xyz", xyz), ("color", color), ("opacity", opacity), ("scaling", scaling), ("rot", rot)):
        assert got[name].shape == want.shape
        assert torch.allclose(got[name], want, rtol=0, atol=1e-6), name


def test_decode_invariants():
    sc = scenes.config5(A=2000)
    vis = torch.ones(2000, dtype=torch.bool)
    vis[::3] = False
    out = ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10)
    G = int(out["keep"].sum())
    assert 0 < G < int(vis.sum()) * 10
    assert out["xyz"].shape == (G, 3) and out["opacity"].shape == (G, 1) and out["rot"].shape == (G, 4)
    assert (out["opacity"] > 0).all() and (out["opacity"] <= 1).all()  # tanh of a positive pre-activation
    assert (out["color"] >= 0).all() and (out["color"] <= 1).all()  # sigmoid (saturates in fp32 for large inputs)
    assert torch.allclose(out["rot"].norm(dim=1), torch.ones(G), atol=1e-6)
    # xyz - anchor = offset * anchor_scaling[:3], scaling <= anchor_scaling[3:6]
    rep = torch.arange(int(vis.sum())).repeat_interleave(10)[out["keep"]]
    a, s = sc.anchor[vis][rep], sc.scaling[vis][rep]
    off = sc.offset[vis].reshape(-1, 3)[out["keep"]]
    assert torch.allclose(out["xyz"] - a, off * s[:, :3], atol=1e-5)
    assert (out["scaling"] >= 0).all() and (out["scaling"] <= s[:, 3:6]).all()
    # invisible anchors contribute nothing; an all-false mask gives empty outputs
    none = ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling,
                     torch.zeros(2000, dtype=torch.bool), sc.mlp, 10)
    assert none["xyz"].shape == (0, 3)


def test_heads_without_distance_input():
    sc = scenes.config5(A=500)
    mlp = dict(sc.mlp)
    w0, b0, w1, b1 = mlp["cov"]
    mlp["cov"] = (w0[:, :35].contiguous(), b0, w1, b1)  # add_cov_dist=False drops the distance column
    vis = torch.ones(500, dtype=torch.bool)
    a = ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, mlp, 10,
                  add_dist=(True, False, True))
    b = ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10)
    assert torch.equal(a["keep"], b["keep"]) and torch.equal(a["color"], b["color"])
    assert not torch.allclose(a["rot"], b["rot"])


def reference_style_bank(feat, bank_weight):
    """The module's feature-bank statements (anchor_decoder.py:169-177) with its own unsqueeze / strided slice /
    repeat formulation; `bank_weight` [n,3] is the softmax output."""
    bank_weight = bank_weight.unsqueeze(dim=1)  # [n, 1, 3]
    feat = feat.unsqueeze(dim=-1)
    feat = (feat[:, ::4, :1].repeat([1, 4, 1]) * bank_weight[:, :, :1]
            + feat[:, ::2, :1].repeat([1, 2, 1]) * bank_weight[:, :, 1:2]
            + feat[:, ::1, :1] * bank_weight[:, :, 2:])
    return feat.squeeze(dim=-1)


def test_feature_bank_mix():
    g = torch.Generator().manual_seed(3)
    feat = torch.randn(50, 32, generator=g)
    w = torch.softmax(torch.randn(50, 3, generator=g), dim=1)
    got = ao.bank_mix(feat, w)
    assert torch.allclose(got, reference_style_bank(feat, w), rtol=0, atol=1e-6)
    # element by element: position j mixes features 4 (j mod 8), 2 (j mod 16) and j
    for j in (0, 1, 7, 8, 9, 15, 16, 31):
        want = feat[:, 4 * (j % 8)] * w[:, 0] + feat[:, 2 * (j % 16)] * w[:, 1] + feat[:, j] * w[:, 2]
        assert torch.allclose(got[:, j], want, atol=1e-6)
    # the weights sum to one: a constant feature vector is unchanged; weight (0, 0, 1) is the identity
    const = torch.full((4, 32), 0.7)
    assert torch.allclose(ao.bank_mix(const, w[:4]), const, atol=1e-6)
    assert torch.equal(ao.bank_mix(feat, torch.tensor([[0.0, 0.0, 1.0]]).expand(50, 3)), feat)


def _with_bank_and_level(sc, g, add_level):
    """Scene MLPs rebuilt for a decoder with a feature bank (and the level input): heads 36 wide reading
    [feat | view | level], or the scene's own heads without a level."""
    k = 4 if add_level else 3
    bank = (torch.randn(32, k, generator=g) * 0.5, torch.randn(32, generator=g) * 0.1,
            torch.randn(3, 32, generator=g) * 0.5, torch.randn(3, generator=g) * 0.1)
    level = torch.randint(0, 5, (sc.anchor.shape[0], 1), generator=g).float()
    return bank, level


def test_decode_with_feature_bank_and_level_equals_the_modules_formulation():
    """Both optional branches against the module's statements: bank weights from an nn.Sequential with Softmax, the
    strided-repeat mix, and [feat | view | level] fed to all three heads (the distance is dropped from both inputs
    once a level is given, anchor_decoder.py:181-182)."""
    sc = scenes.config5(A=1500)
    g = torch.Generator().manual_seed(9)
    vis = torch.rand(1500, generator=g) < 0.7
    cam = sc.camera.camera_center
    for add_level in (False, True):
        bank, level = _with_bank_and_level(sc, g, add_level)
        got = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, sc.n_offsets,
                        level=level, add_level=add_level, bank=bank)
        # the module's way
        bank_seq = nn.Sequential(nn.Linear(bank[0].shape[1], 32), nn.ReLU(True), nn.Linear(32, 3), nn.Softmax(dim=1))
        with torch.no_grad():
            bank_seq[0].weight.copy_(bank[0]), bank_seq[0].bias.copy_(bank[1])
            bank_seq[2].weight.copy_(bank[2]), bank_seq[2].bias.copy_(bank[3])
            a, f = sc.anchor[vis], sc.anchor_feat[vis]
            ob_view = a - cam
            ob_dist = ob_view.norm(dim=1, keepdim=True)
            ob_view = ob_view / ob_dist
            lv = level[vis]
            cat_view = torch.cat([ob_view, lv], dim=1) if add_level else ob_view
            f = reference_style_bank(f, bank_seq(cat_view))
            cat_local_view = torch.cat([f, ob_view, lv], dim=1) if add_level else torch.cat([f, ob_view, ob_dist], dim=1)
            assert cat_local_view.shape[1] == 36
            neural_opacity = torch.tanh(ao.mlp(cat_local_view, sc.mlp["opacity"])).reshape(-1, 1)
            color = torch.sigmoid(ao.mlp(cat_local_view, sc.mlp["color"])).reshape(-1, 3)
        mask = (neural_opacity > 0).view(-1)
        assert torch.equal(got["mask"], mask) and torch.equal(got["keep"], mask)
        assert torch.allclose(got["neural_opacity"], neural_opacity, atol=1e-6)
        assert torch.allclose(got["opacity"], neural_opacity[mask], atol=1e-6)
        assert torch.allclose(got["color"], color[mask], atol=1e-6)
    # the level really is an input: another level changes the opacities; without add_level it is ignored
    bank, level = _with_bank_and_level(sc, g, True)
    one = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10, level=level, add_level=True)
    two = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10, level=level + 1, add_level=True)
    off = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10, level=level + 1, add_level=False)
    ref = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10)
    assert not torch.allclose(one["neural_opacity"], two["neural_opacity"])
    assert torch.equal(off["neural_opacity"], ref["neural_opacity"])
    # a zero weight column for the level gives the 35-wide head on [feat | view]
    mlp0 = {h: (torch.cat([w0[:, :35], torch.zeros(32, 1)], 1), b0, w1, b1) for h, (w0, b0, w1, b1) in sc.mlp.items()}
    mlp35 = {h: (w0[:, :35].contiguous(), b0, w1, b1) for h, (w0, b0, w1, b1) in sc.mlp.items()}
    a = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, mlp0, 10, level=level, add_level=True)
    b = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, mlp35, 10, add_dist=(False, False, False))
    assert torch.allclose(a["neural_opacity"], b["neural_opacity"], atol=1e-6)


def test_training_outputs_cover_every_offset_of_the_visible_anchors():
    sc = scenes.config5(A=400)
    vis = torch.ones(400, dtype=torch.bool)
    vis[100:250] = False
    out = ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 10)
    assert out["neural_opacity"].shape == (250 * 10, 1) and out["mask"].shape == (2500,)
    assert torch.equal(out["neural_opacity"][out["mask"]], out["opacity"])
    assert int(out["mask"].sum()) == out["xyz"].shape[0]
