"""GPU parity of the MFMA anchor decode (through gs355_decode_count / _emit)
against the fp32 torch-CPU oracle of AnchorDecoder.forward."""
import numpy as np
import pytest
import torch

from landmarksystem_amd import scenes
from landmarksystem_amd.anchor_decoder import FusedAnchorDecoder
from oracle import anchor_oracle as ao

pytestmark = pytest.mark.gpu

TOL = 2e-5  # fp32 accumulation order differs between the matrix cores and torch's CPU GEMM


def build_decoder(sc, device, add_dist=(True, True, True)):
    dec = FusedAnchorDecoder(use_feat_bank=False, add_opacity_dist=add_dist[0], add_color_dist=add_dist[2],
                             add_cov_dist=add_dist[1], view_dim=3, feat_dim=32, n_offsets=sc.n_offsets)
    state = {}
    for name, head in (("mlp_opacity", "opacity"), ("mlp_cov", "cov"), ("mlp_color", "color")):
        w0, b0, w1, b1 = sc.mlp[head]
        state.update({name + ".0.weight": w0, name + ".0.bias": b0, name + ".2.weight": w1, name + ".2.bias": b1})
    dec.load_state_dict(state)  # the reference's parameter names
    return dec.to(device).eval()


def compare(got, ref, A_vis):
    xyz, color, opacity, scaling, rot, x5, x6 = got
    assert x5 is None and x6 is None
    # opacities within rounding of zero may legitimately fall on either side of the mask
    raw = ref["raw_opacity"].numpy()
    unsure = int((np.abs(raw) < 1e-5).sum())
    G = ref["xyz"].shape[0]
    assert abs(xyz.shape[0] - G) <= unsure
    if xyz.shape[0] != G:
        pytest.skip("mask differs on an opacity within 1e-5 of zero")
    for name, t in (("xyz", xyz), ("color", color), ("opacity", opacity), ("scaling", scaling), ("rot", rot)):
        want = ref[name].numpy()
        assert t.shape == want.shape, name
        err = float(np.abs(t.cpu().numpy() - want).max()) if want.size else 0.0
        scale = max(1.0, float(np.abs(want).max())) if want.size else 1.0
        assert err / scale <= TOL, "%s: max-abs %g (scale %g)" % (name, err, scale)


@pytest.mark.parametrize("A,frac", [(5000, 0.5), (33, 1.0), (1, 1.0), (4097, 0.1), (100_000, 0.35)])
def test_decode_matches_oracle(gpu_device, A, frac):
    sc = scenes.config5(A=A)
    g = torch.Generator().manual_seed(A)
    vis = torch.rand(A, generator=g) < frac
    if A == 1:
        vis[:] = True
    dec = build_decoder(sc, gpu_device)
    cam = sc.camera.camera_center
    got = dec(camera_center=cam.to(gpu_device), anchor=sc.anchor.to(gpu_device),
              anchor_feat=sc.anchor_feat.to(gpu_device), offset=sc.offset.to(gpu_device),
              scaling=sc.scaling.to(gpu_device), visible_mask=vis.to(gpu_device))
    ref = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, sc.n_offsets)
    compare(got, ref, int(vis.sum()))


def test_decode_heads_without_distance_and_fewer_offsets(gpu_device):
    sc = scenes.config5(A=3000, n_offsets=6)
    mlp = dict(sc.mlp)
    w0, b0, w1, b1 = mlp["color"]
    mlp["color"] = (w0[:, :35].contiguous(), b0, w1, b1)
    sc.mlp = mlp
    dec = build_decoder(sc, gpu_device, add_dist=(True, True, False))
    vis = torch.ones(3000, dtype=torch.bool)
    vis[100:900] = False
    cam = sc.camera.camera_center
    got = dec(cam.to(gpu_device), sc.anchor.to(gpu_device), sc.anchor_feat.to(gpu_device), sc.offset.to(gpu_device),
              sc.scaling.to(gpu_device), vis.to(gpu_device))
    ref = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 6,
                    add_dist=(True, True, False))
    compare(got, ref, int(vis.sum()))


def test_decode_nothing_visible_and_default_mask(gpu_device):
    sc = scenes.config5(A=700)
    dec = build_decoder(sc, gpu_device)
    cam = sc.camera.camera_center.to(gpu_device)
    args = (sc.anchor.to(gpu_device), sc.anchor_feat.to(gpu_device), sc.offset.to(gpu_device),
            sc.scaling.to(gpu_device))
    out = dec(cam, *args, torch.zeros(700, dtype=torch.bool, device=gpu_device))
    assert out[0].shape == (0, 3) and out[4].shape == (0, 4)
    out = dec(cam, *args, None)  # visible_mask=None means every anchor
    ref = ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, None, sc.mlp, 10)
    compare(out, ref, 700)


def test_unsupported_configurations_are_refused():
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(True, True, True, True, 3, 32, 10)
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(False, True, True, True, 3, 32, 10, add_level=True)
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(False, True, True, True, 3, 64, 10)
