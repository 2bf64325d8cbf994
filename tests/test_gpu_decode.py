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


UNSURE = 1e-5  # |opacity| below this: the matrix cores and the CPU GEMM may put the offset on either side of the mask


def compare(got, ref, redo):
    """GPU outputs against the oracle's.  Offsets whose decoded opacity is within UNSURE of zero may legitimately fall
    on either side of the mask `opacity > 0`; every other offset must be present, in order, within TOL.  `redo(keep)`
    re-runs the oracle with a given keep mask (to obtain its values for the doubtful offsets the GPU kept)."""
    xyz, color, opacity, scaling, rot, x5, x6 = got
    assert x5 is None and x6 is None
    raw = ref["raw_opacity"].numpy()
    sure, unsure = raw > UNSURE, np.abs(raw) <= UNSURE
    G = int(xyz.shape[0])
    assert int(sure.sum()) <= G <= int(sure.sum() + unsure.sum())
    if unsure.any():
        # decide, doubtful offset by doubtful offset, whether the GPU kept it: at the slot it would occupy the GPU's
        # position must be the oracle's position of that offset and its opacity must be tiny
        wide = redo(torch.from_numpy(sure | unsure))
        wide_index = np.flatnonzero(sure | unsure)
        slot_in_wide = {int(i): k for k, i in enumerate(wide_index)}
        gx, go = xyz.cpu().numpy(), opacity.cpu().numpy().reshape(-1)
        keep = sure.copy()
        kept_before = np.cumsum(sure) - sure  # sure offsets before each flat index
        extra = 0
        for i in np.flatnonzero(unsure):
            slot = int(kept_before[i]) + extra
            w = wide["xyz"][slot_in_wide[int(i)]].numpy()
            if slot < G and abs(go[slot]) <= 4 * UNSURE and np.abs(gx[slot] - w).max() <= TOL * max(1.0, np.abs(w).max()):
                keep[i] = True
                extra += 1
        ref = redo(torch.from_numpy(keep))
        print("decode: %d offsets within %g of the mask threshold, %d kept by the GPU" % (int(unsure.sum()), UNSURE, extra))
    assert G == ref["xyz"].shape[0]
    for name, t in (("xyz", xyz), ("color", color), ("opacity", opacity), ("scaling", scaling), ("rot", rot)):
        want = ref[name].numpy()
        assert t.shape == want.shape, name
        err = float(np.abs(t.cpu().numpy() - want).max()) if want.size else 0.0
        scale = max(1.0, float(np.abs(want).max())) if want.size else 1.0
        assert err / scale <= TOL, "%s: max-abs %g (scale %g)" % (name, err, scale)


@pytest.mark.parametrize("A,frac", [(5000, 0.5), (33, 1.0), (1, 1.0), (4097, 0.1), (100_000, 0.35), (500_000, 0.45),
                                    (500_000, 1.0)])
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
    redo = lambda keep=None: ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp,  # noqa: E731
                                       sc.n_offsets, keep_override=keep)
    compare(got, redo(), redo)


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
    redo = lambda keep=None: ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, 6,  # noqa: E731
                                       add_dist=(True, True, False), keep_override=keep)
    compare(got, redo(), redo)


def test_decode_nothing_visible_and_default_mask(gpu_device):
    sc = scenes.config5(A=700)
    dec = build_decoder(sc, gpu_device)
    cam = sc.camera.camera_center.to(gpu_device)
    args = (sc.anchor.to(gpu_device), sc.anchor_feat.to(gpu_device), sc.offset.to(gpu_device),
            sc.scaling.to(gpu_device))
    out = dec(cam, *args, torch.zeros(700, dtype=torch.bool, device=gpu_device))
    assert out[0].shape == (0, 3) and out[4].shape == (0, 4)
    out = dec(cam, *args, None)  # visible_mask=None means every anchor
    redo = lambda keep=None: ao.decode(sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling,  # noqa: E731
                                       None, sc.mlp, 10, keep_override=keep)
    compare(out, redo(), redo)


def test_unsupported_configurations_are_refused():
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(True, True, True, True, 3, 32, 10)
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(False, True, True, True, 3, 32, 10, add_level=True)
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(False, True, True, True, 3, 64, 10)
