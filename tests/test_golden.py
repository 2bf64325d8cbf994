"""Committed golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py): frozen inputs with the
CPU checker's outputs.  CPU tests keep the checkers on them; GPU tests hold the HIP path to them through the same
entry points the models use.  Integer results must match exactly; images to 1e-4 outside the pixels the checker
flagged as threshold-adjacent and >= 60 dB overall; the decode to 3e-5 of the output scale."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import anchor_oracle as ao
from oracle import c_oracle as co
from tests.helpers import check_images

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
INT_OUTPUTS = ("radii", "tiles_touched", "keys", "values", "sorted_keys", "sorted_values", "ranges")


def raster_case(tag):
    z = np.load(os.path.join(GOLDEN, "raster_cases.npz"))
    ins = {k[len(tag) + 4:]: z[k] for k in z.files if k.startswith(tag + ".in.")}
    outs = {k[len(tag) + 5:]: z[k] for k in z.files if k.startswith(tag + ".out.")}
    return ins, outs


def decode_case():
    z = np.load(os.path.join(GOLDEN, "decode_case.npz"))
    return ({k[3:]: z[k] for k in z.files if k.startswith("in.")},
            {k[4:]: z[k] for k in z.files if k.startswith("out.")})


@pytest.mark.parametrize("tag", ["a", "b"])
def test_c_oracle_reproduces_the_golden_frames(tag):
    ins, want = raster_case(tag)
    W, H, deg = (int(v) for v in ins["meta"])
    frame = co.Frame(W, H, float(ins["tanfov"][0]), float(ins["tanfov"][1]), ins["viewmatrix"], ins["projmatrix"],
                     ins["campos"], ins["bg"], 1.0, deg)
    g = co.Gaussians(ins["means3D"], ins["opacities"], shs=ins["shs"], scales=ins["scales"], rotations=ins["rotations"])
    out = co.render(frame, g)
    out["tiles_touched"] = out["pre"]["tiles_touched"]
    for k in INT_OUTPUTS:
        np.testing.assert_array_equal(out[k], want[k], err_msg=k)
    assert [out["num_keys"], out["pairs_evaluated"], out["pairs_accepted"]] == want["stats"].tolist()
    assert int(want["stats"][0]) > 500 and want["image"].max() > 0.3  # the fixture is not a trivial frame
    for k in ("image", "depth", "alpha"):  # libm's expf may differ in the last bit between hosts
        np.testing.assert_allclose(out[k], want[k], rtol=0, atol=2e-6, err_msg=k)


def test_anchor_oracle_reproduces_the_golden_decode():
    ins, want = decode_case()
    t = lambda a: torch.from_numpy(a)  # noqa: E731
    mlp = {h: tuple(t(ins["%s.%s" % (h, k)]) for k in ("w0", "b0", "w1", "b1")) for h in ("opacity", "cov", "color")}
    out = ao.decode(t(ins["campos"]), t(ins["anchor"]), t(ins["anchor_feat"]), t(ins["offset"]), t(ins["scaling"]),
                    t(ins["visible"]), mlp, 10)
    assert want["xyz"].shape[0] > 100
    for k in ("xyz", "color", "opacity", "scaling", "rot"):
        assert out[k].shape == want[k].shape, k
        np.testing.assert_allclose(out[k].numpy(), want[k], rtol=0, atol=1e-5, err_msg=k)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["a", "b"])
@pytest.mark.parametrize("fast", [True, False])
def test_hip_path_reproduces_the_golden_frames(gpu_device, tag, fast):
    from landmarksystem_amd import GaussianRasterizationSettings, _lib, pipeline
    ins, want = raster_case(tag)
    W, H, deg = (int(v) for v in ins["meta"])
    d = lambda k: torch.from_numpy(ins[k]).to(gpu_device)  # noqa: E731
    st = GaussianRasterizationSettings(
        image_height=H, image_width=W, tanfovx=float(ins["tanfov"][0]), tanfovy=float(ins["tanfov"][1]), bg=d("bg"),
        scale_modifier=1.0, viewmatrix=d("viewmatrix"), projmatrix=d("projmatrix"), sh_degree=deg, campos=d("campos"),
        prefiltered=False, debug=False)
    inp = pipeline.FrameInputs(st, d("means3D"), opacities=d("opacities"), shs=d("shs"), scales=d("scales"),
                               rotations=d("rotations"))
    out = pipeline.FrameOutputs(inp)
    ws = pipeline.Workspace(gpu_device)
    n_keys = int(want["stats"][0])
    tiles = inp.tiles
    view = lambda name: ws.view(lay, name, inp.P, n_keys, tiles).cpu().numpy()  # noqa: E731
    if fast:
        lay = pipeline.run_stages(inp, out, ws, n_keys + 64, _lib.PIPELINE_FAST)
    else:  # the classic path materialises the emission-order pairs (the sort's ping-pong overwrites them later)
        lay = pipeline.run_stages(inp, out, ws, n_keys + 64,
                                  _lib.STAGE_PREPROCESS | _lib.STAGE_SCAN | _lib.STAGE_DUPLICATE)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(view("keys").view(np.uint64), want["keys"])
        np.testing.assert_array_equal(view("values").view(np.uint32), want["values"])
        pipeline.run_stages(inp, out, ws, n_keys + 64, _lib.STAGE_SORT | _lib.STAGE_RANGES | _lib.STAGE_BLEND)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.radii.cpu().numpy(), want["radii"])
    np.testing.assert_array_equal(view("tiles_touched").view(np.uint32), want["tiles_touched"])
    np.testing.assert_array_equal(view("sorted_keys").view(np.uint64), want["sorted_keys"])
    np.testing.assert_array_equal(view("sorted_values").view(np.uint32), want["sorted_values"])
    np.testing.assert_array_equal(view("ranges").view(np.uint32), want["ranges"])
    check_images(dict(image=out.image.cpu().numpy(), depth=out.depth.cpu().numpy(), alpha=out.alpha.cpu().numpy()), want,
                 "golden frame %s (%s stages)" % (tag, "shipped" if fast else "classic"))


@pytest.mark.gpu
def test_hip_decode_reproduces_the_golden_decode(gpu_device):
    from landmarksystem_amd.anchor_decoder import FusedAnchorDecoder
    ins, want = decode_case()
    dec = FusedAnchorDecoder(use_feat_bank=False, add_opacity_dist=True, add_color_dist=True, add_cov_dist=True,
                             view_dim=3, feat_dim=32, n_offsets=10)
    state = {}
    for name, head in (("mlp_opacity", "opacity"), ("mlp_cov", "cov"), ("mlp_color", "color")):
        for key, part in (("0.weight", "w0"), ("0.bias", "b0"), ("2.weight", "w1"), ("2.bias", "b1")):
            state["%s.%s" % (name, key)] = torch.from_numpy(ins["%s.%s" % (head, part)])
    dec.load_state_dict(state)
    dec = dec.to(gpu_device).eval()
    d = lambda k: torch.from_numpy(ins[k]).to(gpu_device)  # noqa: E731
    xyz, color, opacity, scaling, rot, _, _ = dec(camera_center=d("campos"), anchor=d("anchor"),
                                                  anchor_feat=d("anchor_feat"), offset=d("offset"),
                                                  scaling=d("scaling"), visible_mask=d("visible"))
    assert float(np.abs(want["raw_opacity"]).min()) > 1e-5  # no offset of the fixture sits on the mask threshold
    for name, got in (("xyz", xyz), ("color", color), ("opacity", opacity), ("scaling", scaling), ("rot", rot)):
        assert got.shape == want[name].shape, name
        scale = max(1.0, float(np.abs(want[name]).max()))
        assert float(np.abs(got.cpu().numpy() - want[name]).max()) / scale <= 3e-5, name
