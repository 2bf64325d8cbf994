"""GPU parity of the MFMA anchor decode (through gs355_decode_count / _emit)
against the fp32 torch-CPU oracle of AnchorDecoder.forward."""
import numpy as np
import pytest
import torch

from landmarksystem_amd import scenes
from landmarksystem_amd.anchor_decoder import FusedAnchorDecoder
from oracle import anchor_oracle as ao

pytestmark = pytest.mark.gpu

# fp32 accumulation order differs between the matrix cores and torch's CPU GEMM, and the hi + lo fp16 operands carry
# 22 significant bits: random sweeps over every option reached 2.4e-5 on single outputs with large pre-activations
TOL = 3e-5


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


@pytest.mark.parametrize("A,features_too", [(20_000, False), (20_000, True), (300_000, True)])
def test_decode_with_weights_fp16_cannot_represent(gpu_device, A, features_too):
    """An fp32-trained checkpoint: weights (and features) with all 24 significant bits in use.  The decoder detects
    them and feeds the matrix cores hi + lo fp16 pairs; the result meets the same bar as with fp16-exact weights
    (rounding the weights to fp16 alone would move the outputs by ~1e-3)."""
    sc = scenes.config5(A=A)
    g = torch.Generator().manual_seed(77)
    mlp = {}
    for head, (w0, b0, w1, b1) in sc.mlp.items():
        mlp[head] = (w0 * (1.0 + 1e-3 * torch.randn(w0.shape, generator=g)), 0.1 * torch.randn(b0.shape, generator=g),
                     w1 * (1.0 + 1e-3 * torch.randn(w1.shape, generator=g)), 0.1 * torch.randn(b1.shape, generator=g))
        assert not torch.equal(mlp[head][0].half().float(), mlp[head][0])
    sc.mlp = mlp
    feat = sc.anchor_feat * (1.0 + 1e-3 * torch.randn(sc.anchor_feat.shape, generator=g)) if features_too else sc.anchor_feat
    vis = torch.rand(A, generator=g) < 0.6
    dec = build_decoder(sc, gpu_device)
    cam = sc.camera.camera_center
    got = dec(camera_center=cam.to(gpu_device), anchor=sc.anchor.to(gpu_device), anchor_feat=feat.to(gpu_device),
              offset=sc.offset.to(gpu_device), scaling=sc.scaling.to(gpu_device), visible_mask=vis.to(gpu_device))
    assert dec._decoder_struct(gpu_device).fp32_weights == 1
    redo = lambda keep=None: ao.decode(cam, sc.anchor, feat, sc.offset, sc.scaling, vis, sc.mlp,  # noqa: E731
                                       sc.n_offsets, keep_override=keep)
    compare(got, redo(), redo)
    # the one-call decode (count kept on the device) takes the same variant of the kernels
    dev = dec.decode_on_device(cam.to(gpu_device), sc.anchor.to(gpu_device), feat.to(gpu_device),
                               sc.offset.to(gpu_device), sc.scaling.to(gpu_device), vis.to(gpu_device))
    G = int(dev.counts[0])
    assert G == got[0].shape[0]
    assert torch.equal(dev.xyz[:G], got[0]) and torch.equal(dev.rot[:G], got[4])


@pytest.mark.parametrize("n_offsets", [1, 3, 4, 6])
def test_decode_heads_without_distance_and_fewer_offsets(gpu_device, n_offsets):
    """Fewer offsets leave the heads' last row tiles partly or wholly beyond their outputs (one offset: 7 covariance
    outputs in three tiles of 32 rows): the rows that do not exist must not disturb the ones that do."""
    sc = scenes.config5(A=3000, n_offsets=n_offsets)
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
    redo = lambda keep=None: ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp,  # noqa: E731
                                       n_offsets, add_dist=(True, True, False), keep_override=keep)
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
        FusedAnchorDecoder(False, True, True, True, 3, 32, 10, appearance_dim=32)
    with pytest.raises(NotImplementedError):
        FusedAnchorDecoder(False, True, True, True, 3, 64, 10)


def decoder_with(sc, device, g, use_feat_bank, add_level, add_dist):
    """A decoder with the given options and random weights of the right shapes; returns it with the oracle's view
    of the same weights."""
    dec = FusedAnchorDecoder(use_feat_bank=use_feat_bank, add_opacity_dist=add_dist[0], add_color_dist=add_dist[2],
                             add_cov_dist=add_dist[1], view_dim=3, feat_dim=32, n_offsets=sc.n_offsets,
                             add_level=add_level)
    with torch.no_grad():
        for p in dec.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * (0.5 if p.dim() == 1 else p.shape[1] ** -0.5)).half().float())
    mlp = {}
    for name, head in (("mlp_opacity", "opacity"), ("mlp_cov", "cov"), ("mlp_color", "color")):
        m = getattr(dec, name)
        mlp[head] = tuple(t.detach().clone() for t in (m[0].weight, m[0].bias, m[2].weight, m[2].bias))
    bank = None
    if use_feat_bank:
        m = dec.mlp_feature_bank
        bank = tuple(t.detach().clone() for t in (m[0].weight, m[0].bias, m[2].weight, m[2].bias))
    return dec.to(device).eval(), mlp, bank


@pytest.mark.parametrize("use_feat_bank,add_level", [(True, False), (False, True), (True, True)])
def test_decode_with_feature_bank_and_level(gpu_device, use_feat_bank, add_level):
    """The feature bank (anchor_decoder.py:163-177) and the level input (:179-186): with a level every head reads
    [feat | view | level], so the heads are built without distance inputs (the Octree-GS defaults)."""
    A = 20_000
    sc = scenes.config5(A=A)
    g = torch.Generator().manual_seed(7 + 2 * use_feat_bank + add_level)
    add_dist = (False, False, False) if add_level else (True, False, True)
    dec, mlp, bank = decoder_with(sc, gpu_device, g, use_feat_bank, add_level, add_dist)
    vis = torch.rand(A, generator=g) < 0.6
    level = torch.randint(0, 5, (A, 1), generator=g).float()
    cam = sc.camera.camera_center
    got = dec(camera_center=cam.to(gpu_device), anchor=sc.anchor.to(gpu_device), anchor_feat=sc.anchor_feat.to(gpu_device),
              offset=sc.offset.to(gpu_device), scaling=sc.scaling.to(gpu_device), visible_mask=vis.to(gpu_device),
              level=level.to(gpu_device))
    redo = lambda keep=None: ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, mlp, sc.n_offsets,  # noqa: E731
                                       add_dist=add_dist, keep_override=keep, level=level, add_level=add_level, bank=bank)
    compare(got, redo(), redo)
    assert got[0].shape[0] > A  # a real decode, not an empty one


def test_features_that_fp16_cannot_hold(gpu_device):
    """Anchor features of an fp32-trained checkpoint are general floats: they enter the matrix cores as hi + lo
    fp16 pairs, so the decode still meets the fp32 bar (weights remain fp16-representable here)."""
    A = 12_000
    sc = scenes.config5(A=A)
    g = torch.Generator().manual_seed(12)
    sc.anchor_feat = torch.randn(A, 32, generator=g) * 0.5  # not rounded to fp16
    assert not torch.equal(sc.anchor_feat.half().float(), sc.anchor_feat)
    dec = build_decoder(sc, gpu_device)
    vis = torch.rand(A, generator=g) < 0.8
    cam = sc.camera.camera_center
    got = dec(cam.to(gpu_device), sc.anchor.to(gpu_device), sc.anchor_feat.to(gpu_device), sc.offset.to(gpu_device),
              sc.scaling.to(gpu_device), vis.to(gpu_device))
    redo = lambda keep=None: ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp,  # noqa: E731
                                       sc.n_offsets, keep_override=keep)
    compare(got, redo(), redo)


def test_level_input_follows_the_reference_quirks(gpu_device):
    sc = scenes.config5(A=64)
    g = torch.Generator().manual_seed(1)
    args = [t.to(gpu_device) for t in (sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling)]
    level = torch.zeros(64, 1, device=gpu_device)
    # a head built with a distance column as well (37 wide) cannot be fed by the reference's forward
    dec, _, _ = decoder_with(sc, gpu_device, g, False, True, (True, False, False))
    assert dec.mlp_opacity[0].weight.shape == (32, 37)
    with pytest.raises(RuntimeError, match="shape mismatch"):
        dec(*args, None, level)
    # add_level without a level tensor: the input lacks the column the heads were built for
    dec, _, _ = decoder_with(sc, gpu_device, g, False, True, (False, False, False))
    with pytest.raises(RuntimeError, match="no level was given"):
        dec(*args, None, None)
    # without add_level a level tensor is ignored
    dec, mlp, _ = decoder_with(sc, gpu_device, g, False, False, (True, True, True))
    a, b = dec(*args, None, level), dec(*args, None, None)
    assert all(torch.equal(x, y) for x, y in zip(a[:5], b[:5]))


def test_training_mode_returns_every_opacity_and_the_mask(gpu_device):
    """anchor_decoder.py:239-242: in training mode the 7-tuple also carries the opacity of every offset of the
    visible anchors and the mask that selected the Gaussians (here from the kernels: no gradients asked for)."""
    A = 9000
    sc = scenes.config5(A=A)
    dec = build_decoder(sc, gpu_device).train()
    vis = torch.rand(A, generator=torch.Generator().manual_seed(4)) < 0.5
    cam = sc.camera.camera_center
    with torch.no_grad():
        out = dec(cam.to(gpu_device), sc.anchor.to(gpu_device), sc.anchor_feat.to(gpu_device),
                  sc.offset.to(gpu_device), sc.scaling.to(gpu_device), vis.to(gpu_device))
    ref = ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp, sc.n_offsets)
    neural_opacity, mask = out[5], out[6]
    a_vis = int(vis.sum())
    assert neural_opacity.shape == (a_vis * 10, 1) and mask.shape == (a_vis * 10,) and mask.dtype == torch.bool
    want = ref["neural_opacity"].numpy()
    assert float(np.abs(neural_opacity.cpu().numpy() - want).max()) <= TOL
    sure = np.abs(ref["raw_opacity"].numpy()) > UNSURE
    np.testing.assert_array_equal(mask.cpu().numpy()[sure], ref["mask"].numpy()[sure])
    assert torch.equal(neural_opacity[mask], out[2]) and int(mask.sum()) == out[0].shape[0]
    redo = lambda keep=None: ao.decode(cam, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling, vis, sc.mlp,  # noqa: E731
                                       sc.n_offsets, keep_override=keep)
    compare(out[:5] + (None, None), ref, redo)
    assert dec.eval()(cam.to(gpu_device), sc.anchor.to(gpu_device), sc.anchor_feat.to(gpu_device),
                      sc.offset.to(gpu_device), sc.scaling.to(gpu_device), vis.to(gpu_device))[5] is None


def test_decode_on_device_and_the_two_pass_entry_points_agree(gpu_device):
    """gs355_decode (one call, count kept on the device) against gs355_decode_count + gs355_decode_emit (per-anchor
    offsets, exact output size) through the C ABI: the same Gaussians bit for bit."""
    import ctypes as C

    from landmarksystem_amd import _lib
    A = 70_001
    sc = scenes.config5(A=A)
    dec = build_decoder(sc, gpu_device)
    vis = (torch.rand(A, generator=torch.Generator().manual_seed(8)) < 0.4).to(gpu_device)
    t = [x.to(gpu_device).contiguous() for x in (sc.camera.camera_center, sc.anchor, sc.anchor_feat, sc.offset, sc.scaling)]
    res = dec.decode_on_device(*t, vis)
    G, a_vis = dec.read_counts(res)
    assert a_vis == int(vis.sum()) and 0 < G < a_vis * 10 and res.xyz.shape[0] == A * 10
    exact = dec(*t, vis)
    assert exact[0].shape[0] == G
    lib = _lib.load()
    d = dec._decoder_struct(gpu_device)
    an = _lib.Anchors()
    an.A, an.campos, an.anchor, an.feat, an.offset, an.scaling = A, *(x.data_ptr() for x in t)
    an.visible_mask = vis.data_ptr()
    need = C.c_size_t()
    _lib.check(lib.gs355_decode_scratch_bytes(A, C.byref(need)))
    scratch = torch.empty(need.value, dtype=torch.uint8, device=gpu_device)
    counts = torch.empty(A, dtype=torch.int32, device=gpu_device)
    offsets = torch.empty(A, dtype=torch.int32, device=gpu_device)
    stream = torch.cuda.current_stream(gpu_device).cuda_stream
    _lib.check(lib.gs355_decode_count(C.byref(d), C.byref(an), counts.data_ptr(), offsets.data_ptr(), scratch.data_ptr(),
                                      scratch.numel(), stream))
    assert int(offsets[-1] + counts[-1]) == G
    outs = [torch.empty((G, k), device=gpu_device) for k in (3, 3, 1, 3, 4)]
    o = _lib.Decoded()
    o.xyz, o.color, o.opacity, o.scaling, o.rot = (x.data_ptr() for x in outs)
    _lib.check(lib.gs355_decode_emit(C.byref(d), C.byref(an), offsets.data_ptr(), G, C.byref(o), stream))
    torch.cuda.synchronize()
    for name, two_pass, one_call, sliced in zip(("xyz", "color", "opacity", "scaling", "rot"), outs, exact[:5],
                                                (res.xyz, res.color, res.opacity, res.scaling, res.rot)):
        assert torch.equal(two_pass, one_call), name
        assert torch.equal(sliced[:G], one_call), name


def test_model_frames_without_reading_the_gaussian_count_back(gpu_device):
    """Scaffold- / Octree-GS with the fused path: the decode leaves the number of Gaussians on the device and the
    rasterizer takes it from there.  Same frame as the sequence that reads it back, also through the classic
    stages (images beyond the tile-bucket limit), and the by-products appear when they are asked for."""
    from landmarksystem_amd.models import ScaffoldGS
    for width, height in ((640, 360), (4000, 2400)):
        scene = scenes.config5(A=30_000, width=width, height=height)
        plain = ScaffoldGS.from_scene(scene, fuse_prefilter=False).to(gpu_device).eval()
        fused = ScaffoldGS.from_scene(scene, fuse_prefilter=True).to(gpu_device).eval()
        a, b = plain(scene.camera), fused(scene.camera)
        assert torch.equal(a, b) and float(a.max()) > 0.1
        assert fused._pending is not None  # nothing was read back yet
        assert torch.equal(plain.visibility_filter, fused.visibility_filter) and fused._pending is None
        assert torch.equal(plain(scene.camera), fused(scene.camera))  # a second frame over the same buffers
