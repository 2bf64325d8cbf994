"""Shared test helpers: scene -> oracle inputs / rasterizer settings, metrics."""
import math

import numpy as np
import torch

from landmarksystem_amd import GaussianRasterizationSettings
from oracle import c_oracle as co


def oracle_frame(scene, cam=None, sh_degree=None, scale_modifier=1.0):
    cam = cam or scene.camera
    return co.Frame(
        cam.width, cam.height, math.tan(cam.FovX * 0.5), math.tan(cam.FovY * 0.5),
        cam.world_view_transform.cpu().numpy(), cam.full_proj_transform.cpu().numpy(),
        cam.camera_center.cpu().numpy(), scene.bg.cpu().numpy(), scale_modifier,
        scene.sh_degree if sh_degree is None else sh_degree,
    )


def oracle_gaussians(scene, colors_precomp=None, cov3D_precomp=None):
    kw = {}
    if colors_precomp is not None:
        kw["colors_precomp"] = colors_precomp
    else:
        kw["shs"] = scene.shs.numpy()
    if cov3D_precomp is not None:
        kw["cov3D_precomp"] = cov3D_precomp
    else:
        kw["scales"] = scene.scales.numpy()
        kw["rotations"] = scene.rotations.numpy()
    return co.Gaussians(scene.means3D.numpy(), scene.opacities.numpy(), **kw)


def settings_for(scene, device, cam=None, sh_degree=None, scale_modifier=1.0):
    cam = (cam or scene.camera).to(device)
    return GaussianRasterizationSettings(
        image_height=int(cam.height), image_width=int(cam.width),
        tanfovx=math.tan(cam.FovX * 0.5), tanfovy=math.tan(cam.FovY * 0.5),
        bg=scene.bg.to(device), scale_modifier=scale_modifier,
        viewmatrix=cam.world_view_transform, projmatrix=cam.full_proj_transform,
        sh_degree=scene.sh_degree if sh_degree is None else sh_degree,
        campos=cam.camera_center, prefiltered=False, debug=False,
    )


from oracle.compare import DEPTH_REL, IMG_TOL, PSNR_MIN, plane_errors, psnr  # noqa: E402,F401


def u64(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint64)


def u32(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)


# Numbers of every image comparison of the session, for the terminal summary (tests/conftest.py): label ->
# worst values seen under that label.
IMAGE_REPORT = {}


def _record(label, n_fragile, n_pixels, report):
    slot = IMAGE_REPORT.setdefault(label or "frame", {"frames": 0, "fragile": 0, "pixels": 0})
    slot["frames"] += 1
    slot["fragile"] = max(slot["fragile"], n_fragile)
    slot["pixels"] = max(slot["pixels"], n_pixels)
    for name, r in report.items():
        w = slot.setdefault(name, {"solid": 0.0, "all": 0.0, "over_tol": 0, "psnr": float("inf"), "bar": r["bar"]})
        w["solid"], w["all"] = max(w["solid"], r["solid"]), max(w["all"], r["all"])
        w["over_tol"], w["psnr"], w["bar"] = max(w["over_tol"], r["over_tol"]), min(w["psnr"], r["psnr"]), r["bar"]


def check_images(got, ref, label="", psnr_min=PSNR_MIN, want_depth=True, want_alpha=True, max_fragile_frac=0.02):
    """Image, depth and alpha of a frame against the oracle's (`ref` = co.render output with intermediates).

    `ref["fragile"]` counts, per pixel, the blend decisions the oracle took within rounding distance of their
    threshold (alpha < 1/255, T(1-alpha) < 1e-4); a second implementation with a different exp() may decide those
    the other way.  Bars:
      * pixels with no such decision: max-abs <= 1e-4; for depth, whose sums reach hundreds of scene units,
        max(1e-4, 4e-6 * largest depth of the frame), i.e. about 32 units in the last place of such a sum
        (5.6e-4 for the 6M-Gaussian city frame, whose depths reach 280), printed as the absolute number it is;
      * every pixel: max-abs <= 1e-4 + count * (largest colour / 255), i.e. each near-threshold decision may flip
        one contribution of weight 1/255 (for depth: largest view depth / 255, alpha: 1/255);
      * PSNR >= 60 dB over all pixels.
    Prints the fragile-pixel count and the all-pixel max-abs errors."""
    frag = ref["fragile"].astype(np.float64)
    n_fragile, n_pixels, errors = plane_errors(got, ref, want_depth, want_alpha)
    _record(label, n_fragile, n_pixels, errors)
    assert n_fragile <= max_fragile_frac * n_pixels, "%s too many threshold-adjacent pixels: %d" % (label, n_fragile)
    vis = ref["pre"]["radii"] > 0 if "pre" in ref else None
    if vis is not None and vis.any():
        colour_max = float(np.abs(ref["pre"]["rgb"][vis]).max())
        depth_max = float(np.abs(ref["pre"]["depth"][vis]).max())
    else:
        colour_max = float(max(1.0, np.abs(ref["image"]).max()))
        depth_max = float(max(1.0, np.abs(ref["depth"]).max())) if "depth" in ref else 1.0
    flips = {"image": colour_max, "depth": depth_max, "alpha": 1.0}  # largest single flipped contribution x 255
    report = []
    for name, r in errors.items():
        report.append("%s solid %.3g all %.3g (bar %.3g, %d px > 1e-4, PSNR %.1f dB)"
                      % (name, r["solid"], r["all"], r["bar"], r["over_tol"], min(r["psnr"], 999.0)))
        assert r["solid"] <= r["bar"], "%s %s max-abs %g on safe pixels (bar %g)" % (label, name, r["solid"], r["bar"])
        bound = r["bar"] + frag * (flips[name] / 255.0) * 1.01
        worst = float((r["diff"] - bound).max()) if r["diff"].size else 0.0
        assert worst <= 0.0, "%s %s exceeds the one-flip-per-decision bound by %g" % (label, name, worst)
        assert r["psnr"] >= psnr_min, "%s %s PSNR %g" % (label, name, r["psnr"])
    print("%s: %d threshold-adjacent pixels of %d; max-abs %s" % (label or "frame", n_fragile, n_pixels,
                                                                "; ".join(report)), flush=True)


def vanilla_model_reference(model, camera, bg=None):
    """Oracle frame of the Gaussians a (loaded) vanilla model holds: its own activated tensors, so that the
    log/exp and logit/sigmoid round trips of a checkpoint do not enter the comparison."""
    from landmarksystem_amd import scenes
    bg = model.background.cpu() if bg is None else bg
    act = scenes.GaussianScene("act", model.get_xyz.cpu(), model.get_scaling.cpu(), model.get_rotation.cpu(),
                               model.get_opacity.cpu(), model.get_features.cpu(), model.active_sh_degree,
                               [camera.to("cpu")], bg)
    return co.render(oracle_frame(act), oracle_gaussians(act))


def check_anchor_model_frame(model, camera, image, label=""):
    """A Scaffold-GS / Octree-GS frame `image = model(camera)` against the oracles, from the tensors the model holds.
    (1) oracle decode (fp32 torch) + oracle rasterizer of the anchors the model found visible: the decoded
        Gaussians agree to ~1e-5, so a few discrete radius / tile decisions may differ: PSNR >= 50 dB;
    (2) oracle rasterizer on the Gaussians the GPU decoder produced: radii > 0 bit for bit, image to the frame bars."""
    from landmarksystem_amd import scenes
    from oracle import anchor_oracle as ao
    cam = camera.to("cpu")
    dev = model.get_anchor.device
    dec_mod = model.anchor_decoder
    mlp = {}
    for head, m in (("opacity", dec_mod.mlp_opacity), ("cov", dec_mod.mlp_cov), ("color", dec_mod.mlp_color)):
        mlp[head] = tuple(t.detach().cpu() for t in (m[0].weight, m[0].bias, m[2].weight, m[2].bias))
    add_dist = (dec_mod.add_opacity_dist, dec_mod.add_cov_dist, dec_mod.add_color_dist)
    visible = model.voxel_visible_mask.cpu()
    bg = model.background.cpu()
    dec = ao.decode(cam.camera_center, model.get_anchor.cpu(), model.get_anchor_feat.cpu(), model.get_offset.cpu(),
                    model.get_scaling.cpu(), visible, mlp, dec_mod.n_offsets, add_dist=add_dist)
    tmp = scenes.GaussianScene("dec", dec["xyz"], dec["scaling"], dec["rot"], dec["opacity"],
                               torch.zeros(dec["xyz"].shape[0], 1, 3), 1, [cam], bg)
    ref = co.render(oracle_frame(tmp, sh_degree=1), oracle_gaussians(tmp, colors_precomp=dec["color"].numpy()),
                    keep_intermediates=False)
    unsure = int((dec["raw_opacity"].abs() < 1e-5).sum())
    assert abs(int(model.visibility_filter.shape[0]) - dec["xyz"].shape[0]) <= unsure + 2, label
    p = psnr(image.cpu().numpy(), ref["image"])
    assert p >= 50.0, "%s: PSNR %g against oracle decode + oracle rasterizer" % (label, p)
    xyz, color, opacity, scaling, rot, _, _ = dec_mod(
        camera_center=cam.camera_center.to(dev), anchor=model.get_anchor, anchor_feat=model.get_anchor_feat,
        offset=model.get_offset, scaling=model.get_scaling, visible_mask=model.voxel_visible_mask)
    tmp = scenes.GaussianScene("gpu-dec", xyz.cpu(), scaling.cpu(), rot.cpu(), opacity.cpu(),
                               torch.zeros(xyz.shape[0], 1, 3), 1, [cam], bg)
    ref2 = co.render(oracle_frame(tmp, sh_degree=1), oracle_gaussians(tmp, colors_precomp=color.cpu().numpy()))
    np.testing.assert_array_equal(model.visibility_filter.cpu().numpy(), ref2["radii"] > 0, err_msg=label)
    check_images(dict(image=image.cpu().numpy()), ref2, label + " (rasterizer on the GPU-decoded Gaussians)")
    return dec
