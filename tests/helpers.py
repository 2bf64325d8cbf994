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


def psnr(a, b):
    mse = float(np.mean((np.asarray(a, np.float64) - np.asarray(b, np.float64)) ** 2))
    return float("inf") if mse == 0 else -10.0 * math.log10(mse)


def u64(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint64)


def u32(t: torch.Tensor) -> np.ndarray:
    return t.cpu().numpy().view(np.uint32)
