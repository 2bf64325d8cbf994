"""Drop-in Python surface of the reference's rasterizer package.

The reference's GS models import `GaussianRasterizationSettings` and
`GaussianRasterizer` from the third-party package `opt_gaussian_rasterization`
(benchmarks/nerf/origin_gs/gs_model.py:5, scaffold_gs/gs_model.py:6,
octree_gs/gs_model.py:8) and use them as follows:

  - settings are built with 12 keyword fields, first with placeholders
    (image_height=0, viewmatrix=torch.Tensor([])) at model construction
    (origin_gs/gs_model.py:82-95) and then re-assigned every frame through the
    plain attribute `renderer.raster_settings` (:148-162);
  - `GaussianRasterizer(raster_settings=...)` is stored as a child of an
    nn.Module (:97) and built afresh per frame for the visibility prefilter
    (:297-312), so construction is cheap and the module owns no parameters or
    buffers;
  - `renderer(means3D=..., means2D=..., shs=..., colors_precomp=...,
    opacities=..., scales=..., rotations=..., cov3D_precomp=...)` returns a
    3-tuple whose first two entries are the [3,H,W] image and int32 radii
    (:211-220);
  - `rasterizer.visible_filter(means3D=..., scales=..., rotations=...,
    cov3D_precomp=...)` returns radii only (:327-329).

Forward only: the returned tensors never require grad (the reference's
inference engine calls the model under torch.no_grad(),
landmark/render/inference_engine/inference_engine.py:89-94).
"""
import warnings
from typing import NamedTuple, Optional

import torch
from torch import nn

from . import pipeline


class GaussianRasterizationSettings(NamedTuple):
    image_height: int
    image_width: int
    tanfovx: float
    tanfovy: float
    bg: torch.Tensor
    scale_modifier: float
    viewmatrix: torch.Tensor
    projmatrix: torch.Tensor
    sh_degree: int
    campos: torch.Tensor
    prefiltered: bool
    debug: bool


_warned_grad = False


def _note_forward_only(*tensors):
    global _warned_grad
    if _warned_grad or not torch.is_grad_enabled():
        return
    if any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors):
        _warned_grad = True
        warnings.warn(
            "landmarksystem_amd.GaussianRasterizer is forward-only: outputs do not carry gradients "
            "(call it under torch.no_grad(), as the reference's inference engine does)",
            stacklevel=3,
        )


class GaussianRasterizer(nn.Module):
    def __init__(self, raster_settings: GaussianRasterizationSettings):
        super().__init__()
        self.raster_settings = raster_settings
        # extra outputs of the last forward() beyond the reference's 3-tuple
        self.last_depth: Optional[torch.Tensor] = None
        self.last_alpha: Optional[torch.Tensor] = None
        self.last_num_keys = 0

    def visible_filter(self, means3D, scales=None, rotations=None, cov3D_precomp=None):
        """int32[P] screen-space radii; 0 for Gaussians that are culled or
        touch no tile.  Callers threshold with `> 0`."""
        inputs = pipeline.FrameInputs(self.raster_settings, means3D, scales=scales, rotations=rotations,
                                      cov3D_precomp=cov3D_precomp, need_colour=False)
        return pipeline.visible_filter(inputs)

    def forward(self, means3D, means2D=None, opacities=None, shs=None, colors_precomp=None, scales=None,
                rotations=None, cov3D_precomp=None):
        """Returns (image f32[3,H,W], radii i32[P], depth f32[1,H,W]).
        `means2D` only carries screen-space gradients in the reference's
        training loop and is ignored here.  Alpha (1 - final transmittance,
        f32[1,H,W]) is left in `self.last_alpha`."""
        _note_forward_only(means3D, opacities, shs, colors_precomp, scales, rotations, cov3D_precomp)
        if opacities is None:
            raise ValueError("opacities is required")
        inputs = pipeline.FrameInputs(self.raster_settings, means3D, opacities=opacities, shs=shs,
                                      colors_precomp=colors_precomp, scales=scales, rotations=rotations,
                                      cov3D_precomp=cov3D_precomp)
        out = pipeline.render(inputs)
        self.last_depth, self.last_alpha, self.last_num_keys = out.depth, out.alpha, out.num_keys
        return out.image, out.radii, out.depth
