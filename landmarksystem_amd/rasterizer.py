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

Under torch.no_grad() (the reference's inference engine,
landmark/render/inference_engine/inference_engine.py:89-94) the call is the
plain forward pass.  When gradients are enabled and an input requires them
(the reference's training loop, benchmarks/nerf/origin_gs/gs_trainer.py:
117-124), the call goes through an autograd function whose backward is the
library's backward pass; `means2D` then receives the screen-space gradient
the reference's densification reads (gaussian_encoding.py:729-743).
"""
from types import SimpleNamespace
from typing import NamedTuple, Optional

import torch
from torch import nn
from torch.autograd.function import once_differentiable

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


_INPUT_NAMES = ("means3D", "means2D", "opacities", "shs", "colors_precomp", "scales", "rotations", "cov3D_precomp")


class _RasterizeGaussians(torch.autograd.Function):
    """forward(): one frame in a workspace of its own, kept until backward() has read it.

    Memory: every graph that is still waiting for its backward pass holds the whole workspace of its frame (records,
    keys, values, binning tables: about 0.7 GB at 6M Gaussians / 13.6M keys, 2 GB at 20M Gaussians in 4K), released
    when backward() has run or the graph is dropped.  The backward pass can run once per forward pass."""

    @staticmethod
    def forward(ctx, settings, means3D, means2D, opacities, shs, colors_precomp, scales, rotations, cov3D_precomp):
        inputs = pipeline.FrameInputs(settings, means3D, opacities=opacities, shs=shs, colors_precomp=colors_precomp,
                                      scales=scales, rotations=rotations, cov3D_precomp=cov3D_precomp)
        ws = pipeline.default_workspace(inputs.device)
        out = pipeline.render(inputs, ws=ws)
        # the next frame on this stream gets a fresh buffer; this one lives until the backward pass is done
        ctx.workspace, ws.buffer = ws.buffer, None
        ctx.settings, ctx.key_capacity = settings, out.key_capacity
        ctx.set_materialize_grads(False)
        # outputs go through save_for_backward too: kept on ctx directly they would tie it into a reference cycle
        ctx.save_for_backward(means3D, opacities, shs, colors_precomp, scales, rotations, cov3D_precomp,
                              out.image, out.depth, out.alpha, out.radii)
        ctx.means2D_like = None if means2D is None else (means2D.shape, means2D.dtype)
        ctx.mark_non_differentiable(out.radii)
        return out.image, out.radii, out.depth, out.alpha

    @staticmethod
    @once_differentiable
    def backward(ctx, g_image, _g_radii, g_depth, g_alpha):
        (means3D, opacities, shs, colors_precomp, scales, rotations, cov3D_precomp,
         image, depth, alpha, radii) = ctx.saved_tensors
        out = SimpleNamespace(image=image, depth=depth, alpha=alpha, radii=radii, key_capacity=ctx.key_capacity)
        originals = dict(means3D=means3D, opacities=opacities, shs=shs, colors_precomp=colors_precomp, scales=scales,
                         rotations=rotations, cov3D_precomp=cov3D_precomp)
        needs = dict(zip(_INPUT_NAMES, ctx.needs_input_grad[1:]))
        if g_image is None and g_depth is None and g_alpha is None:
            return (None,) * 9
        if ctx.workspace is None:
            raise RuntimeError("the rasterizer's backward pass ran already for this frame: its workspace is released "
                               "after the first backward pass (retain_graph=True cannot replay it); render the frame "
                               "again")
        inputs = pipeline.FrameInputs(ctx.settings, means3D, opacities=opacities, shs=shs,
                                      colors_precomp=colors_precomp, scales=scales, rotations=rotations,
                                      cov3D_precomp=cov3D_precomp)
        if g_image is None:
            g_image = torch.zeros_like(image)
        want = [n for n in _INPUT_NAMES if needs[n]]
        grads = pipeline.render_backward(inputs, out, ctx.workspace, g_image, g_depth, g_alpha, want=want)
        ctx.workspace = None
        result = [None]
        for n in _INPUT_NAMES:
            g = grads.get(n)
            if g is not None:
                if n == "means2D":
                    shape, dtype = ctx.means2D_like
                else:
                    shape, dtype = originals[n].shape, originals[n].dtype
                g = g.reshape(shape).to(dtype)
            result.append(g)
        return tuple(result)


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
                rotations=None, cov3D_precomp=None, count=None):
        """Returns (image f32[3,H,W], radii i32[P], depth f32[1,H,W]).
        `count` (an extension of the reference's signature): one-element int32 device tensor with the number of
        Gaussians when only the device knows it (the anchor decode's output); the inputs are then sized for a
        capacity P, rows at and beyond `count` are ignored and their radii are not written.  Inference only.
        `means2D` takes no part in the forward pass; when it requires grad it
        receives the screen-space gradient (normalised device units, third
        component zero).  Alpha (1 - final transmittance, f32[1,H,W]) is left
        in `self.last_alpha`; image, depth and alpha are all differentiable."""
        if opacities is None:
            raise ValueError("opacities is required")
        tensors = (means3D, means2D, opacities, shs, colors_precomp, scales, rotations, cov3D_precomp)
        if torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors):
            if count is not None:
                raise ValueError("a device-side Gaussian count cannot be combined with gradients")
            image, radii, depth, alpha = _RasterizeGaussians.apply(self.raster_settings, *tensors)
            self.last_depth, self.last_alpha, self.last_num_keys = depth, alpha, 0
            return image, radii, depth
        inputs = pipeline.FrameInputs(self.raster_settings, means3D, opacities=opacities, shs=shs,
                                      colors_precomp=colors_precomp, scales=scales, rotations=rotations,
                                      cov3D_precomp=cov3D_precomp, count=count)
        out = pipeline.render(inputs)
        self.last_depth, self.last_alpha, self.last_num_keys = out.depth, out.alpha, out.num_keys
        return out.image, out.radii, out.depth
