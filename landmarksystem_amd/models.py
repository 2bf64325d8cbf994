"""Host-side counterparts of the reference's three Gaussian-splatting models:
the callers on either side of the rasterizer.

  GaussianModel  benchmarks/nerf/origin_gs/gs_model.py:112-228 (forward), :280-331 (prefilter_voxel);
                 parameter getters / activations: landmark/nerf_components/model_components/fields/
                 encodings/gaussian_encoding.py:89-97, 745-853
  ScaffoldGS     benchmarks/nerf/scaffold_gs/gs_model.py:162-238, :385-436;
                 getters: .../encodings/scaffoldgs_encoding.py:701-775
  OctreeGS       benchmarks/nerf/octree_gs/gs_model.py:228-325, :445-497;
                 level-of-detail mask: .../encodings/octreegs_encoding.py:238-294

They keep the reference's call sequence (visibility prefilter -> optional
anchor decode -> settings record re-assigned on the renderer -> rasterize),
its eval-mode gather of the visible Gaussians and its `act_cache` behaviour,
and its parameter names so checkpoints map one to one.  The vanilla model also
runs in training mode (every Gaussian rendered, differentiable through the
rasterizer's backward pass, `viewspace_points` kept for densification); the
Scaffold- / Octree-GS models are forward-only.  Optimizers and densification
are not part of this package; checkpoint I/O lives in `checkpoints.py`.
Activations and gathers are a handful of torch elementwise calls, as in the
reference; everything per-Gaussian and per-pixel runs in the HIP library.
"""
import math
from typing import Optional

import torch
from torch import nn

from . import pipeline
from .anchor_decoder import FusedAnchorDecoder
from .rasterizer import GaussianRasterizationSettings, GaussianRasterizer


def _settings(camera, bg, scaling_modifier, sh_degree):
    return GaussianRasterizationSettings(
        image_height=int(camera.height), image_width=int(camera.width),
        tanfovx=math.tan(camera.FovX * 0.5), tanfovy=math.tan(camera.FovY * 0.5), bg=bg,
        scale_modifier=scaling_modifier, viewmatrix=camera.world_view_transform,
        projmatrix=camera.full_proj_transform, sh_degree=sh_degree, campos=camera.camera_center,
        prefiltered=False, debug=False,
    )


def _cfg(config, name, default):
    """Field `name` of a config object (attribute- or key-addressable), else `default`."""
    if isinstance(config, dict):
        return config.get(name, default)
    return getattr(config, name, default)


def _split_prefix(state_dict, prefix):
    """Pop the entries under `prefix` (base_model.py:363-368)."""
    picked = {}
    for key in list(state_dict.keys()):
        if key.startswith(prefix):
            picked[key[len(prefix):]] = state_dict.pop(key)
    if not picked:
        print("WRANING: could not found any key start with %s in provided state_dict" % prefix)
    return picked


def morton_order(xyz: torch.Tensor) -> torch.Tensor:
    """Permutation that sorts points along a 3-D Morton (Z-order) curve: 21 bits per axis on a common scale,
    interleaved x, y, z from the most significant bit down.

    Storing a scene in this order is a load-time choice.  The rasterizer orders by depth, so a frame changes only
    where two Gaussians of exactly equal fp32 depth share a pixel (ties blend in index order, as in the reference;
    the effect is of the order of 1e-4 on isolated pixels).  It makes the memory traffic of a frame coherent:
    Gaussians that land in the same screen tile sit near each other in memory, so culled stretches skip whole
    wavefronts, bucket writes of one slice of the scene fall into few tiles, and the blend's record gathers hit
    lines that are already in cache."""
    p = xyz.detach().double()
    lo = p.min(dim=0).values
    span = float((p.max(dim=0).values - lo).max())
    q = ((p - lo) / (span if span > 0 else 1.0) * float((1 << 21) - 1)).long().clamp_(0, (1 << 21) - 1)

    def spread(v):  # 21 bits -> every third bit of 63
        v = (v | (v << 32)) & 0x1F00000000FFFF
        v = (v | (v << 16)) & 0x1F0000FF0000FF
        v = (v | (v << 8)) & 0x100F00F00F00F00F
        v = (v | (v << 4)) & 0x10C30C30C30C30C3
        v = (v | (v << 2)) & 0x1249249249249249
        return v

    code = (spread(q[:, 0]) << 2) | (spread(q[:, 1]) << 1) | spread(q[:, 2])
    return torch.sort(code, stable=True).indices


def _placeholder_renderer(bg):
    # the reference builds its renderer once with empty placeholders (origin_gs/gs_model.py:82-97)
    return GaussianRasterizer(raster_settings=GaussianRasterizationSettings(
        image_height=0, image_width=0, tanfovx=0, tanfovy=0, bg=bg, scale_modifier=0, viewmatrix=torch.Tensor([]),
        projmatrix=torch.Tensor([]), sh_degree=0, campos=torch.Tensor([]), prefiltered=False, debug=False))


class GaussianModel(nn.Module):
    """Vanilla 3DGS: raw parameters with exp / sigmoid / normalize activations."""

    def __init__(self, xyz=None, features_dc=None, features_rest=None, scaling=None, rotation=None, opacity=None,
                 sh_degree: int = 3, white_bkgd: bool = False, act_cache: bool = False,
                 compute_cov3D_python: bool = False, convert_SHs_python: bool = False, fuse_prefilter: bool = True,
                 config=None, scene_manager=None):
        super().__init__()
        if xyz is not None and not torch.is_tensor(xyz):  # the reference's signature: (config, scene_manager)
            config, xyz = xyz, None
        if config is not None:  # empty model, filled by load_from_state_dict (origin_gs/gs_model.py:62-79)
            sh_degree = _cfg(config, "sh_degree", sh_degree)
            white_bkgd, act_cache = _cfg(config, "white_bkgd", white_bkgd), _cfg(config, "act_cache", act_cache)
            compute_cov3D_python = _cfg(config, "compute_cov3D_python", compute_cov3D_python)
            convert_SHs_python = _cfg(config, "convert_SHs_python", convert_SHs_python)
            fuse_prefilter = _cfg(config, "fuse_prefilter", fuse_prefilter)
        if xyz is None:
            e = torch.empty
            xyz, features_dc, features_rest = e(0, 3), e(0, 1, 3), e(0, (sh_degree + 1) ** 2 - 1, 3)
            scaling, rotation, opacity = e(0, 3), e(0, 4), e(0, 1)
        self.config, self.scene_manager = config, scene_manager
        # fuse_prefilter (default): render all Gaussians in one pass instead of "visibility prefilter, gather the
        # survivors, render them" (False = the reference's sequence, call by call).  The prefilter applies the same cull / radius / tile-rectangle tests as the rasterizer's own
        # preprocess with the same camera, and a boolean-mask gather keeps relative order, so image, visibility_filter
        # and radii come out identical; the second per-Gaussian pass and the 236 B/Gaussian gathers disappear.
        self.fuse_prefilter = fuse_prefilter
        self._xyz = nn.Parameter(xyz, requires_grad=False)  # [P,3]
        self._features_dc = nn.Parameter(features_dc, requires_grad=False)  # [P,1,3]
        self._features_rest = nn.Parameter(features_rest, requires_grad=False)  # [P,(deg+1)^2-1,3]
        self._scaling = nn.Parameter(scaling, requires_grad=False)  # [P,3] log
        self._rotation = nn.Parameter(rotation, requires_grad=False)  # [P,4]
        self._opacity = nn.Parameter(opacity, requires_grad=False)  # [P,1] logit
        self.active_sh_degree = self.max_sh_degree = sh_degree
        self.act_cache = act_cache
        self.compute_cov3D_python, self.convert_SHs_python = compute_cov3D_python, convert_SHs_python
        self.register_buffer("background", torch.tensor([1.0, 1.0, 1.0] if white_bkgd else [0.0, 0.0, 0.0]))
        self.renderer = _placeholder_renderer(self.background)
        self._cache = {}
        self._radii = self._visibility_filter = self._radii_all = None
        self.viewspace_points = None  # training: zero tensor whose .grad receives the screen-space gradient

    # `visibility_filter` (bool[P]) and `radii` (int32 of the visible Gaussians) are by-products the reference
    # leaves on the model for its training loop.  The fused single-pass frame derives them from the rasterizer's
    # radii only when they are read, so a render loop that never looks at them pays nothing (the boolean-mask
    # gather waits for the device).
    @property
    def visibility_filter(self):
        if self._visibility_filter is None and self._radii_all is not None:
            self._visibility_filter = self._radii_all > 0
        return self._visibility_filter

    @visibility_filter.setter
    def visibility_filter(self, value):
        self._visibility_filter = value

    @property
    def radii(self):
        if self._radii is None and self._radii_all is not None:
            self._radii = self._radii_all[self.visibility_filter]
        return self._radii

    @radii.setter
    def radii(self, value):
        self._radii = value

    @classmethod
    def from_activated(cls, means3D, scales, rotations, opacities, shs, **kw):
        """Build from activated values (e.g. a synthetic scene) by inverting the activations."""
        eps = 1e-7
        op = opacities.clamp(eps, 1 - eps)
        return cls(means3D, shs[:, :1].contiguous(), shs[:, 1:].contiguous(), torch.log(scales), rotations,
                   torch.log(op / (1 - op)), **kw)

    @classmethod
    def from_cache(cls, xyz, features, scaling, rotation, opacity, **kw):
        """Build from stored activated values (the `cache_*` checkpoint schema, gaussian_encoding.py:226-266):
        the raw parameters stay empty and the getters serve the cache, so the model is eval-only."""
        kw["act_cache"] = True
        empty = lambda *shape: torch.empty(*shape, device=xyz.device)  # noqa: E731
        m = cls(xyz, empty(0, 1, 3), empty(0, features.shape[1] - 1, 3), empty(0, 3), empty(0, 4), empty(0, 1), **kw)
        m._cache = {"features": features, "scaling": scaling, "rotation": rotation, "opacity": opacity}
        return m.eval()

    def get_state_dict_from_ckpt(self, file_path, map_location="cpu"):
        """PLY columns under `gaussian_encoding.` merged with `state_dict.th` (base_model.py:308-342)."""
        from . import checkpoints
        return checkpoints.merged_state_dict(file_path, "gaussian", map_location, max_sh_degree=self.max_sh_degree)

    def load_from_state_dict(self, state_dict, strict: bool = True):
        """base_model.py:344-372 + gaussian_encoding.py:273-338: raw parameters, or the activation cache."""
        gs = _split_prefix(dict(state_dict), "gaussian_encoding.")
        raw = ("_xyz", "_features_dc", "_features_rest", "_opacity", "_scaling", "_rotation")
        cache = ("_xyz", "_cache_features", "_cache_opacity", "_cache_scaling", "_cache_rotation")
        if "_opacity" in gs or "_features_dc" in gs:
            found = set(gs) & set(raw)
            if strict and len(found) != len(raw):
                raise ValueError("only found keys %s in state dict" % (found,))
            for name in found:
                setattr(self, name, nn.Parameter(gs[name].detach().to(self._xyz.device).float().contiguous(),
                                                 requires_grad=False))
            self._cache = {}
        elif set(gs) & set(cache[1:]):
            found = set(gs) & set(cache)
            if strict and len(found) != len(cache):
                raise ValueError("only found keys %s in state dict" % (found,))
            dev = self._xyz.device
            self._xyz = nn.Parameter(gs["_xyz"].detach().to(dev).float().contiguous(), requires_grad=False)
            self.act_cache = True
            self._cache = {k[len("_cache_"):]: gs[k].detach().to(dev).float().contiguous() for k in found if k != "_xyz"}
        elif strict:
            raise ValueError("not found any param keys in state dict, state dict keys: %s" % (list(gs),))
        self.active_sh_degree = self.max_sh_degree

    def _apply(self, fn, *args, **kwargs):
        out = super()._apply(fn, *args, **kwargs)  # .to()/.cuda(): the activation cache follows the parameters
        self._cache = {k: fn(v) for k, v in self._cache.items()}
        return out

    def _cached(self, name, fn):
        if self.act_cache and not self.training:
            if name not in self._cache:
                self._cache[name] = fn()
            return self._cache[name]
        return fn()

    @property
    def get_xyz(self):
        return self._xyz

    @property
    def get_scaling(self):
        return self._cached("scaling", lambda: torch.exp(self._scaling))

    @property
    def get_rotation(self):
        return self._cached("rotation", lambda: torch.nn.functional.normalize(self._rotation))

    @property
    def get_opacity(self):
        return self._cached("opacity", lambda: torch.sigmoid(self._opacity))

    @property
    def get_features(self):
        return self._cached("features", lambda: torch.cat((self._features_dc, self._features_rest), dim=1))

    def get_covariance(self, scaling_modifier=1.0):
        # L = R diag(mod * s), Sigma = L L^T packed (xx,xy,xz,yy,yz,zz): gaussian_encoding.py:22-38
        s = scaling_modifier * self.get_scaling
        q = self.get_rotation
        r, x, y, z = q[:, 0], q[:, 1], q[:, 2], q[:, 3]
        R = torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y),
                         2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x),
                         2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], dim=1).view(-1, 3, 3)
        L = R * s[:, None, :]
        S = L @ L.transpose(1, 2)
        return torch.stack([S[:, 0, 0], S[:, 0, 1], S[:, 0, 2], S[:, 1, 1], S[:, 1, 2], S[:, 2, 2]], dim=1)

    def prefilter_voxel(self, viewpoint_camera, scaling_modifier=1.0):
        rasterizer = GaussianRasterizer(raster_settings=_settings(viewpoint_camera, self.background,
                                                                  scaling_modifier, 1))
        scales = rotations = cov3D_precomp = None
        if self.compute_cov3D_python:
            cov3D_precomp = self.get_covariance(scaling_modifier)
        else:
            scales, rotations = self.get_scaling, self.get_rotation
        radii_pure = rasterizer.visible_filter(means3D=self.get_xyz, scales=None if scales is None else scales[:, :3],
                                               rotations=rotations, cov3D_precomp=cov3D_precomp)
        return radii_pure > 0

    def forward(self, viewpoint_camera, scaling_modifier=1.0, override_color=None, render_exclude_filter=None):
        """origin_gs/gs_model.py:112-228.  Under torch.no_grad() (the inference engine) this is the plain frame.
        In training mode with gradients enabled every Gaussian is rendered (no gather), the frame is
        differentiable with respect to the parameters, and `viewspace_points` receives the screen-space gradient
        that the reference's densification reads (:129-139, :225-236)."""
        viewpoint_camera = viewpoint_camera.to(self._xyz.device)
        fused = (self.fuse_prefilter and render_exclude_filter is None
                 and scaling_modifier == 1.0)  # the reference's prefilter always uses scale modifier 1
        if not fused:
            voxel_visible_mask = self.prefilter_voxel(viewpoint_camera)
            if render_exclude_filter is not None:
                voxel_visible_mask = voxel_visible_mask & render_exclude_filter
        self.renderer.raster_settings = _settings(viewpoint_camera, self.background, scaling_modifier,
                                                  self.active_sh_degree)
        means3D, opacity = self.get_xyz, self.get_opacity
        scales = rotations = cov3D_precomp = shs = colors_precomp = None
        if self.compute_cov3D_python:
            cov3D_precomp = self.get_covariance(scaling_modifier)
        else:
            scales, rotations = self.get_scaling, self.get_rotation
        if override_color is not None:
            colors_precomp = override_color
        else:
            # convert_SHs_python only chooses where SH -> RGB is evaluated in the reference (torch statements,
            # origin_gs/gs_model.py:184-193, or its rasterizer); here the preprocess kernel evaluates the same
            # expression, clamp_min(eval_sh + 0.5, 0), for either setting
            shs = self.get_features
        screenspace_points = None
        if self.training and torch.is_grad_enabled():
            screenspace_points = torch.zeros_like(means3D, requires_grad=True) + 0
            screenspace_points.retain_grad()
        self.viewspace_points = screenspace_points
        if fused:
            rendered_image, radii, _ = self.renderer(
                means3D=means3D, means2D=screenspace_points, shs=shs, colors_precomp=colors_precomp, opacities=opacity,
                scales=scales, rotations=rotations, cov3D_precomp=cov3D_precomp)
            # eval: radii of the visible subset, as after the reference's gather; training: of all Gaussians
            self._radii_all, self._visibility_filter = radii, None
            self._radii = radii if self.training else None
            return rendered_image
        if not self.training:  # the reference renders only what its prefilter kept (origin_gs/gs_model.py:199-208)
            # (five boolean-index operations there; one pass over the tensors and one wait for the row count here)
            means3D, shs, colors_precomp, opacity, scales, rotations, cov3D_precomp = pipeline.gather_rows(
                voxel_visible_mask, [means3D, shs, colors_precomp, opacity, scales, rotations, cov3D_precomp])
        rendered_image, radii, _ = self.renderer(
            means3D=means3D, means2D=screenspace_points, shs=shs, colors_precomp=colors_precomp, opacities=opacity,
            scales=scales, rotations=rotations, cov3D_precomp=cov3D_precomp)
        self._radii_all, self.visibility_filter, self.radii = None, voxel_visible_mask, radii
        return rendered_image


class ScaffoldGS(nn.Module):
    """Scaffold-GS: anchors decoded into neural Gaussians per frame."""

    _ckpt_kind = "scaffold"
    _decoder_options = (("view_dim", 3),)

    def __init__(self, anchor=None, anchor_feat=None, offset=None, scaling=None, rotation=None, n_offsets: int = 10,
                 feat_dim: int = 32, add_opacity_dist: bool = True, add_cov_dist: bool = True,
                 add_color_dist: bool = True, white_bkgd: bool = False, act_cache: bool = False, opacity=None,
                 config=None, scene_manager=None, fuse_prefilter: bool = True, use_feat_bank: bool = False,
                 add_level: bool = False, appearance_dim: int = 0):
        super().__init__()
        # fuse_prefilter (default; False = the reference's sequence, call by call): the anchor-level prefilter (for Octree-GS including the level-of-detail mask, its gather
        # of the selected anchors and the scatter of the result) runs as one kernel over all anchors, and the
        # number of decoded Gaussians stays on the device: decode and rasterizer are enqueued back to back without
        # a read-back in between (`visibility_filter` reads it when asked for).  Same masks, except that an anchor
        # whose predicted level sits within rounding of a .5 boundary may fall on the other side (the
        # level-of-detail formula is evaluated in the kernel instead of by a chain of torch operations).
        self.fuse_prefilter = fuse_prefilter
        if anchor is not None and not torch.is_tensor(anchor):  # the reference's signature: (config, scene_manager)
            config, anchor = anchor, None
        if config is not None:  # empty model, filled by load_from_state_dict (scaffold_gs/gs_model.py:104-140)
            n_offsets, feat_dim = _cfg(config, "n_offsets", n_offsets), _cfg(config, "feat_dim", feat_dim)
            add_opacity_dist = _cfg(config, "add_opacity_dist", add_opacity_dist)
            add_cov_dist = _cfg(config, "add_cov_dist", add_cov_dist)
            add_color_dist = _cfg(config, "add_color_dist", add_color_dist)
            white_bkgd, act_cache = _cfg(config, "white_bkgd", white_bkgd), _cfg(config, "act_cache", act_cache)
            self.fuse_prefilter = _cfg(config, "fuse_prefilter", fuse_prefilter)
            use_feat_bank = _cfg(config, "use_feat_bank", use_feat_bank)
            # the options the reference's model hands to its AnchorDecoder: scaffold_gs/gs_model.py:126-134 passes
            # neither add_level nor appearance_dim (its config's add_level=True default never reaches the decoder);
            # octree_gs/gs_model.py:165-176 passes both
            if self._ckpt_kind == "octree":
                add_level = _cfg(config, "add_level", add_level)
                appearance_dim = _cfg(config, "appearance_dim", appearance_dim)
            for name, allowed in self._decoder_options:
                if _cfg(config, name, allowed) != allowed:
                    raise NotImplementedError("%s=%r: the fused anchor decode supports %s=%r only"
                                              % (name, _cfg(config, name, allowed), name, allowed))
        if anchor is None:
            e = torch.empty
            anchor, anchor_feat, offset = e(0, 3), e(0, feat_dim), e(0, n_offsets, 3)
            scaling, rotation = e(0, 6), e(0, 4)
        self.config, self.scene_manager = config, scene_manager
        # per-anchor opacity is carried by checkpoints but never read by the forward pass (scaffoldgs_encoding.py:88)
        self._opacity = nn.Parameter(torch.zeros(anchor.shape[0], 1, device=anchor.device) if opacity is None
                                     else opacity, requires_grad=False)  # [A,1] logit
        self._anchor = nn.Parameter(anchor, requires_grad=False)  # [A,3]
        self._anchor_feat = nn.Parameter(anchor_feat, requires_grad=False)  # [A,32]
        self._offset = nn.Parameter(offset, requires_grad=False)  # [A,n,3]
        self._scaling = nn.Parameter(scaling, requires_grad=False)  # [A,6] log
        self._rotation = nn.Parameter(rotation, requires_grad=False)  # [A,4]
        self.act_cache = act_cache
        self.anchor_decoder = FusedAnchorDecoder(
            use_feat_bank=use_feat_bank, add_opacity_dist=add_opacity_dist, add_color_dist=add_color_dist,
            add_cov_dist=add_cov_dist, view_dim=3, feat_dim=feat_dim, n_offsets=n_offsets,
            appearance_dim=appearance_dim, add_level=add_level)
        self.register_buffer("background", torch.tensor([1.0, 1.0, 1.0] if white_bkgd else [0.0, 0.0, 0.0]))
        self.renderer = _placeholder_renderer(self.background)
        self._cache = {}
        self._visibility_filter = self.voxel_visible_mask = None
        self._pending = None  # (decode result, radii sized for its capacity) of a frame whose count is still on the device

    # `visibility_filter` (bool[G] over the decoded Gaussians) is a by-product the reference leaves on the model.
    # A frame rendered without reading the number of Gaussians back derives it when it is asked for.
    @property
    def visibility_filter(self):
        if self._visibility_filter is None and self._pending is not None:
            res, radii = self._pending
            G, _ = self.anchor_decoder.read_counts(res)
            self._visibility_filter = radii[:G] > 0
            self._pending = None
        return self._visibility_filter

    @visibility_filter.setter
    def visibility_filter(self, value):
        self._visibility_filter, self._pending = value, None

    @classmethod
    def from_scene(cls, scene, **kw):
        m = cls(scene.anchor, scene.anchor_feat, scene.offset, torch.log(scene.scaling), scene.rotation,
                n_offsets=scene.n_offsets, **kw)
        state = {}
        for name, head in (("mlp_opacity", "opacity"), ("mlp_cov", "cov"), ("mlp_color", "color")):
            w0, b0, w1, b1 = scene.mlp[head]
            state.update({name + ".0.weight": w0, name + ".0.bias": b0, name + ".2.weight": w1, name + ".2.bias": b1})
        m.anchor_decoder.load_state_dict(state)
        return m

    def _cached(self, name, fn):
        if self.act_cache and not self.training:
            if name not in self._cache:
                self._cache[name] = fn()
            return self._cache[name]
        return fn()

    @property
    def get_anchor(self):
        return self._anchor

    @property
    def get_anchor_feat(self):
        return self._anchor_feat

    @property
    def get_offset(self):
        return self._offset

    @property
    def get_scaling(self):
        return self._cached("scaling", lambda: torch.exp(self._scaling))

    @property
    def get_rotation(self):
        return self._cached("rotation", lambda: torch.nn.functional.normalize(self._rotation))

    def get_state_dict_from_ckpt(self, file_path, map_location="cpu"):
        """PLY columns under `gaussian_encoding.` merged with `state_dict.th` (base_model.py:308-342)."""
        from . import checkpoints
        return checkpoints.merged_state_dict(file_path, self._ckpt_kind, map_location)

    _encoding_keys = ("_anchor_feat", "_offset", "_anchor", "_opacity", "_scaling", "_rotation")

    def load_from_state_dict(self, state_dict, strict: bool = True):
        """base_model.py:344-372 + scaffoldgs_encoding.py:236-281; the rest (`anchor_decoder.*`) loads as an
        ordinary module state dict."""
        state_dict = dict(state_dict)
        gs = _split_prefix(state_dict, "gaussian_encoding.")
        found = set(gs) & set(self._encoding_keys)
        if strict and len(found) != len(self._encoding_keys):
            raise ValueError("only found keys %s in state dict" % (found,))
        dev = self._anchor.device
        for name in found:
            value = gs[name].detach().to(dev)
            if isinstance(getattr(self, name), nn.Parameter):
                setattr(self, name, nn.Parameter(value.float().contiguous(), requires_grad=False))
            else:
                self._load_buffer(name, value)
        self._cache = {}
        decoder = _split_prefix(state_dict, "anchor_decoder.") if any(
            k.startswith("anchor_decoder.") for k in state_dict) else {}
        if decoder or strict:
            self.anchor_decoder.load_state_dict(decoder, strict=strict)
        if strict and state_dict:
            raise ValueError("unexpected keys in state dict: %s" % (sorted(state_dict),))

    def _load_buffer(self, name, value):
        raise KeyError(name)

    def _anchor_subset(self):
        return None  # Scaffold-GS filters all anchors

    def _lod(self, viewpoint_camera):
        return None  # Scaffold-GS has no level of detail

    def prefilter_voxel(self, viewpoint_camera, scaling_modifier=1.0):
        if self.fuse_prefilter and not self.training:
            from . import pipeline
            visible, mask = pipeline.anchor_filter(
                _settings(viewpoint_camera, self.background, scaling_modifier, 1), self.get_anchor, self.get_scaling,
                self.get_rotation, self._lod(viewpoint_camera))
            if mask is not None:
                self._anchor_mask = mask
            return visible
        rasterizer = GaussianRasterizer(raster_settings=_settings(viewpoint_camera, self.background,
                                                                  scaling_modifier, 1))
        subset = self._anchor_subset()
        means3D, scales, rotations = self.get_anchor, self.get_scaling, self.get_rotation
        if subset is not None:
            means3D, scales, rotations = means3D[subset], scales[subset], rotations[subset]
        radii_pure = rasterizer.visible_filter(means3D=means3D, scales=scales[:, :3], rotations=rotations,
                                               cov3D_precomp=None)
        if subset is None:
            return radii_pure > 0
        visible_mask = subset.clone()
        visible_mask[subset] = radii_pure > 0
        return visible_mask

    def _before_prefilter(self, viewpoint_camera):
        pass

    def _decoder_level(self):
        return None  # Scaffold-GS anchors carry no level

    def forward(self, viewpoint_camera, scaling_modifier=1.0, retain_grad=False, render_exclude_filter=None):
        """scaffold_gs/gs_model.py:162-238 (octree_gs/gs_model.py:228-325).  In eval mode: the frame.  In training
        mode: `(rendered_image, scaling)` as the reference returns them, with `viewspace_points`,
        `offset_selection_mask` and `opacity` left on the model for its densification; with gradients enabled the
        pair is differentiable with respect to the anchors' parameters and the decoder's MLPs (under torch.no_grad()
        the same values come from the kernels)."""
        if self.training:
            return self._forward_training(viewpoint_camera, scaling_modifier, retain_grad, render_exclude_filter)
        with torch.no_grad():
            return self._forward_frame(viewpoint_camera, scaling_modifier, render_exclude_filter)

    def _forward_training(self, viewpoint_camera, scaling_modifier, retain_grad, render_exclude_filter):
        viewpoint_camera = viewpoint_camera.to(self._anchor.device)
        with torch.no_grad():  # (the visibility tests are not differentiated)
            self._before_prefilter(viewpoint_camera)
            voxel_visible_mask = self.prefilter_voxel(viewpoint_camera)
            if render_exclude_filter is not None:
                voxel_visible_mask = voxel_visible_mask & render_exclude_filter
        xyz, color, opacity, scaling, rot, neural_opacity, mask = self.anchor_decoder(
            camera_center=viewpoint_camera.camera_center, anchor=self.get_anchor, anchor_feat=self.get_anchor_feat,
            offset=self.get_offset, scaling=self.get_scaling, visible_mask=voxel_visible_mask,
            level=self._decoder_level())
        screenspace_points = torch.zeros_like(xyz, requires_grad=True) + 0
        if retain_grad and screenspace_points.requires_grad:  # (not under torch.no_grad())
            screenspace_points.retain_grad()
        self.renderer.raster_settings = _settings(viewpoint_camera, self.background, scaling_modifier, 1)
        rendered_image, radii, _ = self.renderer(
            means3D=xyz, means2D=screenspace_points, shs=None, colors_precomp=color, opacities=opacity, scales=scaling,
            rotations=rot, cov3D_precomp=None)
        self.viewspace_points = screenspace_points
        self.visibility_filter, self.voxel_visible_mask = radii > 0, voxel_visible_mask
        self.offset_selection_mask, self.opacity = mask, neural_opacity
        return rendered_image, scaling

    def _forward_frame(self, viewpoint_camera, scaling_modifier=1.0, render_exclude_filter=None):
        viewpoint_camera = viewpoint_camera.to(self._anchor.device)
        self._before_prefilter(viewpoint_camera)
        voxel_visible_mask = self.prefilter_voxel(viewpoint_camera)
        if render_exclude_filter is not None:
            voxel_visible_mask = voxel_visible_mask & render_exclude_filter
        self.renderer.raster_settings = _settings(viewpoint_camera, self.background, scaling_modifier, 1)
        decode = dict(camera_center=viewpoint_camera.camera_center, anchor=self.get_anchor,
                      anchor_feat=self.get_anchor_feat, offset=self.get_offset, scaling=self.get_scaling,
                      visible_mask=voxel_visible_mask, level=self._decoder_level())
        if self.fuse_prefilter and not self.training:
            # nothing is read back: the decode leaves the number of Gaussians on the device, the rasterizer takes it
            # from there and works over tensors sized for the most the anchors can emit
            res = self.anchor_decoder.decode_on_device(**decode, reuse_buffers=True)
            rendered_image, radii, _ = self.renderer(
                means3D=res.xyz, means2D=None, shs=None, colors_precomp=res.color, opacities=res.opacity,
                scales=res.scaling, rotations=res.rot, cov3D_precomp=None, count=res.count)
            self._visibility_filter, self._pending = None, (res, radii)
            self.voxel_visible_mask = voxel_visible_mask
            return rendered_image
        xyz, color, opacity, scaling, rot, _, _ = self.anchor_decoder(**decode)
        rendered_image, radii, _ = self.renderer(
            means3D=xyz, means2D=None, shs=None, colors_precomp=color, opacities=opacity, scales=scaling,
            rotations=rot, cov3D_precomp=None)
        self.visibility_filter, self.voxel_visible_mask = radii > 0, voxel_visible_mask
        return rendered_image


class OctreeGS(ScaffoldGS):
    """Octree-GS: Scaffold-GS plus a per-frame level-of-detail mask over the anchors."""

    _ckpt_kind = "octree"
    _decoder_options = ScaffoldGS._decoder_options + (("appearance_dim", 0),)
    _encoding_keys = ScaffoldGS._encoding_keys + ("_level", "_extra_level")

    def __init__(self, anchor=None, anchor_feat=None, offset=None, scaling=None, rotation=None, level=None,
                 voxel_size: float = 0.0, standard_dist: float = 1.0, fork: int = 2, extra_level=None,
                 enable_lod: bool = True, dist2level: str = "round", config=None, scene_manager=None, **kw):
        if anchor is not None and not torch.is_tensor(anchor):  # the reference's signature: (config, scene_manager)
            config, anchor = anchor, None
        if config is not None:  # octree_gs/gs_model.py:139-177; Octree-GS defaults to no distance inputs (:44-46)
            fork, dist2level = _cfg(config, "fork", fork), _cfg(config, "dist2level", dist2level)
            enable_lod = _cfg(config, "enable_lod", enable_lod)
            for name in ("add_opacity_dist", "add_cov_dist", "add_color_dist"):
                kw.setdefault(name, _cfg(config, name, False))
        super().__init__(anchor, anchor_feat, offset, scaling, rotation, config=config, scene_manager=scene_manager,
                         **kw)
        if level is None:
            level = torch.zeros(self._anchor.shape[0])
        anchor = self._anchor
        if dist2level not in ("floor", "round", "ceil"):
            raise NotImplementedError("dist2level=%r (the progressive mode is dead code from the reference's model, "
                                      "octree_gs/gs_model.py:247)" % dist2level)
        self.register_buffer("_level", level.reshape(-1, 1).float())  # [A,1]
        self.register_buffer("_extra_level", torch.zeros(anchor.shape[0]) if extra_level is None else extra_level)
        self.voxel_size, self.standard_dist, self.fork = float(voxel_size), float(standard_dist), int(fork)
        self.enable_lod, self.dist2level = enable_lod, dist2level
        self._anchor_mask: Optional[torch.Tensor] = None
        self._level_span = None  # (the level tensor it was computed from, max level - min level)

    def set_anchor_mask(self, cam_center, iteration, resolution_scale):
        """octreegs_encoding.py:238-264 in eval mode: keep anchors whose level does not exceed the level
        predicted from their distance to the camera."""
        if not self.enable_lod:
            self._anchor_mask = torch.ones(self._level.shape[0], dtype=torch.bool, device=self._level.device)
            return
        anchor_pos = self._anchor + (self.voxel_size / 2) / (float(self.fork) ** self._level)
        dist = torch.sqrt(torch.sum((anchor_pos - cam_center.to(anchor_pos.device)) ** 2, dim=1)) * resolution_scale
        pred_level = torch.log2(self.standard_dist / dist) / math.log2(self.fork) + self._extra_level
        max_level = self._level_span_value()
        if self.dist2level == "floor":
            int_level = torch.floor(pred_level).int()
        elif self.dist2level == "round":
            int_level = torch.round(pred_level).int()
        else:
            int_level = torch.ceil(pred_level).int()
        int_level = torch.clamp(int_level, min=0, max=max_level)
        self._anchor_mask = self._level.squeeze(dim=1) <= int_level

    def get_state_dict_from_ckpt(self, file_path, map_location="cpu"):
        """As Scaffold-GS; reading the PLY also sets `voxel_size` and `standard_dist` from its `info` column
        (octreegs_encoding.py:323-324)."""
        from . import checkpoints
        _, self.voxel_size, self.standard_dist = checkpoints.octree_state_dict(file_path, "cpu")
        return super().get_state_dict_from_ckpt(file_path, map_location)

    def _load_buffer(self, name, value):
        if name == "_level":
            self._level = value.reshape(-1, 1).float()
        elif name == "_extra_level":
            self._extra_level = value.reshape(-1).float()
        else:
            raise KeyError(name)

    def forward(self, viewpoint_camera, scaling_modifier=1.0, retain_grad=False, render_exclude_filter=None,
                ape_code=-1):
        # ape_code selects an appearance embedding in the reference (octree_gs/gs_model.py:254-260); without
        # appearance inputs (appearance_dim = 0, all this decode supports) it has no effect
        return super().forward(viewpoint_camera, scaling_modifier, retain_grad, render_exclude_filter)

    def _decoder_level(self):
        # the reference's model hands its decoder `gaussian_encoding.levels`, the number of levels
        # (octree_gs/gs_model.py:268), where the decoder indexes a per-anchor tensor (anchor_decoder.py:157-158): with
        # add_level that call cannot run.  The per-anchor level is what the decoder's input is built for.
        return self._level if self.anchor_decoder.add_level else None

    def _level_span_value(self) -> int:
        if self._level_span is None or self._level_span[0] is not self._level:
            # the span of the levels is a constant of the loaded model: read it back once, not per frame
            self._level_span = (self._level, int((torch.max(self._level) - torch.min(self._level)).item()))
        return self._level_span[1]

    def _lod(self, viewpoint_camera):
        if not self.enable_lod:
            return None
        return dict(level=self._level.reshape(-1), extra_level=self._extra_level, voxel_size=self.voxel_size,
                    standard_dist=self.standard_dist, fork=self.fork,
                    resolution_scale=float(getattr(viewpoint_camera, "resolution_scale", 1.0)),
                    rounding=self.dist2level, max_level=self._level_span_value())

    def _before_prefilter(self, viewpoint_camera):
        if self.fuse_prefilter and not self.training:
            if not self.enable_lod:
                self._anchor_mask = torch.ones(self._level.shape[0], dtype=torch.bool, device=self._level.device)
            return  # the fused prefilter computes the level-of-detail mask itself
        if not self.training:
            self.set_anchor_mask(viewpoint_camera.camera_center, -1, viewpoint_camera.resolution_scale)

    def _anchor_subset(self):
        return self._anchor_mask
