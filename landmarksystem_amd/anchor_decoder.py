"""MFMA-backed anchor decoder with the reference's module interface.

`FusedAnchorDecoder` takes the constructor keywords of the reference's
`AnchorDecoder` / `FusedAnchorDecoder` (landmark/nerf_components/
model_components/fields/anchor_decoder.py:49-61) and has the same `forward`
signature (:108-120) and 7-tuple result (:239-242), so the reference's
component-swap map (`kernel_fusion_components_convert_map["AnchorDecoder"]`,
landmark/nerf_components/components_convertor/convert_maps.py:40-47) can point
at it.  Parameters keep the reference's names (`mlp_opacity.0.weight`, ...,
cf. tests/test_module/test_util/test_gs_ckpt_transform.py:24-28) so its
checkpoints load unchanged.

Forward only, eval mode; the configuration the Scaffold-GS model builds
(no feature bank, no level / appearance inputs).  All arithmetic runs in the
HIP kernels behind `gs355_decode_count` / `gs355_decode_emit`.
"""
import ctypes as C
from typing import Optional

import torch
from torch import nn

from . import _lib


def _f32c(t: torch.Tensor, device) -> torch.Tensor:
    t = t.detach()
    if t.device != device:
        t = t.to(device)
    if t.dtype != torch.float32:
        t = t.float()
    return t.contiguous()


class FusedAnchorDecoder(nn.Module):
    def __init__(self, use_feat_bank: bool, add_opacity_dist: bool, add_color_dist: bool, add_cov_dist: bool,
                 view_dim: int, feat_dim: int, n_offsets: int, appearance_dim: int = 0, add_level: bool = False,
                 dist2level: str = None):
        super().__init__()
        if use_feat_bank or add_level or appearance_dim > 0:
            raise NotImplementedError(
                "FusedAnchorDecoder covers the Scaffold-GS configuration (use_feat_bank=False, add_level=False, "
                "appearance_dim=0)")
        if view_dim != 3 or feat_dim != 32 or not 1 <= n_offsets <= 10:
            raise NotImplementedError("FusedAnchorDecoder needs view_dim=3, feat_dim=32 and 1..10 offsets")
        self.use_feat_bank, self.add_level, self.dist2level = use_feat_bank, add_level, dist2level
        self.add_opacity_dist, self.add_color_dist, self.add_cov_dist = add_opacity_dist, add_color_dist, add_cov_dist
        self.view_dim, self.feat_dim, self.n_offsets, self.appearance_dim = view_dim, feat_dim, n_offsets, appearance_dim

        def head(with_dist: bool, outputs: int, last: Optional[nn.Module]):
            layers = [nn.Linear(feat_dim + view_dim + (1 if with_dist else 0), feat_dim), nn.ReLU(True),
                      nn.Linear(feat_dim, outputs)]
            if last is not None:
                layers.append(last)
            return nn.Sequential(*layers)

        self.mlp_opacity = head(add_opacity_dist, n_offsets, nn.Tanh())
        self.mlp_cov = head(add_cov_dist, 7 * n_offsets, None)
        self.mlp_color = head(add_color_dist, 3 * n_offsets, nn.Sigmoid())
        self._scratch: Optional[torch.Tensor] = None

    def _decoder_struct(self, device):
        keep = []
        d = _lib.Decoder()
        d.feat_dim, d.n_offsets = self.feat_dim, self.n_offsets
        for j, mlp in enumerate((self.mlp_opacity, self.mlp_cov, self.mlp_color)):
            w0, b0, w1, b1 = (_f32c(t, device) for t in (mlp[0].weight, mlp[0].bias, mlp[2].weight, mlp[2].bias))
            keep += [w0, b0, w1, b1]
            d.in_dim[j] = w0.shape[1]
            d.w0[j], d.b0[j], d.w1[j], d.b1[j] = w0.data_ptr(), b0.data_ptr(), w1.data_ptr(), b1.data_ptr()
        return d, keep

    @torch.no_grad()
    def forward(self, camera_center, anchor, anchor_feat, offset, scaling, visible_mask=None, level=None,
                prog_ratio=None, transition_mask=None, appearance_code=None):
        """Returns (xyz[G,3], color[G,3], opacity[G,1], scaling[G,3], rot[G,4], None, None): the neural Gaussians of
        the visible anchors whose decoded opacity is positive, in boolean-mask order."""
        if not anchor.is_cuda:
            raise ValueError("anchor must be a tensor on the GPU (the decoder has no CPU path)")
        dev = anchor.device
        A = anchor.shape[0]
        if visible_mask is None:
            visible_mask = torch.ones(A, dtype=torch.bool, device=dev)
        vis = visible_mask.to(device=dev, dtype=torch.bool).contiguous()
        an = _lib.Anchors()
        tensors = dict(anchor=_f32c(anchor, dev), feat=_f32c(anchor_feat, dev), offset=_f32c(offset, dev),
                       scaling=_f32c(scaling, dev), campos=_f32c(camera_center, dev))
        an.A = A
        an.anchor, an.feat = tensors["anchor"].data_ptr(), tensors["feat"].data_ptr()
        an.offset, an.scaling = tensors["offset"].data_ptr(), tensors["scaling"].data_ptr()
        an.visible_mask, an.campos = vis.data_ptr(), tensors["campos"].data_ptr()
        dec, keep = self._decoder_struct(dev)
        lib = _lib.load()
        stream = torch.cuda.current_stream(dev).cuda_stream

        need = C.c_size_t()
        _lib.check(lib.gs355_decode_scratch_bytes(A, C.byref(need)))
        if self._scratch is None or self._scratch.device != dev or self._scratch.numel() < need.value:
            self._scratch = torch.empty(need.value, dtype=torch.uint8, device=dev)
        counts = torch.empty(max(A, 1), dtype=torch.int32, device=dev)
        offsets = torch.empty(max(A, 1), dtype=torch.int32, device=dev)
        _lib.check(lib.gs355_decode_count(C.byref(dec), C.byref(an), counts.data_ptr(), offsets.data_ptr(),
                                          self._scratch.data_ptr(), self._scratch.numel(), stream))
        # the output shapes depend on the data: one read-back, as the reference's boolean-mask indexing does
        G = int((offsets[A - 1] + counts[A - 1]).item()) if A > 0 else 0
        out = dict(xyz=torch.empty((G, 3), device=dev), color=torch.empty((G, 3), device=dev),
                   opacity=torch.empty((G, 1), device=dev), scaling=torch.empty((G, 3), device=dev),
                   rot=torch.empty((G, 4), device=dev))
        if G > 0:
            o = _lib.Decoded()
            o.xyz, o.color, o.opacity = out["xyz"].data_ptr(), out["color"].data_ptr(), out["opacity"].data_ptr()
            o.scaling, o.rot = out["scaling"].data_ptr(), out["rot"].data_ptr()
            _lib.check(lib.gs355_decode_emit(C.byref(dec), C.byref(an), offsets.data_ptr(), G, C.byref(o), stream))
        del keep
        return out["xyz"], out["color"], out["opacity"], out["scaling"], out["rot"], None, None
