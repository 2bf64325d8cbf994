"""MFMA-backed anchor decoder with the reference's module interface.

`FusedAnchorDecoder` takes the constructor keywords of the reference's
`AnchorDecoder` / `FusedAnchorDecoder` (landmark/nerf_components/
model_components/fields/anchor_decoder.py:49-61) and has the same `forward`
signature (:108-120) and 7-tuple result (:239-242), so the reference's
component-swap map (`kernel_fusion_components_convert_map["AnchorDecoder"]`,
landmark/nerf_components/components_convertor/convert_maps.py:40-47) can point
at it.  Parameters keep the reference's names (`mlp_opacity.0.weight`, ...,
`mlp_feature_bank.0.weight`, cf. tests/test_module/test_util/
test_gs_ckpt_transform.py:24-28) so its checkpoints load unchanged.

Supported: the feature bank (`use_feat_bank`), the level input (`add_level`)
and the training-mode by-products (`neural_opacity`, `mask`); not the
appearance embedding (`appearance_dim > 0`: the reference's own branch
concatenates a 1-D integer tensor to the 2-D input, anchor_decoder.py:204-211,
and cannot run as written).  Without gradients all arithmetic runs in the HIP
kernels behind `gs355_decode`: one call enqueues the whole decode and the
number of Gaussians stays on the device; `forward` waits for that one number
(the reference's boolean-mask indexing synchronises at the same place) only to
give its results their exact shapes, `decode_on_device` never waits.

In training mode with gradients enabled and something to differentiate (a
parameter or an input that requires grad: the training loops of benchmarks/nerf/scaffold_gs and
octree_gs), `forward` evaluates the module's own statements
(anchor_decoder.py:147-242) as torch operations on the GPU, so autograd
reaches the MLPs, the features, the offsets and the scales -- as in the
reference, whose fused decoder is an inference component and whose training
runs the torch module.  The rasterizer behind it differentiates in HIP.
"""
import ctypes as C
from collections import OrderedDict
from typing import NamedTuple, Optional

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


class DeviceDecode(NamedTuple):
    """Result of `decode_on_device`: tensors with room for A * n_offsets Gaussians, of which the first `count[0]`
    are valid.  `counts` (int32[2], on the device) holds the number of Gaussians and of visible anchors."""
    xyz: torch.Tensor
    color: torch.Tensor
    opacity: torch.Tensor
    scaling: torch.Tensor
    rot: torch.Tensor
    counts: torch.Tensor
    neural_opacity: Optional[torch.Tensor]
    mask: Optional[torch.Tensor]

    @property
    def count(self) -> torch.Tensor:  # int32[1]: what the rasterizer takes as its device-side Gaussian count
        return self.counts[0:1]


class _TallLinear(torch.autograd.Function):
    """y = x W^T + b for x with hundreds of thousands of rows and a few dozen columns (one row per visible anchor).
    Forward and dL/dx are what nn.Linear computes; dL/dW = dy^T x has its long dimension inside the product, which
    the library's matrix multiply runs on a handful of workgroups (0.8 ms each at 500k anchors): here the rows are
    cut into slabs, one small product per slab in a batched multiply, and the slabs' products are added."""

    SLAB = 4096

    @staticmethod
    def forward(ctx, x, weight, bias):
        x = x.contiguous()
        ctx.save_for_backward(x, weight)
        return torch.addmm(bias, x, weight.t())

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dy = dy.contiguous()
        dx = dy @ weight if ctx.needs_input_grad[0] else None
        dw = None
        if ctx.needs_input_grad[1]:
            rows, slab = x.shape[0], _TallLinear.SLAB
            whole = rows // slab * slab
            dw = torch.zeros_like(weight)
            if whole:
                dw += torch.bmm(dy[:whole].view(-1, slab, dy.shape[1]).transpose(1, 2),
                                x[:whole].view(-1, slab, x.shape[1])).sum(dim=0)
            if whole < rows:
                dw += dy[whole:].t() @ x[whole:]
        db = dy.sum(dim=0) if ctx.needs_input_grad[2] else None
        return dx, dw, db


def _mlp(seq, x):
    """The Sequential `seq` (Linear, ReLU, Linear[, activation]) with its Linear layers through _TallLinear."""
    for layer in seq:
        x = _TallLinear.apply(x, layer.weight, layer.bias) if isinstance(layer, torch.nn.Linear) else layer(x)
    return x


class FusedAnchorDecoder(nn.Module):
    def __init__(self, use_feat_bank: bool, add_opacity_dist: bool, add_color_dist: bool, add_cov_dist: bool,
                 view_dim: int, feat_dim: int, n_offsets: int, appearance_dim: int = 0, add_level: bool = False,
                 dist2level: str = None):
        super().__init__()
        if appearance_dim > 0:
            raise NotImplementedError("FusedAnchorDecoder does not take an appearance embedding (appearance_dim=0 only)")
        if view_dim != 3 or feat_dim != 32 or not 1 <= n_offsets <= 10:
            raise NotImplementedError("FusedAnchorDecoder needs view_dim=3, feat_dim=32 and 1..10 offsets")
        self.use_feat_bank, self.add_level, self.dist2level = use_feat_bank, add_level, dist2level
        self.add_opacity_dist, self.add_color_dist, self.add_cov_dist = add_opacity_dist, add_color_dist, add_cov_dist
        self.view_dim, self.feat_dim, self.n_offsets, self.appearance_dim = view_dim, feat_dim, n_offsets, appearance_dim
        level_dim = 1 if add_level else 0

        def head(with_dist: bool, outputs: int, last: Optional[nn.Module]):
            layers = [nn.Linear(feat_dim + view_dim + (1 if with_dist else 0) + level_dim, feat_dim), nn.ReLU(True),
                      nn.Linear(feat_dim, outputs)]
            if last is not None:
                layers.append(last)
            return nn.Sequential(*layers)

        if use_feat_bank:
            self.mlp_feature_bank = nn.Sequential(nn.Linear(view_dim + level_dim, feat_dim), nn.ReLU(True),
                                                  nn.Linear(feat_dim, 3), nn.Softmax(dim=1))
        self.mlp_opacity = head(add_opacity_dist, n_offsets, nn.Tanh())
        self.mlp_cov = head(add_cov_dist, 7 * n_offsets, None)
        self.mlp_color = head(add_color_dist, 3 * n_offsets, nn.Sigmoid())
        # device buffers the decoder keeps between calls, one set per stream that decoded recently (frames of
        # different streams may be in flight together): "workspace" of gs355_decode, "block" of reused outputs
        self._per_stream = OrderedDict()
        self._marshalled = None  # (key, gs355_decoder struct, the tensors it points at)
        self._host_count: Optional[torch.Tensor] = None  # pinned landing place of the device-side counts
        self._feat_checked = None  # (identity of the last feature tensor, whether fp16 holds it exactly)

    # ---- marshalling -----------------------------------------------------------------------------------------
    def _decoder_struct(self, device):
        """The gs355_decoder record of the current parameters, rebuilt only when a parameter was replaced, moved or
        modified in place (tensor identity and version), not per call."""
        key = (device,) + tuple((id(p), p._version, p.data_ptr()) for p in self._parameter_list())
        if self._marshalled is not None and self._marshalled[0] == key:
            return self._marshalled[1]
        keep = []
        d = _lib.Decoder()
        d.feat_dim, d.n_offsets = self.feat_dim, self.n_offsets
        fp16_exact = True  # weights that fp16 cannot hold (fp32-trained checkpoints) go in as hi + lo fp16 pairs
        for j, mlp in enumerate((self.mlp_opacity, self.mlp_cov, self.mlp_color)):
            w0, b0, w1, b1 = (_f32c(t, device) for t in (mlp[0].weight, mlp[0].bias, mlp[2].weight, mlp[2].bias))
            keep += [w0, b0, w1, b1]
            fp16_exact = fp16_exact and all(bool(torch.equal(w.half().float(), w)) for w in (w0, w1))
            d.in_dim[j] = w0.shape[1]
            d.w0[j], d.b0[j], d.w1[j], d.b1[j] = w0.data_ptr(), b0.data_ptr(), w1.data_ptr(), b1.data_ptr()
        d.fp32_weights = 0 if fp16_exact else 1
        d.add_level = 1 if self.add_level else 0
        d.bank_in_dim = 0
        if self.use_feat_bank:
            mlp = self.mlp_feature_bank
            w0, b0, w1, b1 = (_f32c(t, device) for t in (mlp[0].weight, mlp[0].bias, mlp[2].weight, mlp[2].bias))
            keep += [w0, b0, w1, b1]
            d.bank_in_dim = w0.shape[1]
            d.bank_w0, d.bank_b0, d.bank_w1, d.bank_b1 = w0.data_ptr(), b0.data_ptr(), w1.data_ptr(), b1.data_ptr()
        self._marshalled = (key, d, keep)
        return d

    def _parameter_list(self):
        mlps = [self.mlp_opacity, self.mlp_cov, self.mlp_color] + ([self.mlp_feature_bank] if self.use_feat_bank else [])
        return [t for m in mlps for t in (m[0].weight, m[0].bias, m[2].weight, m[2].bias)]

    def _check_level(self, level, A):
        """The reference's behaviour for the level input (anchor_decoder.py:157-186): with add_level and a level
        tensor every head is fed [feat | view | level]; anything else does not match the widths the heads were
        built with and fails in its first matrix product."""
        if not self.add_level:
            return None
        if level is None:
            raise RuntimeError("add_level=True but no level was given: the heads are %d wide, the input without a level "
                               "is not (the reference fails in mlp_opacity with a shape mismatch)"
                               % self.mlp_opacity[0].weight.shape[1])
        for name, flag in (("opacity", self.add_opacity_dist), ("cov", self.add_cov_dist), ("color", self.add_color_dist)):
            if flag:
                raise RuntimeError("add_level=True with add_%s_dist=True: the reference feeds [feat | view | level] "
                                   "(36 columns, anchor_decoder.py:181-182) into a head built 37 wide and fails with a "
                                   "shape mismatch" % name)
        if level.numel() != A:
            raise ValueError("level has %d elements, expected %d" % (level.numel(), A))
        return level.reshape(-1)

    # ---- decode ----------------------------------------------------------------------------------------------
    def _marshal(self, camera_center, anchor, anchor_feat, offset, scaling, visible_mask, level):
        if not anchor.is_cuda:
            raise ValueError("anchor must be a tensor on the GPU (the decoder has no CPU path)")
        dev = anchor.device
        A = anchor.shape[0]
        level = self._check_level(level, A)
        if visible_mask is None:
            visible_mask = torch.ones(A, dtype=torch.bool, device=dev)
        vis = visible_mask.to(device=dev, dtype=torch.bool).contiguous()
        an = _lib.Anchors()
        tensors = [_f32c(anchor, dev), _f32c(anchor_feat, dev), _f32c(offset, dev), _f32c(scaling, dev),
                   _f32c(camera_center, dev), vis]
        an.A = A
        an.anchor, an.feat, an.offset, an.scaling = (t.data_ptr() for t in tensors[:4])
        an.campos, an.visible_mask = tensors[4].data_ptr(), vis.data_ptr()
        if level is not None:
            tensors.append(_f32c(level, dev))
            an.level = tensors[-1].data_ptr()
        dec = self._decoder_struct(dev)
        # features that fp16 cannot hold exactly (fp32-trained checkpoints) go through the matrix cores as hi + lo
        # pairs; checked once per feature tensor, not per frame
        feat_key = (id(anchor_feat), anchor_feat._version, anchor_feat.data_ptr(), tuple(anchor_feat.shape))
        if self._feat_checked is None or self._feat_checked[0] != feat_key:
            f32 = tensors[1]
            self._feat_checked = (feat_key, bool(torch.equal(f32.half().float(), f32)))
        dec.fp32_features = 0 if self._feat_checked[1] else 1
        need = C.c_size_t()
        _lib.check(_lib.load().gs355_decode_workspace_bytes(A, self.n_offsets, 1 if self.use_feat_bank else 0,
                                                            C.byref(need)))
        kept = self._kept(dev)
        if kept.get("workspace") is None or kept["workspace"].numel() < need.value:
            kept["workspace"] = torch.empty(max(need.value, 256), dtype=torch.uint8, device=dev)
        return dev, A, dec, an, tensors

    def _kept(self, dev):
        key = (dev, torch.cuda.current_stream(dev).cuda_stream)
        kept = self._per_stream.get(key)
        if kept is None:
            kept = self._per_stream[key] = {}
            while len(self._per_stream) > 4:
                self._per_stream.popitem(last=False)
        else:
            self._per_stream.move_to_end(key)
        return kept

    def _run(self, dec, an, capacity, o, phases, dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        ws = self._kept(dev)["workspace"]
        _lib.check(_lib.load().gs355_decode(C.byref(dec), C.byref(an), int(capacity), C.byref(o), ws.data_ptr(),
                                            ws.numel(), int(phases), stream))

    @torch.no_grad()
    def decode_on_device(self, camera_center, anchor, anchor_feat, offset, scaling, visible_mask=None, level=None,
                         want_training_outputs: bool = False, reuse_buffers: bool = False) -> DeviceDecode:
        """The whole decode enqueued on the current stream, nothing read back.  Outputs have room for
        A * n_offsets Gaussians; `counts` says how many are valid.  `reuse_buffers`: the outputs live in one block
        the decoder keeps and overwrites at its next call (a render loop that consumes them at once pays no
        per-frame allocation of the capacity-sized block)."""
        dev, A, dec, an, tensors = self._marshal(camera_center, anchor, anchor_feat, offset, scaling, visible_mask, level)
        n = self.n_offsets
        cap = A * n
        # one block for the five outputs (14 floats per Gaussian) and the two counters, carved into views
        kept = self._kept(dev)
        if reuse_buffers and kept.get("block") is not None and kept["block"][0] == cap:
            res = kept["block"][1]
        else:
            block = torch.empty(cap * 14 + 2, dtype=torch.float32, device=dev)
            cut = lambda first, width: block[first * cap:(first + width) * cap].view(cap, width)  # noqa: E731
            res = DeviceDecode(cut(0, 3), cut(3, 3), cut(6, 1), cut(7, 3), cut(10, 4), block[cap * 14:].view(torch.int32),
                               None, None)
            kept["block"] = (cap, res) if reuse_buffers else None
        if want_training_outputs:
            res = res._replace(neural_opacity=torch.empty((cap, 1), dtype=torch.float32, device=dev),
                               mask=torch.empty(cap, dtype=torch.bool, device=dev))
        o = _lib.Decoded()
        if cap > 0:
            o.xyz, o.color, o.opacity = res.xyz.data_ptr(), res.color.data_ptr(), res.opacity.data_ptr()
            o.scaling, o.rot = res.scaling.data_ptr(), res.rot.data_ptr()
            if want_training_outputs:
                o.neural_opacity, o.mask = res.neural_opacity.data_ptr(), res.mask.data_ptr()
        o.count, o.num_visible = res.counts.data_ptr(), res.counts.data_ptr() + 4
        self._run(dec, an, cap, o, _lib.DECODE_ALL, dev)
        del tensors  # torch's allocator keeps their memory alive for the work already enqueued on this stream
        return res

    def read_counts(self, res):
        """(G, visible anchors) from the device-side counters of a decode: one 8-byte copy to pinned memory, waited
        for.  `res`: a `decode_on_device` result or the int32[2] counter tensor."""
        counts = res.counts if isinstance(res, DeviceDecode) else res
        if self._host_count is None:
            self._host_count = torch.zeros(2, dtype=torch.int32, pin_memory=True)
        self._host_count.copy_(counts, non_blocking=True)
        torch.cuda.current_stream(counts.device).synchronize()
        return int(self._host_count[0]), int(self._host_count[1])

    def forward(self, camera_center, anchor, anchor_feat, offset, scaling, visible_mask=None, level=None,
                prog_ratio=None, transition_mask=None, appearance_code=None):
        if self.dist2level == "progressive" and prog_ratio is not None and transition_mask is not None:
            raise NotImplementedError("progressive level-of-detail opacity scaling is not part of this decoder")
        if self.training and torch.is_grad_enabled() and (any(p.requires_grad for p in self.parameters()) or any(
                torch.is_tensor(t) and t.requires_grad for t in (anchor, anchor_feat, offset, scaling))):
            return self._forward_differentiable(camera_center, anchor, anchor_feat, offset, scaling, visible_mask, level)
        with torch.no_grad():
            return self._forward_kernels(camera_center, anchor, anchor_feat, offset, scaling, visible_mask, level)

    def _forward_differentiable(self, camera_center, anchor, anchor_feat, offset, scaling, visible_mask, level):
        """The statements of the reference module (anchor_decoder.py:147-242) as torch operations, for autograd:
        same 7-tuple, the training by-products always present."""
        level = self._check_level(level, anchor.shape[0])
        if visible_mask is None:
            visible_mask = torch.ones(anchor.shape[0], dtype=torch.bool, device=anchor.device)
        # Rows are selected with index_select over index lists computed once, not with boolean masks: the results
        # are the same tensors, but the backward of a boolean-mask index is a sorting index_put (3.7 ms per step at
        # 500k anchors), that of index_select an index_add.
        rows = visible_mask.nonzero(as_tuple=True)[0]
        a, feat, off, sc = (t.index_select(0, rows) for t in (anchor, anchor_feat, offset, scaling))
        view = a - camera_center.to(a.device)
        dist = view.norm(dim=1, keepdim=True)
        view = view / dist
        lvl = level.reshape(-1, 1).index_select(0, rows).to(feat.dtype) if level is not None else None
        if self.use_feat_bank:
            w = _mlp(self.mlp_feature_bank, view if lvl is None else torch.cat([view, lvl], dim=1))  # softmax inside
            feat = feat[:, ::4].repeat(1, 4) * w[:, 0:1] + feat[:, ::2].repeat(1, 2) * w[:, 1:2] + feat * w[:, 2:3]
        if lvl is not None:  # (:181-182: both inputs become [feat | view | level])
            with_dist = without = torch.cat([feat, view, lvl], dim=1)
        else:
            with_dist, without = torch.cat([feat, view, dist], dim=1), torch.cat([feat, view], dim=1)
        n = self.n_offsets
        neural_opacity = _mlp(self.mlp_opacity, with_dist if self.add_opacity_dist else without).reshape(-1, 1)
        mask = (neural_opacity > 0.0).view(-1)
        kept = mask.nonzero(as_tuple=True)[0]
        owner = torch.div(kept, n, rounding_mode="floor")  # anchor (among the visible ones) of each kept offset
        color = _mlp(self.mlp_color, with_dist if self.add_color_dist else without).reshape(-1, 3).index_select(0, kept)
        cov = _mlp(self.mlp_cov, with_dist if self.add_cov_dist else without).reshape(-1, 7).index_select(0, kept)
        sc_kept = sc.index_select(0, owner)
        scaling_out = sc_kept[:, 3:6] * torch.sigmoid(cov[:, 0:3])
        rot = torch.nn.functional.normalize(cov[:, 3:7])
        xyz = a.index_select(0, owner) + off.reshape(-1, 3).index_select(0, kept) * sc_kept[:, 0:3]
        return xyz, color, neural_opacity.index_select(0, kept), scaling_out, rot, neural_opacity, mask

    def _forward_kernels(self, camera_center, anchor, anchor_feat, offset, scaling, visible_mask=None, level=None):
        """Returns (xyz[G,3], color[G,3], opacity[G,1], scaling[G,3], rot[G,4], neural_opacity, mask): the neural
        Gaussians of the visible anchors whose decoded opacity is positive, in boolean-mask order; in training mode
        also the opacity of every offset of the visible anchors ([A_vis * n, 1]) and the mask over them, else None.

        The output shapes depend on the data, so the count phase runs first and its two counters are read back
        (the reference's boolean-mask indexing synchronises at the same place); the emit phase then writes into
        tensors of exactly that size."""
        dev, A, dec, an, tensors = self._marshal(camera_center, anchor, anchor_feat, offset, scaling, visible_mask, level)
        # the two counters go straight into pinned host memory (which the GPU addresses like its own): no copy is
        # enqueued, the host waits for the count phase and reads them
        if self._host_count is None:
            self._host_count = torch.zeros(2, dtype=torch.int32, pin_memory=True)
        counts = self._host_count
        o = _lib.Decoded()
        o.count, o.num_visible = counts.data_ptr(), counts.data_ptr() + 4
        self._run(dec, an, 0, o, _lib.DECODE_COUNT, dev)
        torch.cuda.current_stream(dev).synchronize()
        G, a_vis = int(counts[0]), int(counts[1])
        f = lambda *shape: torch.empty(shape, dtype=torch.float32, device=dev)  # noqa: E731
        out = (f(G, 3), f(G, 3), f(G, 1), f(G, 3), f(G, 4))
        extra = (None, None)
        if self.training:
            extra = (f(a_vis * self.n_offsets, 1), torch.empty(a_vis * self.n_offsets, dtype=torch.bool, device=dev))
        if G > 0 or (self.training and a_vis > 0):
            if G > 0:
                o.xyz, o.color, o.opacity, o.scaling, o.rot = (t.data_ptr() for t in out)
            if self.training and a_vis > 0:
                o.neural_opacity, o.mask = extra[0].data_ptr(), extra[1].data_ptr()
            o.count = o.num_visible = None
            self._run(dec, an, G, o, _lib.DECODE_EMIT, dev)
        del tensors
        return out + extra
