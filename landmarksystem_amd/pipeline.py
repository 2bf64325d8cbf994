"""Host driver of the rasterizer stages: marshals torch tensors into the C ABI
(include/gs355.h), owns the grow-only device workspace and handles the one
data-dependent size of a frame, the number of (tile, Gaussian) keys.

PyTorch is used for device memory and streams only; every computation is a
HIP kernel behind `gs355_run` / `gs355_visible_filter`.
"""
import ctypes as C
import math
from collections import OrderedDict
from typing import Dict, Optional, Tuple

import torch

from . import _lib

_KEY_HEADROOM = 1.25  # capacity = keys needed by the last frame that overflowed x this


def _dev_f32(t: Optional[torch.Tensor], device: torch.device, name: str, shape=None) -> Optional[torch.Tensor]:
    """Contiguous fp32 tensor on `device` (callers pass slices such as
    `scales[:, :3]`, and per-frame matrices may still live on the host)."""
    if t is None:
        return None
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor, got %r" % (name, type(t)))
    t = t.detach()
    if t.device != device:
        t = t.to(device)
    if t.dtype != torch.float32:
        t = t.float()
    if shape is not None:
        if t.numel() != math.prod(shape):
            raise ValueError("%s has %d elements, expected shape %s" % (name, t.numel(), tuple(shape)))
    return t.contiguous()


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None or t.numel() == 0 else t.data_ptr()


class Workspace:
    """Grow-only device buffer plus the key-capacity estimate for one device.

    The library never allocates device memory: this is the caller-owned
    workspace of the C ABI.  Work using one Workspace must stay on one stream
    at a time."""

    def __init__(self, device: torch.device):
        self.device = device
        self.buffer: Optional[torch.Tensor] = None
        self.key_capacity = 0
        self.header_host = torch.zeros(8, dtype=torch.int64, pin_memory=True)
        self.header_event = torch.cuda.Event()
        self.frames = 0
        self.overflows = 0
        self.sort_mispredictions = 0  # frames with buckets in a sorter size class that was expected empty
        self.last_num_keys = 0  # of the latest frame rendered over this workspace
        self.sort_class_idle = [0, 0, 0]  # consecutive frames that left each larger sorter size class empty
        self.sort_class_wait = [4, 4, 4]  # ... and how many of them it takes before the class's launch is left out

    def ensure(self, P: int, n_cap: int, width: int, height: int) -> "_lib.Layout":
        layout = _lib.workspace_layout(P, n_cap, width, height)
        if self.buffer is None or self.buffer.numel() < layout.total_bytes:
            self.buffer = None  # release before growing
            self.buffer = torch.empty(int(layout.total_bytes * 1.1) + 4096, dtype=torch.uint8, device=self.device)
        return layout

    def view(self, layout: "_lib.Layout", name: str, P: int, n_keys: int, tiles: int) -> torch.Tensor:
        """Typed view of one workspace array (for tests and diagnostics)."""
        buf = self.buffer

        def take(off, nbytes, dtype):
            return buf[off:off + nbytes].view(dtype)

        if name == "header":
            return take(layout.header, 64, torch.int64)
        if name == "records":
            return take(layout.records, P * 48, torch.float32).view(P, 12)
        if name == "tiles_touched":
            return take(layout.tiles_touched, P * 4, torch.int32)
        if name == "offsets":
            return take(layout.offsets, P * 4, torch.int32)
        if name in ("keys", "sorted_keys"):
            which = layout.unsorted_buffer if name == "keys" else layout.sorted_buffer
            return take(layout.keys[which], n_keys * 8, torch.int64)
        if name in ("values", "sorted_values"):
            which = layout.unsorted_buffer if name == "values" else layout.sorted_buffer
            return take(layout.values[which], n_keys * 4, torch.int32)
        if name == "ranges":
            return take(layout.ranges, tiles * 8, torch.int32).view(tiles, 2)
        raise KeyError(name)


# One workspace per (device, stream) that rendered recently: frames on different streams may be in flight together
# and must not share buffers.  Least recently used entries beyond _MAX_WORKSPACES are dropped (their device memory
# goes back to torch's allocator, which orders its reuse after the work already enqueued on that stream).
_MAX_WORKSPACES = 8
_workspaces: "OrderedDict[Tuple[int, int], Workspace]" = OrderedDict()


def _workspace_key(device: torch.device, stream=None) -> Tuple[int, int]:
    stream = stream if stream is not None else torch.cuda.current_stream(device)
    return (device.index if device.index is not None else torch.cuda.current_device(), stream.cuda_stream)


def default_workspace(device: torch.device) -> Workspace:
    key = _workspace_key(device)
    ws = _workspaces.get(key)
    if ws is None:
        ws = _workspaces[key] = Workspace(device)
        while len(_workspaces) > _MAX_WORKSPACES:
            _workspaces.popitem(last=False)
    else:
        _workspaces.move_to_end(key)
    return ws


def release_workspace(device: torch.device, stream=None) -> None:
    """Drop the workspace of `stream` (default: the current stream) on `device`, e.g. when a temporary stream
    retires.  Frames already enqueued keep their memory until they have run."""
    _workspaces.pop(_workspace_key(device, stream), None)


class FrameInputs:
    """The tensors of one rasterizer call, validated and marshalled."""

    def __init__(self, settings, means3D, opacities=None, shs=None, colors_precomp=None, scales=None, rotations=None,
                 cov3D_precomp=None, need_colour: bool = True, count: Optional[torch.Tensor] = None):
        """`count`: optional one-element int32 tensor on the device holding the number of Gaussians (the anchor
        decode leaves it there); the tensors are then sized for a capacity and only the first `count` rows are
        rendered, without the host ever reading the number."""
        if need_colour:
            if (shs is None and colors_precomp is None) or (shs is not None and colors_precomp is not None):
                raise Exception("Please provide excatly one of either SHs or precomputed colors!")
        if ((scales is None or rotations is None) and cov3D_precomp is None) or (
            (scales is not None or rotations is not None) and cov3D_precomp is not None
        ):
            raise Exception("Please provide exactly one of either scale/rotation pair or precomputed 3D covariance!")
        if not isinstance(means3D, torch.Tensor) or not means3D.is_cuda:
            raise ValueError("means3D must be a tensor on the GPU (the rasterizer has no CPU path)")
        dev = means3D.device
        self.device = dev
        P = means3D.shape[0]
        self.P = P

        self.means3D = _dev_f32(means3D, dev, "means3D", (P, 3))
        self.opacities = _dev_f32(opacities, dev, "opacities", (P,)) if need_colour else None
        self.shs = _dev_f32(shs, dev, "shs") if need_colour else None
        self.colors_precomp = _dev_f32(colors_precomp, dev, "colors_precomp", (P, 3)) if need_colour else None
        self.scales = _dev_f32(scales, dev, "scales", (P, 3))
        self.rotations = _dev_f32(rotations, dev, "rotations", (P, 4))
        self.cov3D_precomp = _dev_f32(cov3D_precomp, dev, "cov3D_precomp", (P, 6))
        sh_coeffs = 0
        if self.shs is not None:
            if self.shs.dim() != 3 or self.shs.shape[0] != P or self.shs.shape[2] != 3:
                raise ValueError("shs must have shape [P, M, 3], got %s" % (tuple(self.shs.shape),))
            sh_coeffs = int(self.shs.shape[1])

        s = settings
        self.width, self.height = int(s.image_width), int(s.image_height)
        self.viewmatrix = _dev_f32(s.viewmatrix, dev, "viewmatrix", (16,))
        self.projmatrix = _dev_f32(s.projmatrix, dev, "projmatrix", (16,))
        self.campos = _dev_f32(s.campos, dev, "campos", (3,))
        self.bg = _dev_f32(s.bg, dev, "bg", (3,))

        f = _lib.Frame()
        f.image_width, f.image_height = self.width, self.height
        f.tanfovx, f.tanfovy = float(s.tanfovx), float(s.tanfovy)
        f.scale_modifier = float(s.scale_modifier)
        f.sh_degree, f.sh_coeffs = int(s.sh_degree), sh_coeffs
        f.viewmatrix, f.projmatrix = _ptr(self.viewmatrix), _ptr(self.projmatrix)
        f.campos, f.bg = _ptr(self.campos), _ptr(self.bg)
        self.frame = f

        g = _lib.Gaussians()
        g.P = P
        g.means3D, g.shs, g.colors_precomp = _ptr(self.means3D), _ptr(self.shs), _ptr(self.colors_precomp)
        g.opacities, g.scales, g.rotations = _ptr(self.opacities), _ptr(self.scales), _ptr(self.rotations)
        g.cov3D_precomp = _ptr(self.cov3D_precomp)
        self.count = None
        if count is not None:
            if not (isinstance(count, torch.Tensor) and count.device == dev and count.numel() == 1
                    and count.dtype in (torch.int32, torch.uint32)):
                raise ValueError("count must be a one-element int32 tensor on the Gaussians' device")
            self.count = count
            g.P_device = count.data_ptr()
        self.gaussians = g

    @property
    def tiles(self) -> int:
        return ((self.width + 15) // 16) * ((self.height + 15) // 16)


def visible_filter(inputs: FrameInputs) -> torch.Tensor:
    """radii int32[P] of the cull / covariance / radius / tile-rectangle test."""
    radii = torch.empty(inputs.P, dtype=torch.int32, device=inputs.device)
    stream = torch.cuda.current_stream(inputs.device).cuda_stream
    _lib.check(_lib.load().gs355_visible_filter(C.byref(inputs.frame), C.byref(inputs.gaussians), _ptr(radii), stream))
    return radii


def anchor_filter(settings, anchors: torch.Tensor, scaling: torch.Tensor, rotations: torch.Tensor, lod=None):
    """The anchor-level visibility prefilter of Scaffold-GS / Octree-GS in one kernel (gs355_anchor_filter).

    `scaling` is the models' f32[A,6] (or [A,3]); its first three columns are read in place.  `lod`: None, or a dict
    with level f32[A], extra_level f32[A], voxel_size, standard_dist, fork, resolution_scale, rounding
    ("floor" | "round" | "ceil") and max_level.  Returns (visible bool[A], lod_mask bool[A] or None)."""
    if not anchors.is_cuda:
        raise ValueError("anchors must be a tensor on the GPU (the rasterizer has no CPU path)")
    dev, A = anchors.device, anchors.shape[0]
    means = _dev_f32(anchors, dev, "anchors", (A, 3))
    sc = _dev_f32(scaling, dev, "scaling")
    if sc.dim() != 2 or sc.shape[0] != A or sc.shape[1] < 3:
        raise ValueError("scaling must have shape [A, >=3], got %s" % (tuple(sc.shape),))
    rot = _dev_f32(rotations, dev, "rotations", (A, 4))
    keep = [_dev_f32(settings.viewmatrix, dev, "viewmatrix", (16,)), _dev_f32(settings.projmatrix, dev, "projmatrix", (16,)),
            _dev_f32(settings.campos, dev, "campos", (3,))]
    f = _lib.Frame()
    f.image_width, f.image_height = int(settings.image_width), int(settings.image_height)
    f.tanfovx, f.tanfovy, f.scale_modifier = float(settings.tanfovx), float(settings.tanfovy), float(settings.scale_modifier)
    f.viewmatrix, f.projmatrix, f.campos = keep[0].data_ptr(), keep[1].data_ptr(), keep[2].data_ptr()
    g = _lib.Gaussians()
    g.P, g.means3D, g.scales, g.rotations = A, _ptr(means), _ptr(sc), _ptr(rot)
    visible = torch.empty(A, dtype=torch.bool, device=dev)
    mask, lod_c = None, None
    if lod is not None:
        level = _dev_f32(lod["level"], dev, "level", (A,))
        extra = _dev_f32(lod["extra_level"], dev, "extra_level", (A,))
        keep += [level, extra]
        mask = torch.empty(A, dtype=torch.bool, device=dev)
        lod_c = _lib.AnchorLod(_ptr(level), _ptr(extra), float(lod["voxel_size"]), float(lod["standard_dist"]),
                               float(lod["fork"]), float(lod["resolution_scale"]),
                               {"floor": 0, "round": 1, "ceil": 2}[lod["rounding"]], int(lod["max_level"]))
    stream = torch.cuda.current_stream(dev).cuda_stream
    _lib.check(_lib.load().gs355_anchor_filter(C.byref(f), C.byref(g), int(sc.shape[1]),
                                               C.byref(lod_c) if lod_c is not None else None, _ptr(mask),
                                               _ptr(visible), None, stream))
    del keep
    return visible, mask


def gather_rows(mask: torch.Tensor, tensors):
    """Rows of each tensor in `tensors` (None entries pass through) that the boolean `mask` selects, in order: what
    `t[mask]` gives for every one of them, in one pass over all of them (gs355_gather_rows) and with one wait for the
    number of selected rows instead of one per tensor.  Returns the list of gathered tensors."""
    dev, P = mask.device, mask.shape[0]
    if not mask.is_cuda or mask.dtype != torch.bool or mask.dim() != 1:
        raise ValueError("mask must be a one-dimensional bool tensor on the GPU")
    src = [None if t is None else _dev_f32(t, dev, "tensor") for t in tensors]
    given = [t for t in src if t is not None]
    if len(given) > _lib.GATHER_MAX_ARRAYS:
        raise ValueError("at most %d tensors per call" % _lib.GATHER_MAX_ARRAYS)
    for t in given:
        if t.shape[0] != P:
            raise ValueError("every tensor needs one row per mask entry (%d), got shape %s" % (P, tuple(t.shape)))
    dst = [torch.empty_like(t) for t in given]
    arrays = (_lib.GatherArray * max(1, len(given)))()
    for k, (a, b) in enumerate(zip(given, dst)):
        arrays[k].src, arrays[k].dst = a.data_ptr() if P else None, b.data_ptr() if P else None
        arrays[k].row_bytes = 4 * (a.numel() // P if P else 1)
    need = C.c_size_t(0)
    lib = _lib.load()
    _lib.check(lib.gs355_gather_scratch_bytes(P, C.byref(need)))
    scratch = torch.empty(need.value // 8 + 1, dtype=torch.int64, device=dev)
    count = torch.empty(1, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    _lib.check(lib.gs355_gather_rows(P, mask.contiguous().data_ptr() if P else None, len(given), arrays,
                                     count.data_ptr(), scratch.data_ptr(), scratch.numel() * 8, stream))
    n = int(count.item())  # the one wait: the caller's tensors are exactly sized, as after boolean indexing
    it = iter(dst)
    return [None if t is None else next(it)[:n] for t in src]


class FrameOutputs:
    def __init__(self, inputs: FrameInputs, want_depth: bool = True, want_alpha: bool = True):
        dev, H, W = inputs.device, inputs.height, inputs.width
        self.image = torch.empty((3, H, W), dtype=torch.float32, device=dev)
        self.depth = torch.empty((1, H, W), dtype=torch.float32, device=dev) if want_depth else None
        self.alpha = torch.empty((1, H, W), dtype=torch.float32, device=dev) if want_alpha else None
        self.radii = torch.empty(inputs.P, dtype=torch.int32, device=dev)
        o = _lib.Outputs()
        o.image, o.depth, o.alpha, o.radii = _ptr(self.image), _ptr(self.depth), _ptr(self.alpha), _ptr(self.radii)
        self.c = o
        self.num_keys = 0
        self.num_visible = 0
        self.key_capacity = 0  # the capacity the frame was finally rendered with (what a backward pass must pass)


def run_stages(inputs: FrameInputs, outputs: FrameOutputs, ws: Workspace, n_cap: int, stage_mask: int):
    """Enqueue the selected stages over `ws`; returns the layout used."""
    layout = ws.ensure(inputs.P, n_cap, inputs.width, inputs.height)
    stream = torch.cuda.current_stream(inputs.device).cuda_stream
    rc = _lib.load().gs355_run(C.byref(inputs.frame), C.byref(inputs.gaussians), ws.buffer.data_ptr(),
                               ws.buffer.numel(), int(n_cap), C.byref(outputs.c), int(stage_mask), stream)
    _lib.check(rc)
    return layout


def render(inputs: FrameInputs, want_depth: bool = True, want_alpha: bool = True,
           ws: Optional[Workspace] = None, classic: bool = False) -> FrameOutputs:
    """All stages of one frame (`classic`: through scan / duplicate / radix sort / ranges even where the
    tile-bucketed stages apply; same results).

    The key count is only known on the device after the scan.  The kernel that
    computes it also stores the header in pinned host memory; the remaining stages
    are enqueued against the current capacity without waiting, and the host then
    waits for that kernel only (the GPU keeps working on sort and blend).
    If the frame needed more keys than the capacity, it is redone once with
    the exact requirement plus headroom; capacity never shrinks."""
    ws = ws or default_workspace(inputs.device)
    out = FrameOutputs(inputs, want_depth, want_alpha)
    if ws.key_capacity == 0:
        ws.key_capacity = max(1 << 20, 4 * inputs.P)
    if not classic and inputs.tiles <= _lib.MAX_FAST_TILES and inputs.P <= _lib.MAX_FAST_GAUSSIANS:
        front = _lib.STAGE_PREPROCESS | _lib.STAGE_TILE_COUNT
        back = _lib.STAGE_TILE_SCATTER | _lib.STAGE_TILESORT | _lib.STAGE_BLEND
        # the scatter variant that suited the previous frame of this workspace (either is correct for any frame)
        back |= (_lib.STAGE_TILE_SCATTER_TWO_LEVEL if ws.last_num_keys >= _lib.TWO_LEVEL_MIN_KEYS
                 else _lib.STAGE_TILE_SCATTER_ONE_LEVEL)
        # no launch for a sorter size class that the last few frames left empty (a hint: the library sorts the
        # buckets of such a class all the same, but far slower than the launch costs, so a class that turns up
        # unexpectedly has to stay away four times as long before it is left out again)
        skipped = [c for c in range(3) if ws.sort_class_idle[c] >= ws.sort_class_wait[c]]
        for c in skipped:
            back |= _lib.STAGE_TILESORT_SKIP[c]
    else:  # beyond the bucketed stages' limits (images past 8K): classic duplicate / radix sort / ranges
        front = _lib.STAGE_PREPROCESS | _lib.STAGE_SCAN
        back = _lib.STAGE_DUPLICATE | _lib.STAGE_SORT | _lib.STAGE_RANGES | _lib.STAGE_BLEND
        skipped = []
    for attempt in range(3):
        n_cap = ws.key_capacity
        # the stage that produces the header also stores it in pinned host memory (no copy is enqueued)
        out.c.header_copy = ws.header_host.data_ptr()
        run_stages(inputs, out, ws, n_cap, front)
        out.c.header_copy = None
        ws.header_event.record(torch.cuda.current_stream(inputs.device))
        run_stages(inputs, out, ws, n_cap, back)
        ws.header_event.synchronize()
        total = int(ws.header_host[0])
        word1 = int(ws.header_host[1])
        overflow = (word1 >> 32) & 0xFFFFFFFF
        out.num_keys = ws.last_num_keys = total
        out.num_visible = int(ws.header_host[2]) & 0xFFFFFFFF
        ws.frames += 1
        word3 = int(ws.header_host[3])
        counts = ((int(ws.header_host[2]) >> 32) & 0xFFFFFFFF, word3 & 0xFFFFFFFF, (word3 >> 32) & 0xFFFFFFFF)
        for c in range(3):  # (0xFFFFFFFF: this path does not count the classes)
            ws.sort_class_idle[c] = ws.sort_class_idle[c] + 1 if counts[c] == 0 else 0
        wrong = [c for c in skipped if counts[c] != 0]
        if wrong and not overflow:
            ws.sort_mispredictions += 1  # (the frame is right all the same: the library sorts such buckets the slow way)
            for c in wrong:
                ws.sort_class_wait[c] = min(4 * ws.sort_class_wait[c], 4096)
        if not overflow:
            out.key_capacity = n_cap
            return out
        ws.overflows += 1
        for c in [c for c in skipped if counts[c] != 0]:
            back &= ~_lib.STAGE_TILESORT_SKIP[c]
            skipped.remove(c)
        ws.key_capacity = int(total * _KEY_HEADROOM) + 4096
    raise RuntimeError("key capacity still insufficient after regrowing (needed %d keys)" % out.num_keys)


GRAD_NAMES = ("means3D", "means2D", "shs", "colors_precomp", "opacities", "scales", "rotations", "cov3D_precomp")


def render_backward(inputs: FrameInputs, out: FrameOutputs, workspace: torch.Tensor, dL_dimage: torch.Tensor,
                    dL_ddepth: Optional[torch.Tensor] = None, dL_dalpha: Optional[torch.Tensor] = None,
                    want=GRAD_NAMES) -> Dict[str, torch.Tensor]:
    """Gradients of a frame rendered by `render` (gs355_render_backward).  `workspace` is the device buffer that
    frame was rendered in, untouched since; `out` its outputs.  Returns contiguous fp32 tensors for the names in
    `want` whose inputs were given: means3D [P,3], means2D [P,3], shs [P,M,3] / colors_precomp [P,3], opacities [P],
    scales [P,3], rotations [P,4] / cov3D_precomp [P,6]."""
    dev, P, H, W = inputs.device, inputs.P, inputs.height, inputs.width
    given = {"means3D": inputs.means3D, "means2D": inputs.means3D, "shs": inputs.shs,
             "colors_precomp": inputs.colors_precomp, "opacities": inputs.opacities, "scales": inputs.scales,
             "rotations": inputs.rotations, "cov3D_precomp": inputs.cov3D_precomp}
    grads = {n: torch.empty_like(given[n]) for n in want if given[n] is not None}
    gi = _dev_f32(dL_dimage, dev, "dL_dimage", (3, H, W))
    gd = _dev_f32(dL_ddepth, dev, "dL_ddepth", (H, W))
    ga = _dev_f32(dL_dalpha, dev, "dL_dalpha", (H, W))
    if gd is not None and out.depth is None or ga is not None and out.alpha is None:
        raise ValueError("a gradient arrives for an output the forward pass did not produce")
    b = _lib.BackwardInputs(_ptr(out.image), _ptr(out.depth), _ptr(out.alpha), _ptr(out.radii), _ptr(gi), _ptr(gd),
                            _ptr(ga))
    g = _lib.Gradients(*[_ptr(grads.get(n)) for n in GRAD_NAMES])
    need = C.c_size_t(0)
    _lib.check(_lib.load().gs355_backward_scratch_bytes(P, int(out.key_capacity), C.byref(need)))
    scratch = torch.empty(need.value // 4, dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    _lib.check(_lib.load().gs355_render_backward(C.byref(inputs.frame), C.byref(inputs.gaussians), workspace.data_ptr(),
                                                 workspace.numel(), int(out.key_capacity), C.byref(b),
                                                 scratch.data_ptr(), scratch.numel() * 4, C.byref(g), stream))
    return grads
