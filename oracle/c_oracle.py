"""numpy/ctypes front end of the C oracle (oracle/gs_oracle.c).

Test infrastructure only.  Everything takes and returns numpy arrays; no torch.
The stage functions mirror the pipeline of the rasterizer behind the
reference's `GaussianRasterizer.forward` (benchmarks/nerf/origin_gs/
gs_model.py:211-220): preprocess -> scan -> duplicate keys -> stable sort ->
tile ranges -> blend.
"""
import ctypes as C
import os
from dataclasses import dataclass, field

import numpy as np

from . import build as _build

_LIB = None


class _Frame(C.Structure):
    _fields_ = [
        ("image_width", C.c_int32),
        ("image_height", C.c_int32),
        ("tanfovx", C.c_float),
        ("tanfovy", C.c_float),
        ("scale_modifier", C.c_float),
        ("sh_degree", C.c_int32),
        ("sh_coeffs", C.c_int32),
        ("viewmatrix", C.c_float * 16),
        ("projmatrix", C.c_float * 16),
        ("campos", C.c_float * 3),
        ("bg", C.c_float * 3),
    ]


class _Gaussians(C.Structure):
    _fields_ = [("P", C.c_int32)] + [
        (n, C.c_void_p)
        for n in ("means3D", "shs", "colors_precomp", "opacities", "scales", "rotations", "cov3D_precomp")
    ]


def lib():
    global _LIB
    if _LIB is None:
        path = _build.build(force=False)
        _LIB = C.CDLL(path)
        _LIB.orc_scan.restype = C.c_uint64
        _LIB.orc_set_threads.restype = C.c_int
    return _LIB


def set_threads(n: int) -> int:
    return lib().orc_set_threads(int(n))


@dataclass
class Frame:
    """The per-frame record the reference passes as GaussianRasterizationSettings
    (benchmarks/nerf/origin_gs/gs_model.py:148-161), as plain numbers."""

    image_width: int
    image_height: int
    tanfovx: float
    tanfovy: float
    viewmatrix: np.ndarray  # [4,4] f32, p_view = [p,1] @ viewmatrix
    projmatrix: np.ndarray  # [4,4] f32
    campos: np.ndarray  # [3]
    bg: np.ndarray = field(default_factory=lambda: np.zeros(3, np.float32))
    scale_modifier: float = 1.0
    sh_degree: int = 0

    @property
    def grid(self):
        return ((self.image_width + 15) // 16, (self.image_height + 15) // 16)

    def _c(self, sh_coeffs: int) -> _Frame:
        f = _Frame()
        f.image_width, f.image_height = int(self.image_width), int(self.image_height)
        f.tanfovx, f.tanfovy = float(self.tanfovx), float(self.tanfovy)
        f.scale_modifier, f.sh_degree, f.sh_coeffs = float(self.scale_modifier), int(self.sh_degree), int(sh_coeffs)
        f.viewmatrix[:] = np.asarray(self.viewmatrix, np.float32).reshape(16).tolist()
        f.projmatrix[:] = np.asarray(self.projmatrix, np.float32).reshape(16).tolist()
        f.campos[:] = np.asarray(self.campos, np.float32).reshape(3).tolist()
        f.bg[:] = np.asarray(self.bg, np.float32).reshape(3).tolist()
        return f


def _f32(a, shape=None):
    if a is None:
        return None
    a = np.ascontiguousarray(np.asarray(a, dtype=np.float32))
    if shape is not None:
        a = a.reshape(shape)
    return a


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class Gaussians:
    """Inputs of GaussianRasterizer.forward (SH or precomputed colours;
    scale+rotation or precomputed covariance)."""

    def __init__(self, means3D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
                 cov3D_precomp=None):
        self.means3D = _f32(means3D)
        self.P = self.means3D.shape[0]
        P = self.P
        self.opacities = _f32(opacities, (P,))
        self.shs = _f32(shs)
        self.colors_precomp = _f32(colors_precomp, (P, 3)) if colors_precomp is not None else None
        self.scales = _f32(scales, (P, 3)) if scales is not None else None
        self.rotations = _f32(rotations, (P, 4)) if rotations is not None else None
        self.cov3D_precomp = _f32(cov3D_precomp, (P, 6)) if cov3D_precomp is not None else None
        if (self.shs is None) == (self.colors_precomp is None):
            raise ValueError("exactly one of shs / colors_precomp")
        if (self.scales is None or self.rotations is None) == (self.cov3D_precomp is None):
            raise ValueError("exactly one of (scales, rotations) / cov3D_precomp")
        self.sh_coeffs = 0 if self.shs is None else int(self.shs.reshape(P, -1, 3).shape[1])

    def _c(self) -> _Gaussians:
        g = _Gaussians()
        g.P = self.P
        for n in ("means3D", "shs", "colors_precomp", "opacities", "scales", "rotations", "cov3D_precomp"):
            setattr(g, n, _ptr(getattr(self, n)))
        return g


def cov3d(scale, mod, quat):
    out = np.zeros(6, np.float32)
    lib().orc_cov3d(_ptr(_f32(scale, (3,))), C.c_float(mod), _ptr(_f32(quat, (4,))), _ptr(out))
    return out


def sh_to_rgb(deg, sh, direction):
    out = np.zeros(3, np.float32)
    sh = _f32(sh).reshape(-1, 3)
    lib().orc_sh_to_rgb(C.c_int(deg), _ptr(sh), _ptr(_f32(direction, (3,))), _ptr(out))
    return out


def tile_rect(px, py, r, grid_x, grid_y):
    out = np.zeros(4, np.int32)
    lib().orc_tile_rect(C.c_float(px), C.c_float(py), C.c_int(r), C.c_int(grid_x), C.c_int(grid_y), _ptr(out))
    return out


def preprocess(frame: Frame, g: Gaussians):
    P = g.P
    out = dict(
        depth=np.zeros(P, np.float32),
        radii=np.zeros(P, np.int32),
        xy=np.zeros((P, 2), np.float32),
        conic_opacity=np.zeros((P, 4), np.float32),
        rgb=np.zeros((P, 3), np.float32),
        rect=np.zeros((P, 4), np.int32),
        tiles_touched=np.zeros(P, np.uint32),
    )
    cf, cg = frame._c(g.sh_coeffs), g._c()
    lib().orc_preprocess(C.byref(cf), C.byref(cg), *[_ptr(out[k]) for k in
                         ("depth", "radii", "xy", "conic_opacity", "rgb", "rect", "tiles_touched")])
    return out


def visible_filter(frame: Frame, means3D, scales=None, rotations=None, cov3D_precomp=None):
    P = np.asarray(means3D).shape[0]
    g = Gaussians(means3D, np.zeros(P, np.float32), colors_precomp=np.zeros((P, 3), np.float32), scales=scales,
                  rotations=rotations, cov3D_precomp=cov3D_precomp)
    radii = np.zeros(P, np.int32)
    cf, cg = frame._c(0), g._c()
    lib().orc_visible_filter(C.byref(cf), C.byref(cg), _ptr(radii))
    return radii


def scan(tiles_touched):
    t = np.ascontiguousarray(tiles_touched, np.uint32)
    off = np.zeros_like(t)
    total = lib().orc_scan(_ptr(t), C.c_int(t.shape[0]), _ptr(off))
    return off, int(total)


def duplicate_keys(pre, offsets, total, grid_x):
    keys = np.zeros(total, np.uint64)
    vals = np.zeros(total, np.uint32)
    P = pre["radii"].shape[0]
    lib().orc_duplicate_keys(C.c_int(P), _ptr(pre["radii"]), _ptr(pre["rect"]), _ptr(pre["depth"]), _ptr(offsets),
                             C.c_int(grid_x), _ptr(keys), _ptr(vals))
    return keys, vals


def sort_pairs(keys, vals):
    k = np.ascontiguousarray(keys, np.uint64).copy()
    v = np.ascontiguousarray(vals, np.uint32).copy()
    lib().orc_sort_pairs(C.c_uint64(k.shape[0]), _ptr(k), _ptr(v))
    return k, v


def tile_ranges(sorted_keys, tiles):
    r = np.zeros((tiles, 2), np.uint32)
    k = np.ascontiguousarray(sorted_keys, np.uint64)
    lib().orc_tile_ranges(C.c_uint64(k.shape[0]), _ptr(k), C.c_int(tiles), _ptr(r))
    return r


def blend(frame: Frame, ranges, vals, pre):
    H, W = frame.image_height, frame.image_width
    out = dict(
        image=np.zeros((3, H, W), np.float32),
        depth=np.zeros((H, W), np.float32),
        alpha=np.zeros((H, W), np.float32),
        fragile=np.zeros((H, W), np.uint8),
    )
    stats = np.zeros(3, np.uint64)
    cf = frame._c(0)
    ranges = np.ascontiguousarray(ranges, np.uint32)
    vals = np.ascontiguousarray(vals, np.uint32)
    lib().orc_blend(C.byref(cf), _ptr(ranges), _ptr(vals), _ptr(pre["xy"]), _ptr(pre["conic_opacity"]),
                    _ptr(pre["rgb"]), _ptr(pre["depth"]), _ptr(out["image"]), _ptr(out["depth"]), _ptr(out["alpha"]),
                    _ptr(out["fragile"]), _ptr(stats))
    out["pairs_evaluated"], out["pairs_accepted"], out["tile_work"] = (int(s) for s in stats)
    return out


def render(frame: Frame, g: Gaussians, keep_intermediates: bool = True):
    """Whole pipeline; returns image/depth/alpha/radii plus every intermediate."""
    pre = preprocess(frame, g)
    offsets, total = scan(pre["tiles_touched"])
    gx, gy = frame.grid
    keys, vals = duplicate_keys(pre, offsets, total, gx)
    skeys, svals = sort_pairs(keys, vals)
    ranges = tile_ranges(skeys, gx * gy)
    out = blend(frame, ranges, svals, pre)
    out["radii"] = pre["radii"]
    out["num_keys"] = total
    if keep_intermediates:
        out.update(pre=pre, offsets=offsets, keys=keys, values=vals, sorted_keys=skeys, sorted_values=svals,
                   ranges=ranges)
    return out


GRAD_SLOTS = 10  # d/dpx, d/dpy, d/dconic (x, y, z), d/dopacity, d/drgb (3), d/ddepth


def render_backward(frame: Frame, g: Gaussians, fwd, g_image, g_depth=None, g_alpha=None):
    """Gradients of sum(image * g_image) [+ depth * g_depth + alpha * g_alpha] with respect to every input of
    `render`, from the intermediates `fwd` that `render` returned (oracle/gs_oracle_backward.c).  All float64."""
    P, M = g.P, g.sh_coeffs
    H, W = frame.image_height, frame.image_width
    pre = fwd["pre"]
    acc = np.zeros((P, GRAD_SLOTS), np.float64)
    cf = frame._c(M)
    gi = _f32(g_image, (3, H, W))
    gd = _f32(g_depth, (H, W)) if g_depth is not None else None
    ga = _f32(g_alpha, (H, W)) if g_alpha is not None else None
    ranges = np.ascontiguousarray(fwd["ranges"], np.uint32)
    vals = np.ascontiguousarray(fwd["sorted_values"], np.uint32)
    lib().orc_blend_backward(C.byref(cf), _ptr(ranges), _ptr(vals), _ptr(pre["xy"]), _ptr(pre["conic_opacity"]),
                             _ptr(pre["rgb"]), _ptr(pre["depth"]), _ptr(gi), _ptr(gd), _ptr(ga), _ptr(acc))
    out = dict(acc=acc, means3D=np.zeros((P, 3)), means2D=np.zeros((P, 3)), opacities=np.zeros(P))
    out["shs" if g.shs is not None else "colors_precomp"] = np.zeros((P, M, 3) if g.shs is not None else (P, 3))
    if g.cov3D_precomp is not None:
        out["cov3D_precomp"] = np.zeros((P, 6))
    else:
        out["scales"], out["rotations"] = np.zeros((P, 3)), np.zeros((P, 4))
    cg = g._c()
    lib().orc_preprocess_backward(C.byref(cf), C.byref(cg), _ptr(np.ascontiguousarray(pre["radii"], np.int32)),
                                  _ptr(acc), *[_ptr(out.get(k)) for k in
                                               ("means3D", "means2D", "shs", "colors_precomp", "opacities", "scales",
                                                "rotations", "cov3D_precomp")])
    return out
