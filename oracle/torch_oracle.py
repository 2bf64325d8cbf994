"""PyTorch-CPU rasterizer with the reference's semantics.

TEST INFRASTRUCTURE / CPU BASELINE ONLY -- never imported by the shipped
package.  A vectorised torch (CPU, fp32) restatement of the pipeline behind the
reference's `GaussianRasterizer.forward` (benchmarks/nerf/origin_gs/
gs_model.py:211-220), following the same in-tree statements as the C oracle:
SH -> RGB (landmark/nerf_components/utils/sh_utils.py:67-94 and
origin_gs/gs_model.py:184-193), scale/quaternion -> covariance
(landmark/nerf_components/utils/general_utils.py:64-102,
.../encodings/gaussian_encoding.py:22-38), matrix conventions
(landmark/nerf_components/utils/graphics_utils.py:43-77).

Every quantity that feeds the integer pipeline is computed with separate
elementwise multiplies and adds in the same order as oracle/gs_oracle.c (torch
eager never fuses them), so radii, keys, sorted order and ranges are
bit-identical to the C oracle; tests/test_oracle_torch.py checks exactly that.
Pinning: through that equality this file inherits the C oracle's pins (closed
forms, invariants, brute force); the rasterizer as a whole stays "parity
unpinned" against the absent third-party CUDA source.
"""
import math
import os
import time

import torch

C0 = 0.28209479177387814
C1 = 0.4886025119029199
C2 = [1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792, 0.5462742152960396]
C3 = [-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154, -0.4570457994644658,
      1.445305721320277, -0.5900435899266435]


def _f(v):
    return torch.tensor(v, dtype=torch.float32)


def cov3d(scales, mod, quats):
    s = scales * _f(mod)
    r, x, y, z = quats[:, 0], quats[:, 1], quats[:, 2], quats[:, 3]
    R = [
        [1.0 - 2.0 * (y * y + z * z), 2.0 * (x * y - r * z), 2.0 * (x * z + r * y)],
        [2.0 * (x * y + r * z), 1.0 - 2.0 * (x * x + z * z), 2.0 * (y * z - r * x)],
        [2.0 * (x * z - r * y), 2.0 * (y * z + r * x), 1.0 - 2.0 * (x * x + y * y)],
    ]
    L = [[R[i][k] * s[:, k] for k in range(3)] for i in range(3)]
    out = []
    for i in range(3):
        for j in range(i, 3):
            out.append((L[i][0] * L[j][0] + L[i][1] * L[j][1]) + L[i][2] * L[j][2])
    return torch.stack(out, dim=1)


def sh_to_rgb(deg, shs, dirs):
    """shs [V,M,3], dirs [V,3] (unnormalised) -> clamp_min(eval_sh + 0.5, 0)."""
    ln = torch.sqrt((dirs[:, 0] * dirs[:, 0] + dirs[:, 1] * dirs[:, 1]) + dirs[:, 2] * dirs[:, 2])
    x, y, z = (dirs[:, 0] / ln)[:, None], (dirs[:, 1] / ln)[:, None], (dirs[:, 2] / ln)[:, None]
    sh = lambda k: shs[:, k, :]  # noqa: E731
    res = _f(C0) * sh(0)
    if deg > 0:
        res = res - _f(C1) * y * sh(1) + _f(C1) * z * sh(2) - _f(C1) * x * sh(3)
        if deg > 1:
            xx, yy, zz = x * x, y * y, z * z
            xy, yz, xz = x * y, y * z, x * z
            res = (res + _f(C2[0]) * xy * sh(4) + _f(C2[1]) * yz * sh(5) + _f(C2[2]) * (2.0 * zz - xx - yy) * sh(6)
                   + _f(C2[3]) * xz * sh(7) + _f(C2[4]) * (xx - yy) * sh(8))
            if deg > 2:
                res = (res + _f(C3[0]) * y * (3.0 * xx - yy) * sh(9) + _f(C3[1]) * xy * z * sh(10)
                       + _f(C3[2]) * y * (4.0 * zz - xx - yy) * sh(11)
                       + _f(C3[3]) * z * (2.0 * zz - 3.0 * xx - 3.0 * yy) * sh(12)
                       + _f(C3[4]) * x * (4.0 * zz - xx - yy) * sh(13) + _f(C3[5]) * z * (xx - yy) * sh(14)
                       + _f(C3[6]) * x * (xx - 3.0 * yy) * sh(15))
    return torch.clamp_min(res + 0.5, 0.0)


def _tile_clamp(v, grid):
    t = torch.trunc(torch.clamp(v, 0.0, float(grid)))
    return torch.where(v > 0, t, torch.zeros_like(t)).to(torch.int32)


def preprocess(fr, means3D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
               cov3D_precomp=None):
    """fr: dict with image_width/height, tanfovx/y, viewmatrix[4,4], projmatrix[4,4], campos[3], bg[3],
    scale_modifier, sh_degree.  Returns per-Gaussian tensors (zeros where culled)."""
    P = means3D.shape[0]
    V, M = fr["viewmatrix"].reshape(-1), fr["projmatrix"].reshape(-1)
    W, H = fr["image_width"], fr["image_height"]
    gx, gy = (W + 15) // 16, (H + 15) // 16
    x, y, z = means3D[:, 0], means3D[:, 1], means3D[:, 2]
    pvx = ((V[0] * x + V[4] * y) + V[8] * z) + V[12]
    pvy = ((V[1] * x + V[5] * y) + V[9] * z) + V[13]
    pvz = ((V[2] * x + V[6] * y) + V[10] * z) + V[14]
    alive = pvz > 0.2
    phx = ((M[0] * x + M[4] * y) + M[8] * z) + M[12]
    phy = ((M[1] * x + M[5] * y) + M[9] * z) + M[13]
    phw = ((M[3] * x + M[7] * y) + M[11] * z) + M[15]
    pw = 1.0 / (phw + _f(0.0000001))
    ppx, ppy = phx * pw, phy * pw
    S = cov3D_precomp if cov3D_precomp is not None else cov3d(scales, fr["scale_modifier"], rotations)
    Sg = [[S[:, 0], S[:, 1], S[:, 2]], [S[:, 1], S[:, 3], S[:, 4]], [S[:, 2], S[:, 4], S[:, 5]]]
    tfx, tfy = _f(fr["tanfovx"]), _f(fr["tanfovy"])
    fx, fy = _f(float(W)) / (2.0 * tfx), _f(float(H)) / (2.0 * tfy)
    limx, limy = _f(1.3) * tfx, _f(1.3) * tfy
    tz = torch.where(alive, pvz, torch.ones_like(pvz))  # keep culled lanes finite
    tx = torch.minimum(limx, torch.maximum(-limx, pvx / tz)) * tz
    ty = torch.minimum(limy, torch.maximum(-limy, pvy / tz)) * tz
    J00, J02 = fx / tz, -(fx * tx) / (tz * tz)
    J11, J12 = fy / tz, -(fy * ty) / (tz * tz)
    A = [[J00 * V[4 * k + 0] + J02 * V[4 * k + 2] for k in range(3)],
         [J11 * V[4 * k + 1] + J12 * V[4 * k + 2] for k in range(3)]]
    B = [[(A[i][0] * Sg[0][k] + A[i][1] * Sg[1][k]) + A[i][2] * Sg[2][k] for k in range(3)] for i in range(2)]
    c00 = (B[0][0] * A[0][0] + B[0][1] * A[0][1]) + B[0][2] * A[0][2]
    c01 = (B[0][0] * A[1][0] + B[0][1] * A[1][1]) + B[0][2] * A[1][2]
    c11 = (B[1][0] * A[1][0] + B[1][1] * A[1][1]) + B[1][2] * A[1][2]
    a, b, c = c00 + _f(0.3), c01, c11 + _f(0.3)
    det = a * c - b * b
    alive = alive & (det != 0)
    det_inv = 1.0 / det
    mid = 0.5 * (a + c)
    q = torch.sqrt(torch.clamp_min(mid * mid - det, 0.1))
    rf = torch.ceil(3.0 * torch.sqrt(torch.maximum(mid + q, mid - q)))
    alive = alive & (rf < 1073741824.0)
    rf = torch.where(alive, rf, torch.zeros_like(rf))
    px = ((ppx + 1.0) * float(W) - 1.0) * 0.5
    py = ((ppy + 1.0) * float(H) - 1.0) * 0.5
    x0 = _tile_clamp((px - rf) / 16.0, gx)
    y0 = _tile_clamp((py - rf) / 16.0, gy)
    x1 = _tile_clamp((px + rf + 15.0) / 16.0, gx)
    y1 = _tile_clamp((py + rf + 15.0) / 16.0, gy)
    area = (x1 - x0) * (y1 - y0)
    alive = alive & (area != 0)
    zero = torch.zeros_like(px)
    radii = torch.where(alive, rf, zero).to(torch.int32)
    out = dict(
        radii=radii,
        tiles_touched=torch.where(alive, area, torch.zeros_like(area)),
        rect=torch.where(alive[:, None], torch.stack([x0, y0, x1, y1], 1), torch.zeros(P, 4, dtype=torch.int32)),
        depth=torch.where(alive, pvz, zero),
        xy=torch.where(alive[:, None], torch.stack([px, py], 1), torch.zeros(P, 2)),
        conic_opacity=torch.where(alive[:, None], torch.stack([c * det_inv, -b * det_inv, a * det_inv,
                                                              opacities.reshape(-1)], 1), torch.zeros(P, 4)),
    )
    if colors_precomp is not None:
        rgb = colors_precomp
    else:
        rgb = sh_to_rgb(fr["sh_degree"], shs, means3D - fr["campos"][None, :])
    out["rgb"] = torch.where(alive[:, None], rgb, torch.zeros(P, 3))
    return out


def make_keys(pre, grid_x):
    """(keys int64[N], values int32[N], offsets) in emission order."""
    touched = pre["tiles_touched"].to(torch.int64)
    offsets = torch.cumsum(touched, 0)
    N = int(offsets[-1]) if touched.numel() else 0
    idx = torch.repeat_interleave(torch.arange(touched.numel()), touched)
    local = torch.arange(N) - (offsets - touched)[idx]
    rect = pre["rect"].to(torch.int64)
    w = (rect[:, 2] - rect[:, 0])[idx]
    ty = rect[idx, 1] + local // torch.clamp_min(w, 1)
    tx = rect[idx, 0] + local % torch.clamp_min(w, 1)
    depth_bits = pre["depth"].detach().to(torch.float32).view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    keys = ((ty * grid_x + tx) << 32) | depth_bits[idx]
    return keys, idx.to(torch.int32), offsets


def sort_pairs(keys, values):
    skeys, perm = torch.sort(keys, stable=True)
    return skeys, values[perm]


def tile_ranges(skeys, tiles):
    t = skeys >> 32
    ids = torch.arange(tiles)
    lo = torch.searchsorted(t, ids, right=False)
    hi = torch.searchsorted(t, ids, right=True)
    empty = lo == hi
    return torch.stack([torch.where(empty, torch.zeros_like(lo), lo), torch.where(empty, torch.zeros_like(hi), hi)], 1)


def blend_tile(fr, t, ranges, svals, pre, straight_through=False):
    """One 16x16 tile, all its Gaussians at once: [n,256] elementwise passes
    and a sequential cumulative product for the transmittance.  Differentiable
    by torch.autograd in the dtype of `pre` (fp32 or fp64); `straight_through`
    lets the gradient through min(0.99, .) unchanged, as the published backward
    pass of the rasterizer does (the forward value may then differ from the
    clamp's in the last bit, so it is used for gradient checks only)."""
    dt = pre["xy"].dtype
    W, H = fr["image_width"], fr["image_height"]
    gx = (W + 15) // 16
    lo, hi = int(ranges[t, 0]), int(ranges[t, 1])
    px = (t % gx) * 16 + torch.arange(16).repeat(16)
    py = (t // gx) * 16 + torch.arange(16).repeat_interleave(16)
    bg = fr["bg"]
    if hi == lo:
        T = torch.ones(256, dtype=dt)
        return px, py, bg[:, None] * T[None, :], torch.zeros(256, dtype=dt), 1.0 - T, 0
    g = svals[lo:hi].long()
    xy, co, col, dep = pre["xy"][g], pre["conic_opacity"][g], pre["rgb"][g], pre["depth"][g]
    dx = xy[:, 0:1] - px[None, :].to(dt)
    dy = xy[:, 1:2] - py[None, :].to(dt)
    power = -0.5 * (co[:, 0:1] * dx * dx + co[:, 2:3] * dy * dy) - co[:, 1:2] * dx * dy
    alpha = torch.clamp_max(co[:, 3:4] * torch.exp(power), 0.99)
    if straight_through:
        raw = co[:, 3:4] * torch.exp(power)
        alpha = raw + (alpha - raw).detach()
    valid = (power <= 0) & (alpha >= 1.0 / 255.0)
    a = torch.where(valid, alpha, torch.zeros_like(alpha))
    test_T = torch.cumprod(1.0 - a, dim=0)
    stopped = torch.cumsum((valid & (test_T < 0.0001)).to(torch.int32), 0) > 0
    T_before = torch.cat([torch.ones(1, 256, dtype=dt), test_T[:-1]], 0)
    w = torch.where(valid & ~stopped, a * T_before, torch.zeros_like(a))
    C = col.t() @ w  # [3,256]
    D = dep[None, :] @ w
    T_final = torch.where(stopped, torch.ones_like(test_T), test_T).amin(0)
    T_final = torch.where(stopped[0], torch.ones(256, dtype=dt), T_final)
    return px, py, C + bg[:, None] * T_final[None, :], D[0], 1.0 - T_final, (hi - lo)


def blend(fr, ranges, svals, pre, tiles=None, straight_through=False):
    W, H = fr["image_width"], fr["image_height"]
    gx, gy = (W + 15) // 16, (H + 15) // 16
    dt = pre["xy"].dtype
    image = torch.zeros(3, H, W, dtype=dt)
    depth = torch.zeros(H, W, dtype=dt)
    alpha = torch.zeros(H, W, dtype=dt)
    for t in (range(gx * gy) if tiles is None else tiles):
        px, py, C, D, A, _ = blend_tile(fr, t, ranges, svals, pre, straight_through)
        ok = (px < W) & (py < H)
        image[:, py[ok], px[ok]] = C[:, ok]
        depth[py[ok], px[ok]] = D[ok]
        alpha[py[ok], px[ok]] = A[ok]
    return image, depth, alpha


def render(fr, means3D, opacities, straight_through=False, **kw):
    pre = preprocess(fr, means3D, opacities, **kw)
    gx, gy = (fr["image_width"] + 15) // 16, (fr["image_height"] + 15) // 16
    keys, vals, offsets = make_keys(pre, gx)
    skeys, svals = sort_pairs(keys, vals)
    ranges = tile_ranges(skeys, gx * gy)
    image, depth, alpha = blend(fr, ranges, svals, pre, straight_through=straight_through)
    return dict(image=image, depth=depth, alpha=alpha, radii=pre["radii"], pre=pre, keys=keys, values=vals,
                offsets=offsets, sorted_keys=skeys, sorted_values=svals, ranges=ranges)


def frame_dict(scene, cam=None):
    cam = cam or scene.camera
    return dict(image_width=cam.width, image_height=cam.height, tanfovx=math.tan(cam.FovX * 0.5),
                tanfovy=math.tan(cam.FovY * 0.5), viewmatrix=cam.world_view_transform.cpu(),
                projmatrix=cam.full_proj_transform.cpu(), campos=cam.camera_center.cpu(), bg=scene.bg.cpu(),
                scale_modifier=1.0, sh_degree=scene.sh_degree)


def timed_baseline(scene, blend_budget_s: float = 12.0, colors_precomp=None, extra_seconds: float = 0.0,
                   extra_note: str = ""):
    """CPU baseline for bench.py: preprocess, key generation and the stable
    sort are timed in full on all host cores; blending is timed on every k-th
    tile (k chosen so that it fits the budget) and extrapolated by range
    length.  `colors_precomp` replaces the SH evaluation (the Scaffold-GS
    call); `extra_seconds` / `extra_note` add a stage timed by the caller (the
    anchor decode) to the frame time.  Returns the cpu_baseline object of the
    bench line."""
    cores = os.cpu_count() or 1
    cores = min(cores, 16)
    torch.set_num_threads(cores)
    fr = frame_dict(scene)
    W, H = fr["image_width"], fr["image_height"]
    gx, gy = (W + 15) // 16, (H + 15) // 16
    with torch.no_grad():
        t0 = time.perf_counter()
        pre = preprocess(fr, scene.means3D, scene.opacities, shs=None if colors_precomp is not None else scene.shs,
                         colors_precomp=colors_precomp, scales=scene.scales, rotations=scene.rotations)
        t1 = time.perf_counter()
        keys, vals, _ = make_keys(pre, gx)
        t2 = time.perf_counter()
        skeys, svals = sort_pairs(keys, vals)
        ranges = tile_ranges(skeys, gx * gy)
        t3 = time.perf_counter()
        lens = (ranges[:, 1] - ranges[:, 0]).double()
        total_len = float(lens.sum())
        # probe a few tiles to size the sample
        stride = 8
        sample_len, t_blend, done_tiles = 0.0, 0.0, 0
        tb0 = time.perf_counter()
        for t in range(0, gx * gy, stride):
            blend_tile(fr, t, ranges, svals, pre)
            sample_len += float(lens[t])
            done_tiles += 1
            if time.perf_counter() - tb0 > blend_budget_s:
                break
        t_blend = time.perf_counter() - tb0
    blend_full = t_blend * (total_len / sample_len) if sample_len > 0 else t_blend * gx * gy / max(done_tiles, 1)
    frame_s = (t1 - t0) + (t2 - t1) + (t3 - t2) + blend_full + extra_seconds
    return {
        "value": round(1.0 / frame_s, 4),
        "unit": "frames/s",
        "cores": cores,
        "kind": "port",
        "sample": (extra_note + "PyTorch-CPU rasterizer (oracle/torch_oracle.py), same scene: preprocess %.2fs + keys %.2fs + "
                   "stable sort/ranges %.2fs timed in full (%d Gaussians, %d keys); blend timed on %d of %d tiles "
                   "(every %dth, %.2fs) and extrapolated by tile range length to %.1fs"
                   % (t1 - t0, t2 - t1, t3 - t2, scene.P, keys.numel(), done_tiles, gx * gy, stride, t_blend,
                      blend_full)),
        "stages_s": {"preprocess": round(t1 - t0, 3), "keys": round(t2 - t1, 3), "sort_ranges": round(t3 - t2, 3),
                     "blend_extrapolated": round(blend_full, 2)},
    }
