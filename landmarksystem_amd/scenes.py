"""Seeded synthetic scenes for the five benchmark configurations.

No trained checkpoints or datasets are available offline, so the renderer is
measured and tested on synthetic Gaussians with the shapes and layouts the
reference's models hand to the rasterizer (benchmarks/nerf/origin_gs/
gs_model.py:164-220; scaffold_gs/gs_model.py:178-227).  Seeds follow the
reference's default `random_seed` (landmark/nerf_components/configs/
render_config.py:47): 20211202 + config index.  Everything is generated on
the CPU in fp32 so that a CPU checker and the GPU consume identical bits.
"""
import math
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from .cameras import Camera

BASE_SEED = 20211202


@dataclass
class GaussianScene:
    name: str
    means3D: torch.Tensor  # [P,3]
    scales: torch.Tensor  # [P,3] (exp-activated)
    rotations: torch.Tensor  # [P,4] unit (r,x,y,z)
    opacities: torch.Tensor  # [P,1] (sigmoid-activated)
    shs: torch.Tensor  # [P,M,3]
    sh_degree: int
    cameras: List[Camera]
    bg: torch.Tensor = field(default_factory=lambda: torch.zeros(3))

    @property
    def P(self) -> int:
        return self.means3D.shape[0]

    @property
    def camera(self) -> Camera:
        return self.cameras[0]

    def to(self, device) -> "GaussianScene":
        return GaussianScene(
            self.name, self.means3D.to(device), self.scales.to(device), self.rotations.to(device),
            self.opacities.to(device), self.shs.to(device), self.sh_degree,
            [c.to(device) for c in self.cameras], self.bg.to(device),
        )


@dataclass
class AnchorScene:
    """Scaffold-GS style scene: anchors with features, offsets and three MLPs
    (landmark/nerf_components/model_components/fields/anchor_decoder.py:79-104)."""

    name: str
    anchor: torch.Tensor  # [A,3]
    anchor_feat: torch.Tensor  # [A,32] (fp16-representable values, stored fp32)
    offset: torch.Tensor  # [A,10,3]
    scaling: torch.Tensor  # [A,6] (exp-activated)
    rotation: torch.Tensor  # [A,4] identity
    mlp: dict  # {"opacity"|"cov"|"color": (W0[32,36], b0[32], W1[k,32], b1[k])}
    cameras: List[Camera]
    n_offsets: int = 10
    bg: torch.Tensor = field(default_factory=lambda: torch.zeros(3))

    @property
    def camera(self) -> Camera:
        return self.cameras[0]


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _unit_quats(n: int, g: torch.Generator) -> torch.Tensor:
    q = torch.randn(n, 4, generator=g)
    return q / q.norm(dim=1, keepdim=True)


def _shs(n: int, degree: int, g: torch.Generator) -> torch.Tensor:
    m = (degree + 1) ** 2
    shs = torch.empty(n, m, 3)
    shs[:, 0] = torch.randn(n, 3, generator=g) * 0.3
    if m > 1:
        shs[:, 1:] = torch.randn(n, m - 1, 3, generator=g) * 0.05
    return shs


def config1(P: int = 10_000, width: int = 256, height: int = 256) -> GaussianScene:
    """10k Gaussians in [-1,1]^3, camera at z=-3 looking down +z, 60 deg FoV,
    SH degree 0, 256x256: the CPU-runnable case."""
    g = _gen(BASE_SEED + 1)
    means = torch.rand(P, 3, generator=g) * 2 - 1
    scales = torch.exp(torch.randn(P, 3, generator=g) * 0.5 - 4.0)
    rots = _unit_quats(P, g)
    opac = torch.sigmoid(torch.randn(P, 1, generator=g))
    shs = _shs(P, 0, g)
    fov = math.radians(60.0)
    cam = Camera.from_world2cam(torch.eye(3).numpy(), [0.0, 0.0, 3.0], width, height, fov, fov)
    return GaussianScene("C1", means, scales, rots, opac, shs, 0, [cam])


def config2(P: int = 1_000_000, width: int = 1920, height: int = 1080) -> GaussianScene:
    """1M Gaussians ~ N(0, 5^2 I), camera at distance 20, SH degree 3, 1080p."""
    g = _gen(BASE_SEED + 2)
    means = torch.randn(P, 3, generator=g) * 5.0
    scales = torch.exp(torch.randn(P, 3, generator=g) * 0.7 - 3.0)
    rots = _unit_quats(P, g)
    opac = torch.sigmoid(torch.randn(P, 1, generator=g) * 1.5)
    shs = _shs(P, 3, g)
    cam = Camera.look_at([0.0, 0.0, -20.0], [0.0, 0.0, 0.0], [0.0, -1.0, 0.0], width, height, math.radians(60.0))
    return GaussianScene("C2", means, scales, rots, opac, shs, 3, [cam])


def _slab(P: int, half_extent: float, g: torch.Generator):
    xy = (torch.rand(P, 2, generator=g) * 2 - 1) * half_extent
    u = torch.rand(P, generator=g).clamp_min(1e-12)
    z = (-5.0 * torch.log(u)).clamp(0.0, 40.0)
    means = torch.cat([xy, z[:, None]], dim=1)
    log_s = torch.randn(P, 3, generator=g) * 0.8 - 2.5
    s = torch.exp(log_s)
    s = torch.maximum(s, s.max(dim=1, keepdim=True).values / 50.0)  # anisotropy <= 1:50
    return means, s


def config3(P: int = 6_000_000, width: int = 1920, height: int = 1080) -> GaussianScene:
    """City-block slab 200m x 200m x 40m, aerial camera at 150m pitched 45 deg,
    SH degree 3, 1080p.  The headline configuration."""
    g = _gen(BASE_SEED + 3)
    means, scales = _slab(P, 100.0, g)
    rots = _unit_quats(P, g)
    opac = torch.sigmoid(torch.randn(P, 1, generator=g) * 1.5 + 0.5)
    shs = _shs(P, 3, g)
    cam = Camera.look_at([0.0, -150.0, 150.0], [0.0, 0.0, 0.0], [0.0, 0.0, 1.0], width, height, math.radians(60.0))
    return GaussianScene("C3", means, scales, rots, opac, shs, 3, [cam])


def frustum_fraction(cam: Camera, points: torch.Tensor) -> float:
    """Fraction of `points` whose centre lies inside the camera frustum (z_view > 0.2, |ndc| < 1)."""
    hom = torch.cat([points, torch.ones(points.shape[0], 1)], dim=1)
    view_z = (hom @ cam.world_view_transform)[:, 2]
    clip = hom @ cam.full_proj_transform
    ndc = clip[:, :2] / (clip[:, 3:4] + 1e-7)
    inside = (view_z > 0.2) & (ndc.abs() < 1.0).all(dim=1)
    return float(inside.float().mean())


def aerial_poses(n: int, width: int, height: int, g: torch.Generator, target_half: float = 150.0,
                 points: Optional[torch.Tensor] = None, keep=(0.22, 0.58)) -> List[Camera]:
    """Random aerial poses: altitude U[100,300], pitch U[30,60] deg, yaw U[0,360), look-at target on the ground.
    With `points`, candidates are drawn (deterministically, from the same generator) until the fraction of
    points inside the frustum falls in `keep`, so that 20-60 % of the scene survives culling in every frame."""
    cams = []
    while len(cams) < n:
        r = torch.rand(5, generator=g).tolist()
        alt = 100.0 + 200.0 * r[0]
        pitch = math.radians(30.0 + 30.0 * r[1])
        yaw = 2.0 * math.pi * r[2]
        tx, ty = (2 * r[3] - 1) * target_half, (2 * r[4] - 1) * target_half
        ground = alt / math.tan(pitch)
        eye = [tx - ground * math.cos(yaw), ty - ground * math.sin(yaw), alt]
        cam = Camera.look_at(eye, [tx, ty, 0.0], [0.0, 0.0, 1.0], width, height, math.radians(60.0))
        if points is not None and not keep[0] <= frustum_fraction(cam, points) <= keep[1]:
            continue
        cams.append(cam)
    return cams


def config4(P: int = 20_000_000, width: int = 3840, height: int = 2160, n_poses: int = 30) -> GaussianScene:
    """Large slab 600m x 600m at 4K with a trajectory of random aerial poses."""
    g = _gen(BASE_SEED + 4)
    means, scales = _slab(P, 300.0, g)
    rots = _unit_quats(P, g)
    opac = torch.sigmoid(torch.randn(P, 1, generator=g) * 1.5 + 0.5)
    shs = _shs(P, 3, g)
    cams = aerial_poses(n_poses, width, height, g, points=means[: min(P, 100_000)])
    return GaussianScene("C4", means, scales, rots, opac, shs, 3, cams)


def _fp16_values(t: torch.Tensor) -> torch.Tensor:
    return t.half().float()


def config5(A: int = 500_000, width: int = 1920, height: int = 1080, n_offsets: int = 10,
            feat_dim: int = 32) -> AnchorScene:
    """Scaffold-GS: anchors in the config-3 slab, 32-d features, 10 offsets,
    three 36->32->k MLPs with fp16-representable weights."""
    g = _gen(BASE_SEED + 5)
    xy = (torch.rand(A, 2, generator=g) * 2 - 1) * 100.0
    u = torch.rand(A, generator=g).clamp_min(1e-12)
    z = (-5.0 * torch.log(u)).clamp(0.0, 40.0)
    anchor = torch.cat([xy, z[:, None]], dim=1)
    feat = _fp16_values(torch.randn(A, feat_dim, generator=g) * 0.5)
    scaling = torch.exp(torch.randn(A, 6, generator=g) * 0.8 - 2.5)
    offset = torch.randn(A, n_offsets, 3, generator=g) * 0.1
    rotation = torch.zeros(A, 4)
    rotation[:, 0] = 1.0
    in_dim = feat_dim + 3 + 1
    mlp = {}
    for name, k in (("opacity", n_offsets), ("cov", 7 * n_offsets), ("color", 3 * n_offsets)):
        w0 = _fp16_values(torch.randn(feat_dim, in_dim, generator=g) * in_dim ** -0.5)
        w1 = _fp16_values(torch.randn(k, feat_dim, generator=g) * feat_dim ** -0.5)
        mlp[name] = (w0, torch.zeros(feat_dim), w1, torch.zeros(k))
    cam = Camera.look_at([0.0, -150.0, 150.0], [0.0, 0.0, 0.0], [0.0, 0.0, 1.0], width, height, math.radians(60.0))
    return AnchorScene("C5", anchor, feat, offset, scaling, rotation, mlp, [cam], n_offsets)


def tiny_scene(P: int = 48, width: int = 64, height: int = 48, sh_degree: int = 1, seed: int = 7,
               spread: float = 1.0, log_scale_mean: float = -2.0) -> GaussianScene:
    """Small random scene for brute-force checks; the image size need not be
    a multiple of the 16-pixel tile."""
    g = _gen(seed)
    means = (torch.rand(P, 3, generator=g) * 2 - 1) * spread
    scales = torch.exp(torch.randn(P, 3, generator=g) * 0.6 + log_scale_mean)
    rots = _unit_quats(P, g)
    opac = torch.sigmoid(torch.randn(P, 1, generator=g) * 1.5 + 0.5)
    shs = _shs(P, sh_degree, g)
    fov = math.radians(60.0)
    cam = Camera.look_at([0.3, -0.2, -3.0], [0.0, 0.0, 0.0], [0.0, -1.0, 0.0], width, height, fov)
    return GaussianScene("tiny", means, scales, rots, opac, shs, sh_degree, [cam], torch.tensor([0.1, 0.2, 0.3]))


BY_INDEX = {1: config1, 2: config2, 3: config3, 4: config4, 5: config5}
