"""Camera record and matrix conventions that feed the rasterizer.

Restates the reference's conventions so that synthetic cameras produce the
same `viewmatrix` / `projmatrix` / `campos` a LandMarkSystem dataset would:
  - getWorld2View2, getProjectionMatrix, fov2focal, focal2fov:
    landmark/nerf_components/utils/graphics_utils.py:43-85
  - world_view_transform = W2C^T, full_proj_transform = world_view @ P^T,
    camera_center = inverse(world_view)[3,:3]:
    landmark/nerf_components/data/datasets/dataloader/colmap_dataset.py:137-151
  - the fields the renderer reads from a Camera:
    landmark/nerf_components/data/cameras.py:34-108
"""
import math
from dataclasses import dataclass, replace
from typing import Optional

import numpy as np
import torch


def fov2focal(fov: float, pixels: float) -> float:
    return pixels / (2.0 * math.tan(fov / 2.0))


def focal2fov(focal: float, pixels: float) -> float:
    return 2.0 * math.atan(pixels / (2.0 * focal))


def get_world2view2(R, t, translate=(0.0, 0.0, 0.0), scale: float = 1.0) -> np.ndarray:
    """World-to-camera 4x4 (float32).  `R` is stored transposed, as in the
    reference's loaders: W2C[:3,:3] = R^T, W2C[:3,3] = t."""
    Rt = np.zeros((4, 4), dtype=np.float64)
    Rt[:3, :3] = np.asarray(R, dtype=np.float64).T
    Rt[:3, 3] = np.asarray(t, dtype=np.float64)
    Rt[3, 3] = 1.0
    c2w = np.linalg.inv(Rt)
    c2w[:3, 3] = (c2w[:3, 3] + np.asarray(translate, dtype=np.float64)) * scale
    return np.linalg.inv(c2w).astype(np.float32)


def get_projection_matrix(znear: float, zfar: float, fovX: float, fovY: float) -> torch.Tensor:
    """Perspective matrix P (not yet transposed); the only entries the
    rasterizer depends on are P[0,0], P[1,1] and the w row."""
    tan_y = math.tan(fovY / 2.0)
    tan_x = math.tan(fovX / 2.0)
    top, right = tan_y * znear, tan_x * znear
    bottom, left = -top, -right
    P = torch.zeros(4, 4)
    P[0, 0] = 2.0 * znear / (right - left)
    P[1, 1] = 2.0 * znear / (top - bottom)
    P[0, 2] = (right + left) / (right - left)
    P[1, 2] = (top + bottom) / (top - bottom)
    P[3, 2] = 1.0
    P[2, 2] = zfar / (zfar - znear)
    P[2, 3] = -(zfar * znear) / (zfar - znear)
    return P


@dataclass
class Camera:
    """The subset of the reference's Camera that GS rendering reads."""

    width: int
    height: int
    FovX: float
    FovY: float
    world_view_transform: torch.Tensor  # [4,4] = W2C^T
    projection_matrix: torch.Tensor  # [4,4] = P^T
    full_proj_transform: torch.Tensor  # [4,4]
    camera_center: torch.Tensor  # [3]
    znear: float = 0.01
    zfar: float = 100.0
    resolution_scale: float = 1.0

    @property
    def device(self):
        return self.world_view_transform.device

    def to(self, device):
        device = torch.device(device)
        if device == self.device:
            return self
        return replace(
            self,
            world_view_transform=self.world_view_transform.to(device),
            projection_matrix=self.projection_matrix.to(device),
            full_proj_transform=self.full_proj_transform.to(device),
            camera_center=self.camera_center.to(device),
        )

    def cuda(self):
        return self.to(torch.device("cuda", torch.cuda.current_device()))

    def cpu(self):
        return self.to("cpu")

    @staticmethod
    def from_world2cam(R, T, width: int, height: int, FovX: float, FovY: Optional[float] = None,
                       znear: float = 0.01, zfar: float = 100.0) -> "Camera":
        """Build from the reference's (R, T) pair: R is camera-to-world
        rotation (W2C[:3,:3] = R^T), T the world-to-camera translation."""
        if FovY is None:
            FovY = focal2fov(fov2focal(FovX, width), height)
        wv = torch.tensor(get_world2view2(R, T)).transpose(0, 1).contiguous()
        proj = get_projection_matrix(znear, zfar, FovX, FovY).transpose(0, 1).contiguous()
        full = (wv.unsqueeze(0).bmm(proj.unsqueeze(0))).squeeze(0).contiguous()
        center = wv.inverse()[3, :3].contiguous()
        return Camera(int(width), int(height), float(FovX), float(FovY), wv, proj, full, center, znear, zfar)

    @staticmethod
    def look_at(eye, target, up, width: int, height: int, FovX: float, FovY: Optional[float] = None,
                znear: float = 0.01, zfar: float = 100.0) -> "Camera":
        """Pinhole camera at `eye` looking at `target` (+z forward, +x right,
        +y down in view space, the COLMAP axes the reference uses)."""
        eye = np.asarray(eye, dtype=np.float64)
        fwd = np.asarray(target, dtype=np.float64) - eye
        fwd /= np.linalg.norm(fwd)
        upv = np.asarray(up, dtype=np.float64)
        right = np.cross(fwd, upv)
        right /= np.linalg.norm(right)
        down = np.cross(fwd, right)
        c2w_rot = np.stack([right, down, fwd], axis=1)  # columns = camera axes in world
        T = -c2w_rot.T @ eye
        return Camera.from_world2cam(c2w_rot, T, width, height, FovX, FovY, znear, zfar)
