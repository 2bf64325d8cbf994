"""MI355X-native forward renderer for LandMarkSystem's 3D Gaussian Splatting path.

Exports the rasterizer API of the reference's `opt_gaussian_rasterization`
package (see rasterizer.py), backed by hand-written gfx950 HIP kernels behind
the C ABI of include/gs355.h.
"""
from .rasterizer import GaussianRasterizationSettings, GaussianRasterizer  # noqa: F401

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer"]
