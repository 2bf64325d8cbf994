"""Import-name shim: the reference's models do
`from opt_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer`
(benchmarks/nerf/origin_gs/gs_model.py:5); with this repository on sys.path that
import resolves to the MI355X implementation."""
from landmarksystem_amd.rasterizer import GaussianRasterizationSettings, GaussianRasterizer  # noqa: F401

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer"]
