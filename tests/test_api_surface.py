"""The drop-in Python surface: same names, fields and error behaviour as the
package the reference's models import (benchmarks/nerf/origin_gs/gs_model.py:5,
82-97, 148-162, 211-220, 297-329)."""
import pytest
import torch
from torch import nn


def test_import_names_match_the_reference_package():
    import opt_gaussian_rasterization as ogr
    import landmarksystem_amd as lm

    assert ogr.GaussianRasterizer is lm.GaussianRasterizer
    assert ogr.GaussianRasterizationSettings is lm.GaussianRasterizationSettings


def test_settings_accept_the_reference_placeholders():
    from opt_gaussian_rasterization import GaussianRasterizationSettings

    # exactly the construction at origin_gs/gs_model.py:82-95
    s = GaussianRasterizationSettings(
        image_height=0, image_width=0, tanfovx=0, tanfovy=0, bg=torch.Tensor([0, 0, 0]), scale_modifier=0,
        viewmatrix=torch.Tensor([]), projmatrix=torch.Tensor([]), sh_degree=0, campos=torch.Tensor([]),
        prefiltered=False, debug=False,
    )
    assert s._fields == ("image_height", "image_width", "tanfovx", "tanfovy", "bg", "scale_modifier", "viewmatrix",
                         "projmatrix", "sh_degree", "campos", "prefiltered", "debug")
    with pytest.raises(TypeError):
        GaussianRasterizationSettings(image_height=1)  # all 12 fields are required, as upstream


def test_rasterizer_is_a_stateless_module_child():
    from opt_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer

    s = GaussianRasterizationSettings(0, 0, 0, 0, torch.zeros(3), 0, torch.Tensor([]), torch.Tensor([]), 0,
                                      torch.Tensor([]), False, False)

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.renderer = GaussianRasterizer(raster_settings=s)
            self.w = nn.Parameter(torch.zeros(2))

    m = Model()
    assert list(m.state_dict().keys()) == ["w"]  # the rasterizer adds no parameters or buffers
    assert list(m.renderer.parameters()) == [] and list(m.renderer.buffers()) == []
    m.eval()
    m.to("cpu")
    s2 = s._replace(image_height=8, image_width=8)
    m.renderer.raster_settings = s2  # plain attribute, re-assigned every frame
    assert m.renderer.raster_settings.image_height == 8


def test_exclusive_inputs_raise_like_upstream():
    from opt_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer

    s = GaussianRasterizationSettings(16, 16, 0.5, 0.5, torch.zeros(3), 1.0, torch.eye(4), torch.eye(4), 0,
                                      torch.zeros(3), False, False)
    r = GaussianRasterizer(s)
    P = 4
    m, o = torch.zeros(P, 3), torch.ones(P, 1)
    sh, col = torch.zeros(P, 1, 3), torch.zeros(P, 3)
    sc, rot, cov = torch.ones(P, 3), torch.zeros(P, 4), torch.zeros(P, 6)
    with pytest.raises(Exception, match="SHs or precomputed colors"):
        r(means3D=m, means2D=None, shs=None, colors_precomp=None, opacities=o, scales=sc, rotations=rot,
          cov3D_precomp=None)
    with pytest.raises(Exception, match="SHs or precomputed colors"):
        r(means3D=m, means2D=None, shs=sh, colors_precomp=col, opacities=o, scales=sc, rotations=rot,
          cov3D_precomp=None)
    with pytest.raises(Exception, match="scale/rotation pair or precomputed 3D covariance"):
        r(means3D=m, means2D=None, shs=sh, colors_precomp=None, opacities=o, scales=None, rotations=None,
          cov3D_precomp=None)
    with pytest.raises(Exception, match="scale/rotation pair or precomputed 3D covariance"):
        r(means3D=m, means2D=None, shs=sh, colors_precomp=None, opacities=o, scales=sc, rotations=rot,
          cov3D_precomp=cov)
    with pytest.raises(Exception, match="scale/rotation pair or precomputed 3D covariance"):
        r.visible_filter(means3D=m, scales=None, rotations=None, cov3D_precomp=None)


def test_no_cpu_fallback():
    """CPU tensors are refused loudly: there is no path that avoids the HIP library."""
    from opt_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer

    s = GaussianRasterizationSettings(16, 16, 0.5, 0.5, torch.zeros(3), 1.0, torch.eye(4), torch.eye(4), 0,
                                      torch.zeros(3), False, False)
    r = GaussianRasterizer(s)
    with pytest.raises(ValueError, match="no CPU path"):
        r.visible_filter(means3D=torch.zeros(4, 3), scales=torch.ones(4, 3), rotations=torch.zeros(4, 4),
                         cov3D_precomp=None)


def test_product_never_imports_the_oracle():
    import os
    import re

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for sub in ("landmarksystem_amd", "opt_gaussian_rasterization"):
        for dirpath, _, files in os.walk(os.path.join(root, sub)):
            for f in files:
                if f.endswith((".py", ".hip", ".h", ".cpp")):
                    text = open(os.path.join(dirpath, f)).read()
                    assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), os.path.join(dirpath, f)
                    assert "gs_oracle" not in text, os.path.join(dirpath, f)
