"""Drop-in import name of the reference's rasterizer package
(rasterization_kernels/diff-gaussian-rasterization-half-gaussian/
diff_gaussian_rasterization_half_gaussian/__init__.py), so that
`from diff_gaussian_rasterization_half_gaussian import GaussianRasterizationSettings, GaussianRasterizer`
(gaussian_renderer/render_half_gs.py:3) keeps working unchanged on top of the gfx950 library.
"""
from retinags_amd.rasterizer import (GaussianRasterizationSettings, GaussianRasterizer, _RasterizeGaussians,  # noqa: F401
                                     cpu_deep_copy_tuple, rasterize_gaussians)

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer", "_RasterizeGaussians", "rasterize_gaussians",
           "cpu_deep_copy_tuple"]
