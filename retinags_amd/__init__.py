"""MI355X-native (gfx950) half-Gaussian rasterizer and partial-image compositor.

`retinags_amd.rasterizer` mirrors the reference's
`diff_gaussian_rasterization_half_gaussian` module; `retinags_amd.compositor` mirrors the
compositing step of its result aggregator.  Both drive librgs_gfx950.so through ctypes.
"""
from .rasterizer import (GaussianRasterizationSettings, GaussianRasterizer, _RasterizeGaussians,  # noqa: F401
                         rasterize_gaussians)
from .compositor import blender_render_result, composite_partial_images  # noqa: F401

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer", "_RasterizeGaussians", "rasterize_gaussians",
           "blender_render_result", "composite_partial_images"]
