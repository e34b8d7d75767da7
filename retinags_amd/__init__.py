"""MI355X-native (gfx950) half-Gaussian rasterizer and partial-image compositor.

`retinags_amd.rasterizer` mirrors the reference's
`diff_gaussian_rasterization_half_gaussian` module; `retinags_amd.compositor` mirrors the
compositing step of its result aggregator.  `retinags_amd.activation` (stored parameters to renderer inputs), `retinags_amd.sharing` (boundary straddlers),
`retinags_amd.loss` (L1 + SSIM) and `retinags_amd.optimizer` (Adam) cover the steps either side of
them.  All drive librgs_gfx950.so through ctypes.
"""
from .rasterizer import (GaussianRasterizationSettings, GaussianRasterizer, _RasterizeGaussians,  # noqa: F401
                         rasterize_gaussians)
from .compositor import blender_render_result, composite_partial_images  # noqa: F401
from .sharing import SharedGSInfo, merge_shared, select_straddlers  # noqa: F401
from .activation import activate_gaussians  # noqa: F401
from .loss import l1_loss, l1_ssim_loss, ssim  # noqa: F401
from .optimizer import Adam  # noqa: F401

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer", "_RasterizeGaussians", "rasterize_gaussians",
           "blender_render_result", "composite_partial_images", "SharedGSInfo", "select_straddlers", "merge_shared",
           "activate_gaussians", "l1_ssim_loss", "l1_loss", "ssim", "Adam"]
