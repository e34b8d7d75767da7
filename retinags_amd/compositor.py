"""Front-to-back compositing of per-submodel partial images, forward and backward, as
one fused HIP pass each.  Host-side mirror of blender_render_result
(parallel_utils/basic_parallel_trainer/result_aggregator.py:193-260): the same ordering
rule (ascending value of the relation vector, negative = not related), the same three
outputs (render, depth, alpha) and the same gradients torch autograd produces for the
reference's cat / cumprod / sum expression.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional, Sequence

import torch

from . import _capi
from ._capi import lib, check, ptr, ptr_table


def _prep(t: torch.Tensor, device, shape) -> torch.Tensor:
    if t.device != device or t.dtype != torch.float32:
        t = t.to(device=device, dtype=torch.float32)
    if tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"partial image plane has shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.contiguous()


class _CompositePartialImages(torch.autograd.Function):
    """apply(background_or_None, K, image_0.., depth_0.., alpha_0..) -> (image, depth, alpha)."""

    @staticmethod
    def forward(ctx, background, K, *planes):
        images, depths, alphas = planes[:K], planes[K:2 * K], planes[2 * K:3 * K]
        device = images[0].device
        if not images[0].is_cuda:
            raise RuntimeError("the compositor needs its inputs on a GPU (device memory)")
        H, W = int(images[0].shape[-2]), int(images[0].shape[-1])
        images = [_prep(t, device, (3, H, W)) for t in images]
        depths = [_prep(t, device, (1, H, W)) for t in depths]
        alphas = [_prep(t, device, (1, H, W)) for t in alphas]
        bg = None if background is None else _prep(background.reshape(-1), device, (3,))
        out_image = torch.empty((3, H, W), dtype=torch.float32, device=device)
        out_depth = torch.empty((1, H, W), dtype=torch.float32, device=device)
        out_alpha = torch.empty((1, H, W), dtype=torch.float32, device=device)
        with torch.cuda.device(device):
            check(lib.rgs_composite_forward(
                K, H, W, ptr_table(images), ptr_table(depths), ptr_table(alphas), ptr(bg), ptr(out_image),
                ptr(out_depth), ptr(out_alpha), C.c_void_p(torch.cuda.current_stream(device).cuda_stream)))
        ctx.set_materialize_grads(False)  # absent depth / alpha gradients come back as None and go down as null pointers
        ctx.K, ctx.hw = K, (H, W)
        ctx.has_bg = bg is not None
        ctx.save_for_backward(*(images + depths + alphas + ([bg] if bg is not None else [])))
        return out_image, out_depth, out_alpha

    @staticmethod
    def backward(ctx, g_image, g_depth, g_alpha):
        K, (H, W) = ctx.K, ctx.hw
        saved = ctx.saved_tensors
        images, depths, alphas = list(saved[:K]), list(saved[K:2 * K]), list(saved[2 * K:3 * K])
        bg = saved[3 * K] if ctx.has_bg else None
        device = images[0].device
        f32 = dict(dtype=torch.float32, device=device)
        g_image = torch.zeros((3, H, W), **f32) if g_image is None else _prep(g_image, device, (3, H, W))
        g_depth = None if g_depth is None else _prep(g_depth, device, (1, H, W))
        g_alpha = None if g_alpha is None else _prep(g_alpha, device, (1, H, W))
        # a layer's three gradients in one (5,H,W) block, the layout of RenderResult.zip_grad
        # (parallel_utils/basic_parallel_trainer/task_utils.py:187-195)
        blocks = [torch.empty((5, H, W), **f32) for _ in range(K)]
        d_images = [b[0:3] for b in blocks]
        d_depths = [b[3:4] for b in blocks]
        d_alphas = [b[4:5] for b in blocks]
        with torch.cuda.device(device):
            check(lib.rgs_composite_backward(
                K, H, W, ptr_table(images), ptr_table(depths), ptr_table(alphas), ptr(bg), ptr(g_image), ptr(g_depth),
                ptr(g_alpha), ptr_table(d_images), ptr_table(d_depths), ptr_table(d_alphas),
                C.c_void_p(torch.cuda.current_stream(device).cuda_stream)))
        # The reference's background is a constant (or a fresh random tensor); it gets no gradient.
        if g_depth is None:
            # no gradient for the composited depth: none for the layers' depths either (their planes of the blocks hold
            # the zeros the kernel wrote); told so, the rasterizer's backward leaves out the terms it would multiply
            return (None, None, *d_images, *([None] * K), *d_alphas)
        return (None, None, *d_images, *d_depths, *d_alphas)


def composite_partial_images(images: Sequence[torch.Tensor], depths: Sequence[torch.Tensor],
                             alphas: Sequence[torch.Tensor], background: Optional[torch.Tensor] = None):
    """Composite K partial images that are already in front-to-back order.
    images[k]: (3,H,W); depths[k], alphas[k]: (1,H,W).  Returns (image, depth, alpha).
    More than MAX_COMPOSITE inputs are folded in groups: compositing is associative in
    (image, depth, alpha) when the inner groups use a black background."""
    K = len(images)
    if K == 0 or len(depths) != K or len(alphas) != K:
        raise RuntimeError("composite_partial_images needs K >= 1 images, depths and alphas")
    images, depths, alphas = list(images), list(depths), list(alphas)
    while len(images) > _capi.MAX_COMPOSITE:
        n = _capi.MAX_COMPOSITE
        img, dep, alp = _CompositePartialImages.apply(None, n, *images[:n], *depths[:n], *alphas[:n])
        images, depths, alphas = [img] + images[n:], [dep] + depths[n:], [alp] + alphas[n:]
    K = len(images)
    return _CompositePartialImages.apply(background, K, *images, *depths, *alphas)


def blender_render_result(render_results: Dict[int, dict], relation_vector, background: Optional[torch.Tensor]):
    """Same contract as the reference function of this name
    (parallel_utils/basic_parallel_trainer/result_aggregator.py:193-260) for one camera on
    one GPU: `render_results` maps submodel id -> {"render","depth","alpha"} (what
    render4renderinfo returns), `relation_vector[model_id]` is the compositing rank of that
    submodel or a negative value when it is not related to the camera.  Returns a dict with
    "render", "depth", "alpha".  A missing background draws a random colour, like the
    reference (:256)."""
    if isinstance(relation_vector, torch.Tensor):
        relation_vector = relation_vector.cpu().numpy()
    related = [(int(relation_vector[m]), m) for m in render_results if relation_vector[m] >= 0]
    num_related = int(sum(1 for v in relation_vector if v >= 0))
    if len(related) != num_related:
        raise RuntimeError("NUM_RELATED mis-match")
    related.sort(key=lambda x: x[0])
    pk = [render_results[m] for _, m in related]
    device = pk[0]["render"].device
    bkg = background if background is not None else torch.rand((3,), device=device)
    image, depth, alpha = composite_partial_images([p["render"] for p in pk], [p["depth"] for p in pk],
                                                   [p["alpha"] for p in pk], bkg)
    return {"render": image, "depth": depth, "alpha": alpha}


def partial_image_package(render: torch.Tensor, depth: torch.Tensor, alpha: torch.Tensor) -> torch.Tensor:
    """The (5,H,W) tensor in which the reference ships a partial image or its gradient between ranks
    (RenderResult.zip_content / zip_grad, parallel_utils/basic_parallel_trainer/task_utils.py:156-163,
    187-195): colour, depth, alpha stacked.  The rasterizer and the compositor's backward of this
    package already write the three into one such block, so this returns that block itself when it is
    given them (no copy), and concatenates otherwise."""
    base = render._base
    if (base is not None and depth._base is base and alpha._base is base and tuple(base.shape) == (5,) + tuple(render.shape[1:])
            and base.is_contiguous() and render.data_ptr() == base.data_ptr()
            and depth.data_ptr() == base[3:4].data_ptr() and alpha.data_ptr() == base[4:5].data_ptr()):
        return base.detach()
    with torch.no_grad():
        return torch.cat([render, depth, alpha], dim=0).to(dtype=torch.float32)


def unpack_partial_image(package: torch.Tensor):
    """Views of a (5,H,W) package: colour (3,H,W), depth (1,H,W), alpha (1,H,W)
    (RenderResult.unzip_content / unzip_grad, task_utils.py:176-185, 206-214, without the copies)."""
    if package.dim() != 3 or package.shape[0] != 5:
        raise RuntimeError("a partial-image package has shape (5, H, W)")
    return package[0:3], package[3:4], package[4:5]
