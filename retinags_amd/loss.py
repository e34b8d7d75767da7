"""Image loss of a training iteration on the GPU: (1 - lambda) L1 + lambda (1 - SSIM) with its
gradient in two kernels (rgs_l1_ssim_forward / rgs_l1_ssim_backward, include/rgs.h), under the
names of the reference's utils/loss_utils.py."""
from __future__ import annotations

import ctypes as C
from typing import Tuple

import torch

from ._capi import check, lib, ptr


def _stream(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _as_planes(image: torch.Tensor, gt: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, int, int, int]:
    if image.shape != gt.shape:
        raise RuntimeError(f"image {tuple(image.shape)} and ground truth {tuple(gt.shape)} differ in shape")
    if image.dim() not in (3, 4):
        raise RuntimeError("expected (C,H,W) or (B,C,H,W) images")
    if not image.is_cuda or not gt.is_cuda:
        raise RuntimeError("the loss runs on the GPU only: both images must be device tensors")
    image = image.contiguous().float()
    gt = gt.contiguous().float()
    H, W = int(image.shape[-2]), int(image.shape[-1])
    planes = int(image.numel() // (H * W))   # batch and channel planes are windowed independently
    return image, gt, planes, H, W


class _L1SSIM(torch.autograd.Function):
    @staticmethod
    def forward(ctx, image: torch.Tensor, gt: torch.Tensor, lambda_dssim: float):
        x, y, planes, H, W = _as_planes(image, gt)
        keep = bool(ctx.needs_input_grad[0])
        workspace = torch.empty(lib.rgs_loss_workspace_bytes(planes, H, W), dtype=torch.uint8, device=x.device)
        out = torch.empty(3, device=x.device)
        check(lib.rgs_l1_ssim_forward(planes, H, W, ptr(x), ptr(y), float(lambda_dssim), ptr(out), ptr(workspace),
                                      1 if keep else 0, _stream(x.device)))
        ctx.save_for_backward(x, y, workspace)
        ctx.lambda_dssim = float(lambda_dssim)
        ctx.shape = tuple(image.shape)
        ctx.mark_non_differentiable(out)
        return out[0], out
    @staticmethod
    def backward(ctx, grad_loss, _):
        x, y, workspace = ctx.saved_tensors
        H, W = int(x.shape[-2]), int(x.shape[-1])
        planes = int(x.numel() // (H * W))
        d_image = torch.empty_like(x)
        g = grad_loss.contiguous().float()
        check(lib.rgs_l1_ssim_backward(planes, H, W, ptr(x), ptr(y), ctx.lambda_dssim, ptr(g), ptr(workspace),
                                       ptr(d_image), _stream(x.device)))
        return d_image.view(ctx.shape), None, None


def l1_ssim_loss(image: torch.Tensor, gt: torch.Tensor, lambda_dssim: float = 0.2) -> Tuple[torch.Tensor, torch.Tensor]:
    """(loss, Ll1) of loss_local (parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:
    449-450): loss = (1 - lambda_dssim) * l1_loss + lambda_dssim * (1 - ssim); differentiable in
    `image`.  Ll1 is returned for logging, detached."""
    loss, parts = _L1SSIM.apply(image, gt, lambda_dssim)
    return loss, parts[1]


def l1_loss(network_output: torch.Tensor, gt: torch.Tensor) -> torch.Tensor:
    """utils/loss_utils.py:17-18 (value only; train through l1_ssim_loss)."""
    with torch.no_grad():
        return _L1SSIM.apply(network_output, gt, 0.0)[1][1]


def ssim(img1: torch.Tensor, img2: torch.Tensor) -> torch.Tensor:
    """utils/loss_utils.py:39-63 with its defaults (window 11, mean over everything); value only."""
    with torch.no_grad():
        return _L1SSIM.apply(img1, img2, 1.0)[1][2]
