"""From a submodel's stored parameters to the tensors its renderer and neighbours see, in one kernel
each way (rgs_activate_forward / rgs_activate_backward, include/rgs.h): what the get_* properties of
the reference's Gaussian model compute with one tensor operation each
(scene/gaussian_nn_module.py:373-394)."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ._capi import check, lib, ptr
from .sharing import SharedGSInfo


def _stream(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _rows_with_room(n: int, width, spare: int, device) -> torch.Tensor:
    """An (n, *width) tensor at the start of an allocation of n + spare rows."""
    room = torch.empty((n + spare,) + tuple(width), dtype=torch.float32, device=device)
    if spare == 0:
        return room
    return torch.empty(0, dtype=torch.float32, device=device).set_(room.untyped_storage(), 0, (n,) + tuple(width),
                                                                   room.stride())


class _Activate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, features_dc, features_rest, scaling, rotation, opacity, spare_rows: int):
        tensors = [features_dc, features_rest, scaling, rotation, opacity]
        for t in tensors:
            if not t.is_cuda:
                raise RuntimeError("activation runs on the GPU only: the parameters must be device tensors")
        features_dc, features_rest, scaling, rotation, opacity = (t.contiguous().float() for t in tensors)
        n, rest = int(features_dc.shape[0]), int(features_rest.shape[1])
        if tuple(features_dc.shape[1:]) != (1, 3) or tuple(features_rest.shape) != (n, rest, 3):
            raise RuntimeError("features_dc must be (N,1,3) and features_rest (N,R,3)")
        if tuple(scaling.shape) != (n, 3) or tuple(rotation.shape) != (n, 4) or tuple(opacity.shape) != (n, 1):
            raise RuntimeError("scaling (N,3), rotation (N,4), opacity (N,1) expected")
        device = features_dc.device
        shs = _rows_with_room(n, (1 + rest, 3), spare_rows, device)
        scales = _rows_with_room(n, (3,), spare_rows, device)
        rotations = _rows_with_room(n, (4,), spare_rows, device)
        opacities = _rows_with_room(n, (1,), spare_rows, device)
        check(lib.rgs_activate_forward(n, rest, ptr(features_dc), ptr(features_rest), ptr(scaling), ptr(rotation),
                                       ptr(opacity), ptr(shs), ptr(scales), ptr(rotations), ptr(opacities),
                                       _stream(device)))
        ctx.save_for_backward(rotation, scales, opacities)
        ctx.sizes = (n, rest)
        ctx.set_materialize_grads(False)   # an output outside the loss arrives as None and costs nothing
        return shs, scales, rotations, opacities

    @staticmethod
    def backward(ctx, g_shs, g_scales, g_rotations, g_opacities):
        rotation, scales, opacities = ctx.saved_tensors
        n, rest = ctx.sizes
        device = rotation.device
        prep = lambda g: None if g is None else g.contiguous().float()
        g_shs, g_scales, g_rotations, g_opacities = prep(g_shs), prep(g_scales), prep(g_rotations), prep(g_opacities)
        new = lambda g, *shape: None if g is None else torch.empty(shape, dtype=torch.float32, device=device)
        d_dc, d_rest = new(g_shs, n, 1, 3), new(g_shs, n, rest, 3)
        d_scaling, d_rotation, d_opacity = new(g_scales, n, 3), new(g_rotations, n, 4), new(g_opacities, n, 1)
        check(lib.rgs_activate_backward(n, rest, ptr(rotation), ptr(scales), ptr(opacities), ptr(g_shs), ptr(g_scales),
                                        ptr(g_rotations), ptr(g_opacities), ptr(d_dc), ptr(d_rest), ptr(d_scaling),
                                        ptr(d_rotation), ptr(d_opacity), _stream(device)))
        return d_dc, d_rest, d_scaling, d_rotation, d_opacity, None


def activate_gaussians(xyz: torch.Tensor, features_dc: torch.Tensor, features_rest: torch.Tensor, scaling: torch.Tensor,
                       rotation: torch.Tensor, opacity: torch.Tensor, means2D: Optional[torch.Tensor] = None,
                       spare_rows: int = 0) -> SharedGSInfo:
    """The SharedGSInfo that gather_local_SharedGSInfo builds from a model's properties
    (parallel_utils/basic_parallel_trainer/result_aggregator.py:40-52).  means3D is xyz itself, as
    in the reference; means2D is the caller's screen-space placeholder (zeros if absent).
    spare_rows: room behind every activated tensor, which sharing.merge_shared(append=True) needs
    (xyz and means2D must then bring their own)."""
    shs, scales, rotations, opacities = _Activate.apply(features_dc, features_rest, scaling, rotation, opacity,
                                                        int(spare_rows))
    if means2D is None:
        means2D = _rows_with_room(int(xyz.shape[0]), (3,), int(spare_rows), xyz.device).zero_()
        means2D.requires_grad_(xyz.requires_grad)
    return SharedGSInfo(xyz, means2D, opacities, scales, rotations, shs)
