"""Host-side mirror of the reference's rasterizer module
(K/diff_gaussian_rasterization_half_gaussian/__init__.py with
K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian): the same
names, argument order, return values and error behaviour, driving PyTorch-ROCm
tensors through the C ABI of librgs_gfx950.so instead of a pybind extension.

PyTorch only provides device memory and the current stream here; every stage of
the rasterizer runs in the HIP library.
"""
from __future__ import annotations

import ctypes as C
import math
import threading
from typing import NamedTuple

import torch
import torch.nn as nn

from . import _capi
from ._capi import lib, check, ptr


def cpu_deep_copy_tuple(input_tuple):
    copied_tensors = [item.cpu().clone() if isinstance(item, torch.Tensor) else item for item in input_tuple]
    return tuple(copied_tensors)


class GaussianRasterizationSettings(NamedTuple):
    """K/diff_gaussian_rasterization_half_gaussian/__init__.py:166-181, field for field."""
    image_height: int
    image_width: int
    tanfovx: float
    tanfovy: float
    bg: torch.Tensor
    scale_modifier: float
    viewmatrix: torch.Tensor
    projmatrix: torch.Tensor
    projmatrix_inv: torch.Tensor
    range_low: torch.Tensor
    range_up: torch.Tensor
    sh_degree: int
    campos: torch.Tensor
    prefiltered: bool
    debug: bool


_pinned_words = threading.local()


def _pinned_word(device: torch.device) -> torch.Tensor:
    """One pinned uint32 per host thread and device: the landing spot of the instance count of a
    call that waits for it.  The count is copied out before the call returns, so calls of one
    thread can share the word; another thread has its own."""
    words = _pinned_words.__dict__.setdefault("words", {})
    key = (device.type, device.index)
    t = words.get(key)
    if t is None:
        t = torch.zeros(1, dtype=torch.int32).pin_memory()
        words[key] = t
    return t


def _dev_f32(t: torch.Tensor, device, name: str) -> torch.Tensor:
    """Contiguous fp32 tensor on `device`; the reference calls .contiguous() on every
    argument (K/rasterize_points.cu:99-121)."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if t.numel() == 0:
        return t
    if t.device != device or t.dtype != torch.float32:
        t = t.to(device=device, dtype=torch.float32)
    return t.contiguous()


def _stream_ptr(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


class GeometryStage:
    """What the first half of a forward call leaves behind: the geometry workspace, the
    radii and the place where the instance count lands.  Produced by
    GaussianRasterizer.enqueue_geometry, consumed once by GaussianRasterizer.forward."""

    __slots__ = ("device", "stream", "P", "H", "W", "tensors", "settings", "radii", "geomBuffer", "geom_bytes",
                 "count", "event", "source", "used", "instance_bound", "_instances")

    def matches(self, means3D, raster_settings) -> bool:
        return (self.source == (means3D.data_ptr(), int(means3D.shape[0])) and self.settings is raster_settings
                and not self.used)

    def instances(self) -> int:
        """The number of (Gaussian, tile) instances of this call; waits for it if it is still on
        its way.  A stage that was given an instance_bound must be asked once its forward has
        been issued: a count above the bound means the images of that forward are wrong."""
        if self._instances is None:
            if self.count is None:
                raise RuntimeError("the instance count of this stage has been handed on already")
            if self.event is not None:
                self.event.synchronize()
                self._instances = int(self.count.item())
                _free_count_slots.setdefault((self.device.type, self.device.index), []).append((self.count, self.event))
                self.event = None
            else:
                self._instances = int(self.count.item())
            self.count = None
        return self._instances

    def within_bound(self) -> bool:
        return self.instance_bound is None or self.P == 0 or self.instances() <= self.instance_bound


_EMPTY = torch.Tensor([])  # stands for an absent input, as in the reference (it becomes a null pointer)

_free_count_slots = {}   # per device: (pinned word, event) pairs of finished calls, for reuse


def _new_count_slot(device):
    """A pinned word for an instance count and the event that says it has arrived."""
    event = torch.cuda.Event()
    event.record(torch.cuda.current_stream(device))  # the first record creates the hipEvent_t
    return torch.zeros(1, dtype=torch.int32).pin_memory(), event



def _forward_geometry(bg, means3D, colors_precomp, opacities, scales, rotations, scale_modifier, cov3Ds_precomp,
                      viewmatrix, projmatrix, projmatrix_inv, range_low, range_up, tanfovx, tanfovy, image_height,
                      image_width, sh, sh_degree, campos, prefiltered, debug, wait=True):
    """First half of RasterizeGaussiansCUDA_hgs (K/rasterize_points.cu:35-125): argument checks,
    the geometry workspace, per-Gaussian preprocess and the instance count.  With wait=False the
    count is still on its way when this returns."""
    if means3D.ndim != 2 or means3D.shape[1] != 3:
        raise RuntimeError("means3D must have dimensions (num_points, 3)")
    if not means3D.is_cuda:
        raise RuntimeError("the rasterizer needs its inputs on a GPU (device memory)")
    device = means3D.device
    st = GeometryStage()
    st.device = device
    st.source = (means3D.data_ptr(), int(means3D.shape[0]))
    st.used = False
    st.P, st.H, st.W = int(means3D.shape[0]), int(image_height), int(image_width)
    st.stream = torch.cuda.current_stream(device).cuda_stream
    st.settings = None
    st.event = None
    st.count = None
    st.instance_bound = None
    st._instances = None
    byte = dict(dtype=torch.uint8, device=device)
    st.radii = torch.empty((st.P,), dtype=torch.int32, device=device)
    names = ("means3D", "colors_precomp", "opacities", "scales", "rotations", "cov3Ds_precomp", "sh", "bg",
             "viewmatrix", "projmatrix", "projmatrix_inv", "range_low", "range_up", "campos")
    values = (means3D, colors_precomp, opacities, scales, rotations, cov3Ds_precomp, sh, bg, viewmatrix, projmatrix,
              projmatrix_inv, range_low, range_up, campos)
    st.tensors = {n: _dev_f32(v, device, n) for n, v in zip(names, values)}
    st.tensors.update(tanfovx=float(tanfovx), tanfovy=float(tanfovy), debug=int(bool(debug)))
    if st.P == 0:
        st.geomBuffer, st.geom_bytes = torch.empty(0, **byte), 0
        return st
    t = st.tensors
    M = int(t["sh"].shape[1]) if t["sh"].numel() != 0 else 0
    with torch.cuda.device(device):
        st.geom_bytes = lib.rgs_geom_bytes(st.P)
        st.geomBuffer = torch.empty(st.geom_bytes, **byte)
        args = (st.P, int(sh_degree), M, st.W, st.H, ptr(t["means3D"]), ptr(t["sh"]), ptr(t["colors_precomp"]),
                ptr(t["opacities"]), ptr(t["scales"]), float(scale_modifier), ptr(t["rotations"]),
                ptr(t["cov3Ds_precomp"]), ptr(t["viewmatrix"]), ptr(t["projmatrix"]), ptr(t["campos"]),
                float(tanfovx), float(tanfovy), int(bool(prefiltered)), ptr(st.radii), ptr(st.geomBuffer),
                st.geom_bytes)
        if wait:
            word = _pinned_word(device)
            check(lib.rgs_forward_geom(*args, C.c_void_p(word.data_ptr()), C.c_void_p(st.stream),
                                       int(bool(debug))))
            st._instances = int(word.item())   # the call returned with the count in place
        else:
            try:   # list.pop is atomic: two threads never get the same slot
                st.count, st.event = _free_count_slots.setdefault((device.type, device.index), []).pop()
            except IndexError:
                st.count, st.event = _new_count_slot(device)
            check(lib.rgs_forward_geom_enqueue(*args, C.c_void_p(st.count.data_ptr()),
                                               C.c_void_p(st.event.cuda_event), C.c_void_p(st.stream),
                                               int(bool(debug))))
    return st


def _forward_blend(st: GeometryStage):
    """Second half: waits for the instance count if it is still on its way, sizes the binning
    workspace with it, sorts and blends.  Returns the 8-tuple of K/rasterize_points.cu:124."""
    device, P, H, W = st.device, st.P, st.H, st.W
    if st.used:
        raise RuntimeError("this geometry stage has already been consumed")
    st.used = True
    f32 = dict(dtype=torch.float32, device=device)
    byte = dict(dtype=torch.uint8, device=device)
    if torch.cuda.current_stream(device).cuda_stream != st.stream:
        raise RuntimeError("the geometry stage was enqueued on another stream than the one current now")
    # One (5,H,W) block: colour, depth, accumulated alpha in the order in which the reference packs a
    # partial image for transport (RenderResult.zip_content,
    # parallel_utils/basic_parallel_trainer/task_utils.py:156-163); see compositor.partial_image_package.
    package = torch.empty((5, H, W), **f32)
    out_color, out_depth, out_alpha = package[0:3], package[3:4], package[4:5]
    if P == 0:
        out_color.zero_(); out_depth.zero_(); out_alpha.zero_()
        empty = torch.empty(0, **byte)
        return 0, out_color, out_depth, out_alpha, st.radii, empty, empty, empty
    t = st.tensors
    with torch.cuda.device(device):
        image_bytes = lib.rgs_image_bytes(W, H)
        imgBuffer = torch.empty(image_bytes, **byte)
        if st.instance_bound is not None:
            # no wait: the kernels read the count on the device; the caller checks it afterwards
            rendered, raster = int(st.instance_bound), lib.rgs_forward_raster_bounded
        else:
            rendered, raster = st.instances(), lib.rgs_forward_raster
        if rendered >= 1 << 30:
            raise _capi.RgsError(f"{rendered} (Gaussian, tile) instances exceed the 2^30 limit of the sort")
        binning_bytes = lib.rgs_binning_bytes(rendered) if rendered > 0 else 0
        binningBuffer = torch.empty(binning_bytes, **byte)
        check(raster(
            P, rendered, W, H, ptr(t["bg"]), t["tanfovx"], t["tanfovy"], ptr(t["projmatrix_inv"]),
            ptr(t["range_low"]), ptr(t["range_up"]), ptr(t["colors_precomp"]), ptr(st.radii), ptr(st.geomBuffer),
            st.geom_bytes, ptr(binningBuffer), binning_bytes, ptr(imgBuffer), image_bytes, ptr(out_color),
            ptr(out_depth), ptr(out_alpha), C.c_void_p(st.stream), t["debug"]))
    return rendered, out_color, out_depth, out_alpha, st.radii, st.geomBuffer, binningBuffer, imgBuffer


def _rasterize_forward(*args):
    """Counterpart of RasterizeGaussiansCUDA_hgs (K/rasterize_points.cu:35-125): allocates the
    outputs and the three workspaces, runs the forward, returns the same 8-tuple."""
    return _forward_blend(_forward_geometry(*args, wait=True))


def _gradient_outputs(P, M, device, scratch=()):
    """The eight dense gradient tensors of K/rasterize_points.cu:165-174, carved out of one
    uninitialised allocation (the library writes every row of them: those of Gaussians that were
    not rendered as zeros), and the backward's scratch for the per-Gaussian sums in an
    allocation of its own (the library clears it), so that a
    gradient the caller keeps (the means2D gradient, say, for densification statistics) does not
    hold on to the scratch.  The eight do share one block: keeping any of them keeps all (about
    280 bytes per Gaussian with SH degree 3).  `scratch` names those of the eight that the caller
    hands to nobody (the colour gradient when the colours come from SH, the covariance gradient
    when it comes from scale and rotation): they are not made at all (None), and the library
    does not write them."""
    shapes = {"means2D": (P, 3), "opacity": (P, 1), "colors": (P, 3), "means3D": (P, 3), "cov3D": (P, 6),
              "sh": (P, M, 3), "scales": (P, 3), "rotations": (P, 4)}
    order = [k for k in shapes if k not in scratch]
    sizes = {k: (math.prod(v) + 63) // 64 * 64 for k, v in shapes.items()}  # 256-byte aligned parts
    flat = torch.empty((sum(sizes[k] for k in order),), dtype=torch.float32, device=device)
    out, at = {k: None for k in scratch}, 0
    for k in order:
        out[k] = flat[at:at + math.prod(shapes[k])].view(shapes[k])
        at += sizes[k]
    out["sums"] = torch.empty((P, _capi.ACC_FLOATS), dtype=torch.float32, device=device)
    return out


def _rasterize_backward(bg, means3D, radii, colors_precomp, scales, rotations, scale_modifier, cov3Ds_precomp,
                        viewmatrix, projmatrix, projmatrix_inv, range_low, range_up, tanfovx, tanfovy, grad_color,
                        grad_depth, grad_alpha, sh, sh_degree, campos, geomBuffer, num_rendered, binningBuffer,
                        imgBuffer, alpha, debug):
    """Counterpart of RasterizeGaussiansBackwardCUDA_hgs (K/rasterize_points.cu:127-220);
    returns the same 8 tensors in the same order."""
    device = means3D.device
    P = int(means3D.shape[0])
    H, W = int(grad_color.shape[1]), int(grad_color.shape[2])
    M = int(sh.shape[1]) if sh.numel() != 0 else 0
    f32 = dict(dtype=torch.float32, device=device)

    if P == 0:
        z = lambda *s: torch.zeros(s, **f32)
        return z(0, 3), z(0, 3), z(0, 1), z(0, 3), z(0, 6), z(0, M, 3), z(0, 3), z(0, 4)

    means3D = _dev_f32(means3D, device, "means3D")
    colors_precomp = _dev_f32(colors_precomp, device, "colors_precomp")
    scales = _dev_f32(scales, device, "scales")
    rotations = _dev_f32(rotations, device, "rotations")
    cov3Ds_precomp = _dev_f32(cov3Ds_precomp, device, "cov3Ds_precomp")
    sh = _dev_f32(sh, device, "sh")
    grad_color = _dev_f32(grad_color, device, "grad_color")
    grad_depth = _dev_f32(grad_depth, device, "grad_depth")
    grad_alpha = _dev_f32(grad_alpha, device, "grad_alpha")
    alpha = _dev_f32(alpha, device, "alpha")
    bg = _dev_f32(bg, device, "bg")
    viewmatrix = _dev_f32(viewmatrix, device, "viewmatrix")
    projmatrix = _dev_f32(projmatrix, device, "projmatrix")
    projmatrix_inv = _dev_f32(projmatrix_inv, device, "projmatrix_inv")
    range_low = _dev_f32(range_low, device, "range_low")
    range_up = _dev_f32(range_up, device, "range_up")
    campos = _dev_f32(campos, device, "campos")

    out = _gradient_outputs(P, M, device)
    acc = out["sums"]  # scratch rows in which the blend accumulates its per-Gaussian sums
    dL_dmeans2D, dL_dopacity, dL_dcolors = out["means2D"], out["opacity"], out["colors"]
    dL_dmeans3D, dL_dcov3D, dL_dsh = out["means3D"], out["cov3D"], out["sh"]
    dL_dscales, dL_drotations = out["scales"], out["rotations"]

    with torch.cuda.device(device):
        check(lib.rgs_backward(
            P, int(sh_degree), M, int(num_rendered), W, H, ptr(bg), ptr(means3D), ptr(sh), ptr(colors_precomp),
            ptr(alpha), ptr(scales), float(scale_modifier), ptr(rotations), ptr(cov3Ds_precomp), ptr(viewmatrix),
            ptr(projmatrix), ptr(projmatrix_inv), ptr(range_low), ptr(range_up), ptr(campos), float(tanfovx),
            float(tanfovy), ptr(radii), ptr(geomBuffer), ptr(binningBuffer), ptr(imgBuffer), ptr(grad_color),
            ptr(grad_depth), ptr(grad_alpha), ptr(acc), ptr(dL_dmeans2D), ptr(dL_dopacity), ptr(dL_dcolors),
            ptr(dL_dmeans3D), ptr(dL_dcov3D), ptr(dL_dsh),
            ptr(dL_dscales), ptr(dL_drotations), 0, _stream_ptr(device), int(bool(debug))))

    return dL_dmeans2D, dL_dcolors, dL_dopacity, dL_dmeans3D, dL_dcov3D, dL_dsh, dL_dscales, dL_drotations


def _mark_visible(means3D, viewmatrix, projmatrix):
    """Counterpart of markVisible_hgs (K/rasterize_points.cu:222-241)."""
    device = means3D.device
    if not means3D.is_cuda:
        raise RuntimeError("the rasterizer needs its inputs on a GPU (device memory)")
    P = int(means3D.shape[0])
    present = torch.zeros((P,), dtype=torch.bool, device=device)
    if P != 0:
        means3D = _dev_f32(means3D, device, "means3D")
        viewmatrix = _dev_f32(viewmatrix, device, "viewmatrix")
        projmatrix = _dev_f32(projmatrix, device, "projmatrix")
        with torch.cuda.device(device):
            check(lib.rgs_mark_visible(P, ptr(means3D), ptr(viewmatrix), ptr(projmatrix), ptr(present),
                                       _stream_ptr(device)))
    return present


def rasterize_gaussians(means3D, means2D, sh, colors_precomp, opacities, scales, rotations, cov3Ds_precomp,
                        raster_settings, geometry=None):
    return _RasterizeGaussians.apply(means3D, means2D, sh, colors_precomp, opacities, scales, rotations,
                                     cov3Ds_precomp, raster_settings, geometry)


class _RasterizeGaussians(torch.autograd.Function):
    """K/diff_gaussian_rasterization_half_gaussian/__init__.py:44-164."""

    @staticmethod
    def forward(ctx, means3D, means2D, sh, colors_precomp, opacities, scales, rotations, cov3Ds_precomp,
                raster_settings, geometry=None):
        if geometry is not None:
            if not geometry.matches(means3D, raster_settings):
                raise RuntimeError("the geometry stage was enqueued for other inputs or settings, or already used")
            outs = _forward_blend(geometry)
            return _RasterizeGaussians._finish_forward(ctx, outs, raster_settings, colors_precomp, means3D, scales,
                                                       rotations, cov3Ds_precomp, sh)
        args = (
            raster_settings.bg, means3D, colors_precomp, opacities, scales, rotations, raster_settings.scale_modifier,
            cov3Ds_precomp, raster_settings.viewmatrix, raster_settings.projmatrix, raster_settings.projmatrix_inv,
            raster_settings.range_low, raster_settings.range_up, raster_settings.tanfovx, raster_settings.tanfovy,
            raster_settings.image_height, raster_settings.image_width, sh, raster_settings.sh_degree,
            raster_settings.campos, raster_settings.prefiltered, raster_settings.debug,
        )
        if raster_settings.debug:
            cpu_args = cpu_deep_copy_tuple(args)  # copy them before they can be corrupted
            try:
                outs = _rasterize_forward(*args)
            except Exception as ex:
                torch.save(cpu_args, "snapshot_fw.dump")
                print("\nAn error occured in forward. Please forward snapshot_fw.dump for debugging.")
                raise ex
        else:
            outs = _rasterize_forward(*args)
        return _RasterizeGaussians._finish_forward(ctx, outs, raster_settings, colors_precomp, means3D, scales,
                                                   rotations, cov3Ds_precomp, sh)

    @staticmethod
    def _finish_forward(ctx, outs, raster_settings, colors_precomp, means3D, scales, rotations, cov3Ds_precomp, sh):
        num_rendered, color, depth, alpha, radii, geomBuffer, binningBuffer, imgBuffer = outs

        ctx.set_materialize_grads(False)  # an output that took no part in the loss comes back as None, not as a tensor of zeros
        ctx.raster_settings = raster_settings
        ctx.num_rendered = num_rendered
        ctx.save_for_backward(colors_precomp, means3D, scales, rotations, cov3Ds_precomp, radii, sh, geomBuffer,
                              binningBuffer, imgBuffer, alpha)
        ctx.mark_non_differentiable(radii)
        return color, radii, depth, alpha

    @staticmethod
    def backward(ctx, grad_color, grad_radii, grad_depth, grad_alpha):
        num_rendered = ctx.num_rendered
        raster_settings = ctx.raster_settings
        (colors_precomp, means3D, scales, rotations, cov3Ds_precomp, radii, sh, geomBuffer, binningBuffer, imgBuffer,
         alpha) = ctx.saved_tensors

        # Outputs that did not take part in the loss arrive as None.  The reference's C++ side
        # always receives dense tensors; here an absent depth / alpha gradient goes down as a
        # null pointer, which the library takes as zero.
        if grad_color is None:
            grad_color = torch.zeros((3,) + tuple(alpha.shape[1:]), dtype=alpha.dtype, device=alpha.device)
        if grad_depth is None:
            grad_depth = _EMPTY
        if grad_alpha is None:
            grad_alpha = _EMPTY

        args = (raster_settings.bg, means3D, radii, colors_precomp, scales, rotations,
                raster_settings.scale_modifier, cov3Ds_precomp, raster_settings.viewmatrix,
                raster_settings.projmatrix, raster_settings.projmatrix_inv, raster_settings.range_low,
                raster_settings.range_up, raster_settings.tanfovx, raster_settings.tanfovy, grad_color, grad_depth,
                grad_alpha, sh, raster_settings.sh_degree, raster_settings.campos, geomBuffer, num_rendered,
                binningBuffer, imgBuffer, alpha, raster_settings.debug)

        if raster_settings.debug:
            cpu_args = cpu_deep_copy_tuple(args)
            try:
                outs = _rasterize_backward(*args)
            except Exception as ex:
                torch.save(cpu_args, "snapshot_bw.dump")
                print("\nAn error occured in backward. Writing snapshot_bw.dump for debugging.\n")
                raise ex
        else:
            outs = _rasterize_backward(*args)
        (grad_means2D, grad_colors_precomp, grad_opacities, grad_means3D, grad_cov3Ds_precomp, grad_sh, grad_scales,
         grad_rotations) = outs

        grads = (
            grad_means3D,
            grad_means2D,
            grad_sh if sh.numel() else None,
            grad_colors_precomp if colors_precomp.numel() else None,
            grad_opacities,
            grad_scales if scales.numel() else None,
            grad_rotations if rotations.numel() else None,
            grad_cov3Ds_precomp if cov3Ds_precomp.numel() else None,
            None,
            None,
        )
        return grads


class _RasterizeFrame(torch.autograd.Function):
    """The submodels that a camera sees ("layers"), rasterized together: what the reference does with one
    _RasterizeGaussians call per submodel (gather_RenderResult_pool,
    parallel_utils/basic_parallel_trainer/result_aggregator.py:22-38), as three library calls per frame
    (every layer's geometry stage, then binning and one blend launch for all, and for the backward one
    blend launch for all and every layer's per-Gaussian backward).

    apply(settings, streams, workspaces, *flat): `settings` a tuple of K GaussianRasterizationSettings (same
    camera and image size), `streams` None or a tuple of K HIP stream handles (the first that differs from the
    current stream serves the backward as a second stream for its memory-bound work), `workspaces` None or a
    list that receives, per layer, what a single call returns beside its images: (num_rendered, geomBuffer,
    binningBuffer, imgBuffer), flat = for every layer (means3D, means2D, sh, colors_precomp, opacities, scales,
    rotations, cov3Ds_precomp).  Returns for every layer (color, radii, depth, alpha)."""

    FIELDS = 8

    @staticmethod
    def forward(ctx, settings, streams, workspaces, *flat):
        K = len(settings)
        if K == 0 or len(flat) != _RasterizeFrame.FIELDS * K:
            raise RuntimeError("rasterize_frame: one group of eight tensors per layer is needed")
        if K > _capi.MAX_FRAME_LAYERS:
            raise RuntimeError(f"rasterize_frame: at most {_capi.MAX_FRAME_LAYERS} layers")
        rs0 = settings[0]
        H, W = int(rs0.image_height), int(rs0.image_width)
        device = flat[0].device
        if not flat[0].is_cuda:
            raise RuntimeError("the rasterizer needs its inputs on a GPU (device memory)")
        f32 = dict(dtype=torch.float32, device=device)
        byte = dict(dtype=torch.uint8, device=device)
        main = torch.cuda.current_stream(device).cuda_stream
        debug = int(bool(rs0.debug))
        view_t = {n: _dev_f32(v, device, n) for n, v in (("viewmatrix", rs0.viewmatrix), ("projmatrix", rs0.projmatrix),
                                                          ("projmatrix_inv", rs0.projmatrix_inv), ("campos", rs0.campos))}
        view = _capi.FrameView(W, H, float(rs0.tanfovx), float(rs0.tanfovy), ptr(view_t["viewmatrix"]),
                               ptr(view_t["projmatrix"]), ptr(view_t["projmatrix_inv"]), ptr(view_t["campos"]))
        arr = (_capi.FrameLayer * K)()
        records, live = [], []
        with torch.cuda.device(device):
            image_bytes = lib.rgs_image_bytes(W, H)
            for k, rs in enumerate(settings):
                means3D, means2D, sh, colors_precomp, opacities, scales, rotations, cov3Ds = flat[8 * k:8 * k + 8]
                if int(rs.image_height) != H or int(rs.image_width) != W:
                    raise RuntimeError("rasterize_frame: the layers of a frame share one image size")
                if means3D.ndim != 2 or means3D.shape[1] != 3:
                    raise RuntimeError("means3D must have dimensions (num_points, 3)")
                P = int(means3D.shape[0])
                M = int(sh.shape[1]) if sh.numel() != 0 else 0
                package = torch.empty((5, H, W), **f32)
                t = {n: _dev_f32(v, device, n) for n, v in (
                    ("means3D", means3D), ("sh", sh), ("colors_precomp", colors_precomp), ("opacities", opacities),
                    ("scales", scales), ("rotations", rotations), ("cov3Ds_precomp", cov3Ds), ("bg", rs.bg),
                    ("range_low", rs.range_low), ("range_up", rs.range_up))}
                rec = dict(P=P, M=M, t=t, package=package, radii=torch.empty((P,), dtype=torch.int32, device=device),
                           rendered=0, geom=torch.empty(0, **byte), binning=torch.empty(0, **byte), img=torch.empty(0, **byte))
                records.append(rec)
                if P == 0:
                    package.zero_()
                    continue
                L = arr[len(live)]
                live.append(k)
                L.P, L.D, L.M = P, int(rs.sh_degree), M
                L.means3D, L.shs, L.colors_precomp, L.opacities = ptr(t["means3D"]), ptr(t["sh"]), ptr(t["colors_precomp"]), ptr(t["opacities"])
                L.scales, L.rotations, L.cov3D_precomp = ptr(t["scales"]), ptr(t["rotations"]), ptr(t["cov3Ds_precomp"])
                L.scale_modifier = float(rs.scale_modifier)
                L.background, L.range_low, L.range_up = ptr(t["bg"]), ptr(t["range_low"]), ptr(t["range_up"])
                L.radii = ptr(rec["radii"])
                geom_bytes = lib.rgs_geom_bytes(P)
                rec["geom"] = torch.empty(geom_bytes, **byte)
                rec["img"] = torch.empty(image_bytes, **byte)
                L.geom_ws, L.image_ws = ptr(rec["geom"]), ptr(rec["img"])
                L.geom_bytes, L.image_bytes = geom_bytes, image_bytes
                L.out_color, L.out_depth, L.out_alpha = ptr(package[0:3]), ptr(package[3:4]), ptr(package[4:5])
            if live:
                counts = _frame_counts(device, len(live))
                check(lib.rgs_frame_forward_geom(len(live), arr, C.byref(view), C.c_void_p(counts.data_ptr()), C.c_void_p(main), debug))
                got = counts[:len(live)].tolist()
                for j, k in enumerate(live):
                    rec = records[k]
                    rec["rendered"] = int(got[j])
                    binning_bytes = lib.rgs_binning_bytes(rec["rendered"]) if rec["rendered"] > 0 else 0
                    rec["binning"] = torch.empty(binning_bytes, **byte)
                    arr[j].R = rec["rendered"]
                    arr[j].binning_ws, arr[j].binning_bytes = ptr(rec["binning"]), binning_bytes
                check(lib.rgs_frame_forward_raster(len(live), arr, C.byref(view), C.c_void_p(main), debug))
        ctx.set_materialize_grads(False)  # an output that took no part in the loss comes back as None, not as a tensor of zeros
        ctx.settings = settings
        ctx.streams = streams
        ctx.meta = []
        saved, outs = [], []
        for k, rec in enumerate(records):
            t = rec["t"]
            ctx.meta.append(dict(rendered=rec["rendered"]))
            saved += [t["colors_precomp"], t["means3D"], t["scales"], t["rotations"], t["cov3Ds_precomp"], rec["radii"], t["sh"],
                      rec["geom"], rec["binning"], rec["img"], rec["package"][4:5]]
            outs += [rec["package"][0:3], rec["radii"], rec["package"][3:4], rec["package"][4:5]]
        ctx.save_for_backward(*saved)
        ctx.mark_non_differentiable(*[outs[4 * k + 1] for k in range(K)])
        if workspaces is not None:
            workspaces.extend((rec["rendered"], rec["geom"], rec["binning"], rec["img"]) for rec in records)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        settings, streams = ctx.settings, ctx.streams
        K = len(settings)
        saved = ctx.saved_tensors
        rs0 = settings[0]
        H, W = int(rs0.image_height), int(rs0.image_width)
        device = saved[1].device
        main = torch.cuda.current_stream(device).cuda_stream
        arr = (_capi.FrameLayer * K)()
        keep, results, live = [], [], 0
        view = None
        for k in range(K):
            (colors_precomp, means3D, scales, rotations, cov3Ds, radii, sh, geomBuffer, binningBuffer, imgBuffer,
             alpha) = saved[11 * k:11 * (k + 1)]
            rs, meta = settings[k], ctx.meta[k]
            g_color, _, g_depth, g_alpha = grads[4 * k:4 * (k + 1)]
            P = int(means3D.shape[0])
            M = int(sh.shape[1]) if sh.numel() != 0 else 0
            f32 = dict(dtype=torch.float32, device=device)
            if P == 0:
                z = lambda *shape: torch.zeros(shape, **f32)
                results.append((z(0, 3), z(0, 3), z(0, 1), z(0, 3), z(0, 6), z(0, M, 3), z(0, 3), z(0, 4)))
                continue
            if g_color is None:
                g_color = torch.zeros((3, H, W), **f32)
            out = _gradient_outputs(P, M, device, scratch=_frame_scratch(colors_precomp, cov3Ds))
            keep.append(out)   # its scratch rows must outlive the library call below
            t = dict(bg=_dev_f32(rs.bg, device, "bg"), low=_dev_f32(rs.range_low, device, "range_low"),
                     up=_dev_f32(rs.range_up, device, "range_up"), g_color=_dev_f32(g_color, device, "grad_color"),
                     g_depth=None if g_depth is None else _dev_f32(g_depth, device, "grad_depth"),
                     g_alpha=None if g_alpha is None else _dev_f32(g_alpha, device, "grad_alpha"))
            keep.append(t)
            if view is None:
                vt = dict(v=_dev_f32(rs.viewmatrix, device, "viewmatrix"), p=_dev_f32(rs.projmatrix, device, "projmatrix"),
                          pi=_dev_f32(rs.projmatrix_inv, device, "projmatrix_inv"), c=_dev_f32(rs.campos, device, "campos"))
                keep.append(vt)
                view = _capi.FrameView(W, H, float(rs.tanfovx), float(rs.tanfovy), ptr(vt["v"]), ptr(vt["p"]), ptr(vt["pi"]),
                                       ptr(vt["c"]))
            L = arr[live]
            live += 1
            L.P, L.D, L.M, L.R = P, int(rs.sh_degree), M, int(meta["rendered"])
            L.means3D, L.shs, L.colors_precomp = ptr(means3D), ptr(sh), ptr(colors_precomp)
            L.scales, L.rotations, L.cov3D_precomp = ptr(scales), ptr(rotations), ptr(cov3Ds)
            L.scale_modifier = float(rs.scale_modifier)
            L.background, L.range_low, L.range_up = ptr(t["bg"]), ptr(t["low"]), ptr(t["up"])
            L.radii = ptr(radii)
            L.geom_ws, L.binning_ws, L.image_ws = ptr(geomBuffer), ptr(binningBuffer), ptr(imgBuffer)
            L.out_alpha = ptr(alpha)
            L.dL_dpix, L.dL_dpix_depth, L.dL_dalphas = ptr(t["g_color"]), ptr(t["g_depth"]), ptr(t["g_alpha"])
            L.grad_accum = ptr(out["sums"])
            L.dL_dmean2D, L.dL_dopacity, L.dL_dcolor = ptr(out["means2D"]), ptr(out["opacity"]), ptr(out["colors"])
            L.dL_dmean3D, L.dL_dcov3D, L.dL_dsh = ptr(out["means3D"]), ptr(out["cov3D"]), ptr(out["sh"])
            L.dL_dscale, L.dL_drot = ptr(out["scales"]), ptr(out["rotations"])
            L.accum_zeroed = 0   # the library clears the rows of the sums (48 bytes per Gaussian) ahead of the blend
            L.stream = C.c_void_p(streams[k]) if streams is not None and streams[k] != main else C.c_void_p(0)
            results.append((out["means2D"], out["colors"], out["opacity"], out["means3D"], out["cov3D"], out["sh"],
                            out["scales"], out["rotations"]))
        if live:
            with torch.cuda.device(device):
                check(lib.rgs_frame_backward(live, arr, C.byref(view), C.c_void_p(main), int(bool(rs0.debug))))
        flat = []
        for k in range(K):
            (colors_precomp, means3D, scales, rotations, cov3Ds, radii, sh) = saved[11 * k:11 * k + 7]
            g_means2D, g_colors, g_opacity, g_means3D, g_cov3D, g_sh, g_scales, g_rot = results[k]
            flat += [g_means3D, g_means2D, g_sh if sh.numel() else None, g_colors if colors_precomp.numel() else None,
                     g_opacity, g_scales if scales.numel() else None, g_rot if rotations.numel() else None,
                     g_cov3D if cov3Ds.numel() else None]
        return (None, None, None, *flat)


def _frame_scratch(colors_precomp, cov3Ds_precomp):
    """Which gradient arrays of a frame's layer nobody gets to see: see _gradient_outputs."""
    return tuple(name for name, given in (("colors", colors_precomp), ("cov3D", cov3Ds_precomp)) if given.numel() == 0)


_frame_count_words = threading.local()


def _frame_counts(device: torch.device, n: int) -> torch.Tensor:
    """Pinned words for the layers' instance counts, per host thread and device; read before the call returns."""
    words = _frame_count_words.__dict__.setdefault("words", {})
    key = (device.type, device.index)
    t = words.get(key)
    if t is None or t.numel() < n:
        t = torch.zeros(max(n, _capi.MAX_FRAME_LAYERS), dtype=torch.int32).pin_memory()
        words[key] = t
    return t


def rasterize_frame(rasterizers, inputs, streams=None, workspaces=None):
    """All layers of a frame through one call.  `rasterizers`: K GaussianRasterizer (their settings share the
    camera and the image size); `inputs`: K dicts with the keyword arguments of GaussianRasterizer.forward
    (means3D, means2D, opacities, shs / colors_precomp, scales + rotations / cov3D_precomp); `streams`: None,
    or for every layer the handle of a HIP stream; the first that is not the current stream takes memory-bound work
    beside the kernels of the current one: the backward runs the per-Gaussian part of the layers whose blend is done
    on it (the caller's stream waits for it); every forward stage runs on the current stream.  `workspaces`: None, or a
    list that receives per layer (num_rendered, geomBuffer, binningBuffer, imgBuffer), the rest of the 8-tuple a single
    forward call returns (K/rasterize_points.cu:124).  Returns K tuples (color, radii, depth, alpha), the results of K
    forward calls, and differentiates like them."""
    flat = []
    for rz, kw in zip(rasterizers, inputs):
        shs, colors_precomp, scales, rotations, cov3D = GaussianRasterizer._check_and_fill(
            kw.get("shs"), kw.get("colors_precomp"), kw.get("scales"), kw.get("rotations"), kw.get("cov3D_precomp"))
        flat += [kw["means3D"], kw["means2D"], shs, colors_precomp, kw["opacities"], scales, rotations, cov3D]
    outs = _RasterizeFrame.apply(tuple(rz.raster_settings for rz in rasterizers),
                                 None if streams is None else tuple(streams), workspaces, *flat)
    return [tuple(outs[4 * k:4 * k + 4]) for k in range(len(rasterizers))]


class GaussianRasterizer(nn.Module):
    """K/diff_gaussian_rasterization_half_gaussian/__init__.py:183-232."""

    def __init__(self, raster_settings):
        super().__init__()
        self.raster_settings = raster_settings

    def markVisible(self, positions):
        # Mark visible points (based on frustum culling for camera) with a boolean
        with torch.no_grad():
            raster_settings = self.raster_settings
            visible = _mark_visible(positions, raster_settings.viewmatrix, raster_settings.projmatrix)
        return visible

    @staticmethod
    def _check_and_fill(shs, colors_precomp, scales, rotations, cov3D_precomp):
        if (shs is None and colors_precomp is None) or (shs is not None and colors_precomp is not None):
            raise Exception('Please provide excatly one of either SHs or precomputed colors!')

        if ((scales is None or rotations is None) and cov3D_precomp is None) or \
                ((scales is not None or rotations is not None) and cov3D_precomp is not None):
            raise Exception('Please provide exactly one of either scale/rotation pair or precomputed 3D covariance!')

        if shs is None:
            shs = _EMPTY
        if colors_precomp is None:
            colors_precomp = _EMPTY
        if scales is None:
            scales = _EMPTY
        if rotations is None:
            rotations = _EMPTY
        if cov3D_precomp is None:
            cov3D_precomp = _EMPTY
        return shs, colors_precomp, scales, rotations, cov3D_precomp

    def forward(self, means3D, means2D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
                cov3D_precomp=None, geometry=None):
        """As the reference's forward.  `geometry`, if given, is what enqueue_geometry returned for
        these same inputs: the call then only waits for that stage and goes on from there."""
        raster_settings = self.raster_settings
        shs, colors_precomp, scales, rotations, cov3D_precomp = self._check_and_fill(
            shs, colors_precomp, scales, rotations, cov3D_precomp)
        return rasterize_gaussians(means3D, means2D, shs, colors_precomp, opacities, scales, rotations, cov3D_precomp,
                                   raster_settings, geometry)

    def enqueue_geometry(self, means3D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
                         cov3D_precomp=None, instance_bound=None) -> GeometryStage:
        """Starts the first half of a forward call (preprocess and instance count) on the current
        stream and returns without waiting for it.  No counterpart in the reference, whose forward
        always blocks on the count (K/cuda_rasterizer_hgs/rasterizer_impl.cu:287): a caller that
        renders several submodels on separate streams enqueues every geometry stage first and
        then calls forward(..., geometry=stage) for each, on the stream the stage was enqueued
        on, so that the host's wait for one count no longer holds back the other submodels.

        instance_bound: room for that many (Gaussian, tile) instances is set aside and the forward
        does not wait for the count at all (the reference grows its buffers on demand instead,
        K/rasterize_points.cu:27-33).  The caller must then ask stage.within_bound() after the
        forward has been issued (at the end of the iteration is early enough) and, if it is
        false, repeat the forward with a bound of at least stage.instances()."""
        rs = self.raster_settings
        shs, colors_precomp, scales, rotations, cov3D_precomp = self._check_and_fill(
            shs, colors_precomp, scales, rotations, cov3D_precomp)
        with torch.no_grad():
            stage = _forward_geometry(
                rs.bg, means3D, colors_precomp, opacities, scales, rotations, rs.scale_modifier, cov3D_precomp,
                rs.viewmatrix, rs.projmatrix, rs.projmatrix_inv, rs.range_low, rs.range_up, rs.tanfovx, rs.tanfovy,
                rs.image_height, rs.image_width, shs, rs.sh_degree, rs.campos, rs.prefiltered, rs.debug, wait=False)
        stage.settings = rs
        if instance_bound is not None:
            if int(instance_bound) < 0:
                raise ValueError("instance_bound must not be negative")
            stage.instance_bound = int(instance_bound)
        return stage
