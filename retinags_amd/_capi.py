"""ctypes binding of librgs_gfx950.so (declarations: include/rgs.h).

The library is the only implementation: if it is missing, importing this module
fails with instructions to build it; nothing falls back to another code path.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# RGS_LIBRARY selects another build of the same library (used when comparing kernel variants)
LIB_PATH = os.environ.get("RGS_LIBRARY") or os.path.join(_HERE, "librgs_gfx950.so")

GEOM_FIELDS = ("depths", "tiles_touched", "point_offsets",
               "clamped", "block_sums", "total", "blend_record", "depth_order", "block_visible", "visible_count",
               "order_scratch")
BIN_FIELDS = ("keys_unsorted", "keys_sorted", "values_unsorted", "values_sorted", "sort_temp", "strip_lists")
IMG_FIELDS = ("ranges", "n_contrib", "strip_filed", "strip_order", "strip_total", "strip_order_forward")
ACC_FLOATS = 12
MAX_COMPOSITE = 64
MAX_SHARE_BOXES = 64


class SharedRows(C.Structure):
    """rgs_shared_rows of include/rgs.h."""
    _fields_ = [("means3D", C.c_void_p), ("opacity", C.c_void_p), ("scales", C.c_void_p), ("rotations", C.c_void_p),
                ("shs", C.c_void_p), ("rows", C.c_void_p), ("count", C.c_uint32)]


class SharedGrads(C.Structure):
    """rgs_shared_grads of include/rgs.h."""
    _fields_ = [("means3D", C.c_void_p), ("means2D", C.c_void_p), ("opacity", C.c_void_p), ("scales", C.c_void_p),
                ("rotations", C.c_void_p), ("shs", C.c_void_p), ("rows", C.c_void_p), ("count", C.c_uint32)]


class AdamTensor(C.Structure):
    """rgs_adam_tensor of include/rgs.h."""
    _fields_ = [("param", C.c_void_p), ("grad", C.c_void_p), ("exp_avg", C.c_void_p), ("exp_avg_sq", C.c_void_p),
                ("n", C.c_size_t), ("lr", C.c_double), ("step", C.c_int)]


class FrameView(C.Structure):
    """rgs_frame_view of include/rgs.h."""
    _fields_ = [("width", C.c_int), ("height", C.c_int), ("tan_fovx", C.c_float), ("tan_fovy", C.c_float),
                ("viewmatrix", C.c_void_p), ("projmatrix", C.c_void_p), ("projmatrix_inv", C.c_void_p),
                ("cam_pos", C.c_void_p)]


class FrameLayer(C.Structure):
    """rgs_frame_layer of include/rgs.h."""
    _fields_ = [("P", C.c_int), ("D", C.c_int), ("M", C.c_int), ("R", C.c_int),
                ("means3D", C.c_void_p), ("shs", C.c_void_p), ("colors_precomp", C.c_void_p), ("opacities", C.c_void_p),
                ("scales", C.c_void_p), ("rotations", C.c_void_p), ("cov3D_precomp", C.c_void_p),
                ("scale_modifier", C.c_float),
                ("background", C.c_void_p), ("range_low", C.c_void_p), ("range_up", C.c_void_p), ("radii", C.c_void_p),
                ("geom_ws", C.c_void_p), ("binning_ws", C.c_void_p), ("image_ws", C.c_void_p),
                ("geom_bytes", C.c_size_t), ("binning_bytes", C.c_size_t), ("image_bytes", C.c_size_t),
                ("out_color", C.c_void_p), ("out_depth", C.c_void_p), ("out_alpha", C.c_void_p),
                ("dL_dpix", C.c_void_p), ("dL_dpix_depth", C.c_void_p), ("dL_dalphas", C.c_void_p),
                ("grad_accum", C.c_void_p), ("dL_dmean2D", C.c_void_p), ("dL_dopacity", C.c_void_p),
                ("dL_dcolor", C.c_void_p), ("dL_dmean3D", C.c_void_p), ("dL_dcov3D", C.c_void_p), ("dL_dsh", C.c_void_p),
                ("dL_dscale", C.c_void_p), ("dL_drot", C.c_void_p), ("accum_zeroed", C.c_int),
                ("stream", C.c_void_p)]


class RgsError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m retinags_amd.build` "
            "(hipcc, gfx950). There is no fallback implementation.")
    lib = C.CDLL(LIB_PATH)
    vp, f, i, sz = C.c_void_p, C.c_float, C.c_int, C.c_size_t
    lib.rgs_version.restype = i
    lib.rgs_last_error.restype = C.c_char_p
    lib.rgs_get_higher_msb.restype = C.c_uint32
    lib.rgs_get_higher_msb.argtypes = [C.c_uint32]
    for name, args in (("rgs_geom_bytes", [i]), ("rgs_binning_bytes", [i]), ("rgs_image_bytes", [i, i]),
                       ("rgs_scan_temp_bytes", [sz]), ("rgs_sort_temp_bytes", [sz])):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = sz, args
    lib.rgs_geom_layout.argtypes = [i, C.POINTER(sz)]
    lib.rgs_binning_layout.argtypes = [i, i, i, C.POINTER(sz)]
    lib.rgs_image_layout.argtypes = [i, i, C.POINTER(sz)]
    lib.rgs_mark_visible.argtypes = [i, vp, vp, vp, vp, vp]
    lib.rgs_covariance3d.argtypes = [i, vp, f, vp, vp, vp]
    lib.rgs_forward_geom.argtypes = [i, i, i, i, i, vp, vp, vp, vp, vp, f, vp, vp, vp, vp, vp, f, f, i,
                                     vp, vp, sz, vp, vp, i]
    lib.rgs_forward_geom_enqueue.argtypes = lib.rgs_forward_geom.argtypes[:-2] + [vp, vp, i]
    lib.rgs_forward_raster.argtypes = [i, i, i, i, vp, f, f, vp, vp, vp, vp, vp, vp, sz, vp, sz, vp, sz,
                                       vp, vp, vp, vp, i]
    lib.rgs_forward_raster_bounded.argtypes = lib.rgs_forward_raster.argtypes
    lib.rgs_backward.argtypes = [i, i, i, i, i, i, vp, vp, vp, vp, vp, vp, f, vp, vp, vp, vp, vp, vp, vp, vp,
                                 f, f, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i, vp, i]
    lib.rgs_inclusive_sum.argtypes = [vp, vp, sz, vp, vp]
    lib.rgs_sort_pairs.argtypes = [vp, vp, vp, vp, sz, i, vp, vp]
    lib.rgs_sort_pairs_static.argtypes = [vp, vp, vp, vp, sz, i, vp]
    lib.rgs_frame_forward_geom.argtypes = [i, C.POINTER(FrameLayer), C.POINTER(FrameView), vp, vp, i]
    lib.rgs_frame_forward_raster.argtypes = [i, C.POINTER(FrameLayer), C.POINTER(FrameView), vp, i]
    lib.rgs_frame_backward.argtypes = [i, C.POINTER(FrameLayer), C.POINTER(FrameView), vp, i]
    lib.rgs_sort_fault.argtypes = [vp]
    lib.rgs_set_lookback_spin_limit.argtypes = [i]
    pp = C.POINTER(vp)
    lib.rgs_composite_forward.argtypes = [i, i, i, pp, pp, pp, vp, vp, vp, vp, vp]
    lib.rgs_composite_backward.argtypes = [i, i, i, pp, pp, pp, vp, vp, vp, vp, pp, pp, pp, vp]
    lib.rgs_straddler_scratch_bytes.restype, lib.rgs_straddler_scratch_bytes.argtypes = sz, [i, i]
    fp = C.POINTER(C.c_float)
    lib.rgs_straddler_select.argtypes = [i, vp, vp, fp, fp, i, fp, fp, i, vp, vp, C.c_uint32, vp, vp]
    lib.rgs_merge_rows.argtypes = [i, C.POINTER(SharedRows), C.c_uint32, i, vp, vp, vp, vp, vp, vp]
    lib.rgs_merge_rows_backward.argtypes = [i, C.POINTER(SharedGrads), C.c_uint32, i, vp, vp, vp, vp, vp, vp, vp]
    lib.rgs_loss_workspace_bytes.restype, lib.rgs_loss_workspace_bytes.argtypes = sz, [i, i, i]
    lib.rgs_l1_ssim_forward.argtypes = [i, i, i, vp, vp, f, vp, vp, i, vp]
    lib.rgs_l1_ssim_backward.argtypes = [i, i, i, vp, vp, f, vp, vp, vp, vp]
    lib.rgs_activate_forward.argtypes = [i, i] + [vp] * 10
    lib.rgs_activate_backward.argtypes = [i, i] + [vp] * 13
    lib.rgs_adam_step.argtypes = [i, C.POINTER(AdamTensor), C.c_double, C.c_double, C.c_double, vp]
    lib.rgs_stage_timing.argtypes = [i]
    lib.rgs_stage_timing_read.argtypes = [i, C.POINTER(C.c_char_p), C.POINTER(C.c_float), C.POINTER(C.c_int)]
    lib.rgs_blend_work_counters.argtypes = [i, i, i, i, f, f, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    for name in ("rgs_stage_timing", "rgs_stage_timing_read", "rgs_blend_work_counters", "rgs_geom_layout", "rgs_binning_layout", "rgs_image_layout", "rgs_mark_visible", "rgs_covariance3d",
                 "rgs_forward_geom", "rgs_forward_geom_enqueue", "rgs_forward_raster", "rgs_forward_raster_bounded", "rgs_backward", "rgs_inclusive_sum", "rgs_sort_pairs",
                 "rgs_composite_forward", "rgs_composite_backward", "rgs_straddler_select", "rgs_merge_rows",
                 "rgs_merge_rows_backward", "rgs_l1_ssim_forward", "rgs_l1_ssim_backward", "rgs_adam_step",
                 "rgs_activate_forward", "rgs_activate_backward", "rgs_sort_pairs_static", "rgs_sort_fault",
                 "rgs_set_lookback_spin_limit", "rgs_frame_forward_geom", "rgs_frame_forward_raster",
                 "rgs_frame_backward"):
        getattr(lib, name).restype = i
    return lib


lib = _load()

EXPORTS = ("rgs_version", "rgs_last_error", "rgs_get_higher_msb", "rgs_geom_bytes", "rgs_binning_bytes",
           "rgs_image_bytes", "rgs_geom_layout", "rgs_binning_layout", "rgs_image_layout", "rgs_mark_visible", "rgs_covariance3d",
           "rgs_forward_geom", "rgs_forward_geom_enqueue", "rgs_forward_raster", "rgs_forward_raster_bounded", "rgs_backward", "rgs_scan_temp_bytes", "rgs_inclusive_sum",
           "rgs_sort_temp_bytes", "rgs_sort_pairs", "rgs_composite_forward", "rgs_composite_backward",
           "rgs_stage_timing", "rgs_stage_timing_read", "rgs_blend_work_counters", "rgs_straddler_scratch_bytes",
           "rgs_straddler_select", "rgs_merge_rows", "rgs_merge_rows_backward", "rgs_loss_workspace_bytes",
           "rgs_l1_ssim_forward", "rgs_l1_ssim_backward", "rgs_adam_step", "rgs_activate_forward",
           "rgs_activate_backward", "rgs_sort_pairs_static", "rgs_sort_fault", "rgs_set_lookback_spin_limit",
           "rgs_frame_forward_geom", "rgs_frame_forward_raster", "rgs_frame_backward")
MAX_FRAME_LAYERS = 64
STATIC_SORT_MAX_PAIRS = 1 << 22
WORK_COUNTERS = 8


def check(rc: int) -> None:
    if rc != 0:
        raise RgsError(lib.rgs_last_error().decode("utf-8", "replace"))


def geom_layout(P: int) -> dict:
    off = (C.c_size_t * len(GEOM_FIELDS))()
    check(lib.rgs_geom_layout(P, off))
    return dict(zip(GEOM_FIELDS, off))


def binning_layout(R: int, width: int, height: int) -> dict:
    off = (C.c_size_t * len(BIN_FIELDS))()
    check(lib.rgs_binning_layout(R, width, height, off))
    return dict(zip(BIN_FIELDS, off))


def image_layout(width: int, height: int) -> dict:
    off = (C.c_size_t * len(IMG_FIELDS))()
    check(lib.rgs_image_layout(width, height, off))
    return dict(zip(IMG_FIELDS, off))


def stage_timing(enable: bool) -> None:
    check(lib.rgs_stage_timing(1 if enable else 0))


def stage_timing_read(max_stages: int = 64) -> dict:
    """{stage: (total_ms, launches)} recorded since the last read; waits for the work."""
    names = (C.c_char_p * max_stages)()
    ms = (C.c_float * max_stages)()
    cnt = (C.c_int * max_stages)()
    n = lib.rgs_stage_timing_read(max_stages, names, ms, cnt)
    if n < 0:
        raise RgsError(lib.rgs_last_error().decode("utf-8", "replace"))
    return {names[k].decode(): (float(ms[k]), int(cnt[k])) for k in range(n)}


def ptr(t) -> C.c_void_p:
    """Device (or pinned host) address of a tensor; None and empty tensors map to NULL,
    which is how the reference passes absent inputs (torch.Tensor([]) -> nullptr)."""
    if t is None or t.numel() == 0:
        return C.c_void_p(0)
    return C.c_void_p(t.data_ptr())


def ptr_table(tensors):
    arr = (C.c_void_p * len(tensors))()
    for k, t in enumerate(tensors):
        arr[k] = t.data_ptr()
    return arr
