"""ctypes/numpy front end of the CPU checker (``rgs_oracle.c``) plus the numpy
restatement of the partial-image compositor.

TEST INFRASTRUCTURE ONLY.  Tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the shipped package
must not.  The stage functions mirror the reference's stage sequence
(K/cuda_rasterizer_hgs/rasterizer_impl.cu:198-351 forward, :355-466 backward,
with K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian) and
keep every intermediate so a test can compare stage by stage.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librgs_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the C restatement with the Makefile beside it."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE, "librgs_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.orc_get_higher_msb.restype = C.c_uint32
        _lib.orc_get_higher_msb.argtypes = [C.c_uint32]
    return _lib


def set_threads(n: int) -> None:
    lib().orc_set_threads(C.c_int(int(n)))


def max_threads() -> int:
    return int(lib().orc_max_threads())


def _p(a: Optional[np.ndarray]):
    if a is None:
        return C.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"]
    return C.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _cf(v) -> C.c_float:
    # Python doubles reach the reference as C floats (K/rasterize_points.h:26,33-34).
    return C.c_float(float(v))


def get_higher_msb(n: int) -> int:
    return int(lib().orc_get_higher_msb(C.c_uint32(n)))


@dataclass
class Settings:
    """Field-for-field numpy twin of GaussianRasterizationSettings
    (K/diff_gaussian_rasterization_half_gaussian/__init__.py:166-181)."""
    image_height: int
    image_width: int
    tanfovx: float
    tanfovy: float
    bg: np.ndarray
    scale_modifier: float
    viewmatrix: np.ndarray
    projmatrix: np.ndarray
    projmatrix_inv: np.ndarray
    range_low: np.ndarray
    range_up: np.ndarray
    sh_degree: int
    campos: np.ndarray
    prefiltered: bool = False
    debug: bool = False

    def __post_init__(self):
        for k in ("bg", "viewmatrix", "projmatrix", "projmatrix_inv", "range_low", "range_up", "campos"):
            setattr(self, k, _f32(getattr(self, k)).reshape(-1))

    @property
    def grid(self):
        return ((self.image_width + 15) // 16, (self.image_height + 15) // 16)


def settings_from_camera(cam, range_low, range_up, bg, sh_degree=3, scale_modifier=1.0) -> Settings:
    """Settings for a harness camera (retinags_amd.harness.scenes.Camera, torch CPU tensors)
    and a submodel box, exactly the fields render4renderinfo fills
    (gaussian_renderer/render_half_gs.py:121-137)."""
    import math
    a = lambda t: np.ascontiguousarray(np.asarray(t.detach().cpu().numpy() if hasattr(t, "detach") else t,
                                                  dtype=np.float32))
    return Settings(
        image_height=int(cam.image_height), image_width=int(cam.image_width), tanfovx=math.tan(cam.FoVx * 0.5),
        tanfovy=math.tan(cam.FoVy * 0.5), bg=a(bg), scale_modifier=scale_modifier,
        viewmatrix=a(cam.world_view_transform), projmatrix=a(cam.full_proj_transform),
        projmatrix_inv=a(cam.projection_matrix_inv), range_low=a(range_low), range_up=a(range_up),
        sh_degree=sh_degree, campos=a(cam.camera_center))


@dataclass
class ForwardState:
    """Everything the forward produced (the reference keeps the same data in
    its three opaque byte buffers, K/cuda_rasterizer_hgs/rasterizer_impl.h:30-63)."""
    P: int
    R: int
    radii: np.ndarray
    xy: np.ndarray
    zw: np.ndarray
    depths: np.ndarray
    cov3D: np.ndarray
    rgb: np.ndarray
    conic_opacity: np.ndarray
    tiles_touched: np.ndarray
    clamped: np.ndarray
    point_offsets: np.ndarray
    keys_unsorted: np.ndarray
    values_unsorted: np.ndarray
    keys: np.ndarray
    point_list: np.ndarray
    ranges: np.ndarray
    color: np.ndarray
    depth: np.ndarray
    alpha: np.ndarray
    n_contrib: np.ndarray
    counters: np.ndarray
    margin: Optional[np.ndarray] = None
    inputs: dict = field(default_factory=dict)


def preprocess(s: Settings, means3D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
               cov3D_precomp=None):
    means3D = _f32(means3D)
    P = means3D.shape[0]
    opacities = _f32(opacities).reshape(-1)
    M = 0
    if shs is not None:
        shs = _f32(shs)
        M = shs.shape[1]
    if colors_precomp is not None:
        colors_precomp = _f32(colors_precomp)
    if scales is not None:
        scales = _f32(scales)
        rotations = _f32(rotations)
    if cov3D_precomp is not None:
        cov3D_precomp = _f32(cov3D_precomp)
    out = dict(
        radii=np.zeros(P, np.int32), xy=np.zeros((P, 2), np.float32), zw=np.zeros((P, 2), np.float32),
        depths=np.zeros(P, np.float32), cov3D=np.zeros((P, 6), np.float32), rgb=np.zeros((P, 3), np.float32),
        conic_opacity=np.zeros((P, 4), np.float32), tiles_touched=np.zeros(P, np.uint32),
        clamped=np.zeros((P, 3), np.uint8))
    lib().orc_preprocess(
        C.c_int(P), C.c_int(s.sh_degree), C.c_int(M), _p(means3D), _p(scales), _cf(s.scale_modifier), _p(rotations),
        _p(opacities), _p(shs), _p(cov3D_precomp), _p(colors_precomp), _p(s.viewmatrix), _p(s.projmatrix), _p(s.campos),
        C.c_int(s.image_width), C.c_int(s.image_height), _cf(s.tanfovx), _cf(s.tanfovy),
        _p(out["radii"]), _p(out["xy"]), _p(out["zw"]), _p(out["depths"]), _p(out["cov3D"]), _p(out["rgb"]),
        _p(out["conic_opacity"]), _p(out["tiles_touched"]), _p(out["clamped"]))
    out["inputs"] = dict(means3D=means3D, opacities=opacities, shs=shs, colors_precomp=colors_precomp, scales=scales,
                         rotations=rotations, cov3D_precomp=cov3D_precomp, M=M)
    return out


def mark_visible(s: Settings, means3D) -> np.ndarray:
    means3D = _f32(means3D)
    present = np.zeros(means3D.shape[0], np.uint8)
    lib().orc_mark_visible(C.c_int(means3D.shape[0]), _p(means3D), _p(s.viewmatrix), _p(s.projmatrix), _p(present))
    return present.astype(bool)


def inclusive_sum(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.uint32)
    out = np.zeros_like(x)
    lib().orc_inclusive_sum(C.c_int(x.shape[0]), _p(x), _p(out))
    return out


def duplicate_with_keys(xy, depths, offsets, radii, grid, R):
    keys = np.zeros(R, np.uint64)
    vals = np.zeros(R, np.uint32)
    lib().orc_duplicate_with_keys(C.c_int(radii.shape[0]), _p(xy), _p(depths), _p(offsets), _p(keys), _p(vals),
                                  _p(radii), C.c_int(grid[0]), C.c_int(grid[1]))
    return keys, vals


def sort_pairs(keys, vals, end_bit):
    keys = np.ascontiguousarray(keys, np.uint64)
    vals = np.ascontiguousarray(vals, np.uint32)
    n = keys.shape[0]
    ko, vo = np.zeros_like(keys), np.zeros_like(vals)
    tk, tv = np.zeros_like(keys), np.zeros_like(vals)
    lib().orc_sort_pairs(C.c_size_t(n), _p(keys), _p(ko), _p(vals), _p(vo), C.c_int(end_bit), _p(tk), _p(tv))
    return ko, vo


def identify_tile_ranges(keys, T):
    ranges = np.zeros((T, 2), np.uint32)
    lib().orc_identify_tile_ranges(C.c_size_t(keys.shape[0]), _p(keys), _p(ranges), C.c_int(T))
    return ranges


def render_forward(s: Settings, ranges, point_list, zw, xy, features, depths, conic_opacity, want_margin=False):
    H, W = s.image_height, s.image_width
    color = np.zeros((3, H, W), np.float32)
    depth = np.zeros((1, H, W), np.float32)
    alpha = np.zeros((1, H, W), np.float32)
    n_contrib = np.zeros(H * W, np.uint32)
    counters = np.zeros(5, np.uint64)
    margin = np.zeros(H * W, np.float32) if want_margin else None
    lib().orc_render_forward(
        C.c_int(W), C.c_int(H), _p(ranges), _p(point_list), _cf(s.tanfovx), _cf(s.tanfovy), _p(zw),
        _p(s.projmatrix_inv), _p(s.range_low), _p(s.range_up), _p(xy), _p(features), _p(depths), _p(conic_opacity),
        _p(s.bg), _p(color), _p(depth), _p(alpha), _p(n_contrib), _p(counters), _p(margin))
    return color, depth, alpha, n_contrib, counters, margin


def forward(s: Settings, means3D, opacities, shs=None, colors_precomp=None, scales=None, rotations=None,
            cov3D_precomp=None, want_margin=False) -> ForwardState:
    """Rasterizer::forward, K/cuda_rasterizer_hgs/rasterizer_impl.cu:198-351."""
    pre = preprocess(s, means3D, opacities, shs, colors_precomp, scales, rotations, cov3D_precomp)
    P = pre["radii"].shape[0]
    gx, gy = s.grid
    T = gx * gy
    offsets = inclusive_sum(pre["tiles_touched"])
    R = int(offsets[-1]) if P > 0 else 0
    keys_u, vals_u = duplicate_with_keys(pre["xy"], pre["depths"], offsets, pre["radii"], (gx, gy), R)
    bit = get_higher_msb(T)
    keys, plist = sort_pairs(keys_u, vals_u, 32 + bit)
    ranges = identify_tile_ranges(keys, T)
    feats = pre["inputs"]["colors_precomp"] if colors_precomp is not None else pre["rgb"]
    color, depth, alpha, n_contrib, counters, margin = render_forward(
        s, ranges, plist, pre["zw"], pre["xy"], feats, pre["depths"], pre["conic_opacity"], want_margin)
    return ForwardState(P=P, R=R, point_offsets=offsets, keys_unsorted=keys_u, values_unsorted=vals_u, keys=keys,
                        point_list=plist, ranges=ranges, color=color, depth=depth, alpha=alpha, n_contrib=n_contrib,
                        counters=counters, margin=margin, **pre)


def backward(s: Settings, st: ForwardState, dL_dcolor, dL_ddepth=None, dL_dalpha=None):
    """Rasterizer::backward, K/cuda_rasterizer_hgs/rasterizer_impl.cu:355-466, with the
    zero-initialised buffers of K/rasterize_points.cu:165-174.  Returns the 8
    gradients in the order of _RasterizeGaussians.backward
    (K/diff_gaussian_rasterization_half_gaussian/__init__.py:150-162) plus the
    internal dL_dconic / dL_ddepths scratch."""
    H, W, P = s.image_height, s.image_width, st.P
    inp = st.inputs
    M = inp["M"]
    dL_dcolor = _f32(dL_dcolor).reshape(3, H, W)
    dL_ddepth = np.zeros((1, H, W), np.float32) if dL_ddepth is None else _f32(dL_ddepth).reshape(1, H, W)
    dL_dalpha = np.zeros((1, H, W), np.float32) if dL_dalpha is None else _f32(dL_dalpha).reshape(1, H, W)
    g = dict(
        means2D=np.zeros((P, 3), np.float32), conic=np.zeros((P, 2, 2), np.float32),
        opacity=np.zeros((P, 1), np.float32), colors=np.zeros((P, 3), np.float32), depths=np.zeros((P, 1), np.float32),
        means3D=np.zeros((P, 3), np.float32), cov3D=np.zeros((P, 6), np.float32), sh=np.zeros((P, M, 3), np.float32),
        scales=np.zeros((P, 3), np.float32), rotations=np.zeros((P, 4), np.float32))
    if P == 0:
        return g
    feats = inp["colors_precomp"] if inp["colors_precomp"] is not None else st.rgb
    lib().orc_render_backward(
        C.c_int(W), C.c_int(H), _p(st.ranges), _p(st.point_list), _cf(s.tanfovx), _cf(s.tanfovy),
        _p(s.projmatrix_inv), _p(s.range_low), _p(s.range_up), _p(st.zw), _p(s.bg), _p(st.xy), _p(st.conic_opacity),
        _p(feats), _p(st.depths), _p(st.alpha), _p(st.n_contrib), _p(dL_dcolor), _p(dL_ddepth), _p(dL_dalpha),
        _p(g["means2D"]), _p(g["conic"]), _p(g["opacity"]), _p(g["colors"]), _p(g["depths"]))
    cov3D = inp["cov3D_precomp"] if inp["cov3D_precomp"] is not None else st.cov3D
    # focal lengths: K/cuda_rasterizer_hgs/rasterizer_impl.cu:407-408
    tany, tanx = np.float32(s.tanfovy), np.float32(s.tanfovx)
    fy = np.float32(H) / (np.float32(2.0) * tany)
    fx = np.float32(W) / (np.float32(2.0) * tanx)
    lib().orc_cov2d_backward(
        C.c_int(P), _p(inp["means3D"]), _p(st.radii), _p(cov3D), _cf(fx), _cf(fy), _cf(s.tanfovx), _cf(s.tanfovy),
        _p(s.viewmatrix), _p(g["conic"]), _p(g["means3D"]), _p(g["cov3D"]))
    lib().orc_preprocess_backward(
        C.c_int(P), C.c_int(s.sh_degree), C.c_int(M), _p(inp["means3D"]), _p(st.radii), _p(inp["shs"]),
        _p(st.clamped), _p(inp["scales"]), _p(inp["rotations"]), _cf(s.scale_modifier), _p(s.viewmatrix),
        _p(s.projmatrix), _p(s.campos), _p(g["means2D"]), _p(g["means3D"]), _p(g["colors"]), _p(g["depths"]),
        _p(g["cov3D"]), _p(g["sh"]), _p(g["scales"]), _p(g["rotations"]))
    return g


# ---------------------------------------------------------------------------------------
# Compositor: parallel_utils/basic_parallel_trainer/result_aggregator.py:244-259.
# Inputs are already in compositing order (the reference sorts by the relation
# vector at :233 first).  T_0 = 1, T_k = prod_{j<k}(1 - alpha_j), accumulated
# front to back in float32 like torch.cumprod; sums run k = 0..K-1 in order.
# ---------------------------------------------------------------------------------------

def composite_forward(images, depths, alphas, bg):
    K = len(images)
    H, W = images[0].shape[-2:]
    bg = _f32(bg).reshape(3)
    T = np.ones((H, W), np.float32)
    img = np.zeros((3, H, W), np.float32)
    dep = np.zeros((1, H, W), np.float32)
    for k in range(K):
        img += T[None] * _f32(images[k]).reshape(3, H, W)
        dep += T[None] * _f32(depths[k]).reshape(1, H, W)
        T = T * (np.float32(1.0) - _f32(alphas[k]).reshape(H, W))
    out_img = img + bg[:, None, None] * T[None]
    out_alpha = (np.float32(1.0) - T)[None]
    return out_img, dep, out_alpha


def composite_backward(images, depths, alphas, bg, g_img, g_depth=None, g_alpha=None):
    """Gradients of composite_forward w.r.t. every partial image, depth and alpha
    (what torch autograd returns for the reference's cumprod/sum graph)."""
    K = len(images)
    H, W = images[0].shape[-2:]
    bg = _f32(bg).reshape(3)
    g_img = _f32(g_img).reshape(3, H, W)
    g_depth = np.zeros((1, H, W), np.float32) if g_depth is None else _f32(g_depth).reshape(1, H, W)
    g_alpha = np.zeros((1, H, W), np.float32) if g_alpha is None else _f32(g_alpha).reshape(1, H, W)
    Ts = [np.ones((H, W), np.float32)]
    for k in range(K):
        Ts.append(Ts[-1] * (np.float32(1.0) - _f32(alphas[k]).reshape(H, W)))
    d_img, d_dep, d_alp = [None] * K, [None] * K, [None] * K
    # R_k = d(out)/d(T_{k+1}) contracted with the upstream gradients, built back to front
    Rk = (bg[:, None, None] * g_img).sum(0) - g_alpha[0]
    for k in range(K - 1, -1, -1):
        d_img[k] = Ts[k][None] * g_img
        d_dep[k] = Ts[k][None] * g_depth
        d_alp[k] = (-(Ts[k] * Rk))[None]
        Rk = (_f32(images[k]).reshape(3, H, W) * g_img).sum(0) + _f32(depths[k]).reshape(H, W) * g_depth[0] \
            + (np.float32(1.0) - _f32(alphas[k]).reshape(H, W)) * Rk
    return d_img, d_dep, d_alp
