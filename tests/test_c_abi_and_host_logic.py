"""CPU-side checks: the C-ABI library loads and exports every symbol that include/rgs.h
declares, size/layout queries behave (they launch nothing), and the Python mirror of the
reference module validates arguments like the reference
(K/diff_gaussian_rasterization_half_gaussian/__init__.py:199-207,
 K = rasterization_kernels/diff-gaussian-rasterization-half-gaussian).  No kernel runs here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from helpers import ROOT, orc


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "rgs.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rgs_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from retinags_amd import _capi
    names = _declared_symbols()
    assert len(names) >= 20
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/rgs.h but not exported"
    assert set(_capi.EXPORTS) == set(names)
    assert _capi.lib.rgs_version() >= 100
    assert _capi.lib.rgs_last_error() is not None


def test_higher_msb_matches_checker():
    from retinags_amd import _capi
    for n in list(range(1, 3000)) + [6500, 8160, 68250, 2 ** 20 - 1, 2 ** 20, 2 ** 31 - 1]:
        assert _capi.lib.rgs_get_higher_msb(n) == orc.get_higher_msb(n) == n.bit_length()


def test_workspace_sizes_and_layouts_are_consistent():
    from retinags_amd import _capi
    for P in (1, 255, 256, 257, 100_000):
        lay = _capi.geom_layout(P)
        total = _capi.lib.rgs_geom_bytes(P)
        sizes = dict(depths=4 * P, tiles_touched=4 * P, point_offsets=4 * P, clamped=P, block_sums=4 * ((P + 255) // 256 + 1), total=4,
                     blend_record=64 * P, depth_order=4 * P, block_visible=4 * ((P + 255) // 256 + 1),
                     visible_count=4, order_scratch=16 * P)
        spans = sorted((lay[k], lay[k] + sizes[k]) for k in sizes)
        assert all(a % 256 == 0 for a, _ in spans)
        assert all(spans[i][1] <= spans[i + 1][0] for i in range(len(spans) - 1))
        assert spans[-1][1] <= total
    for R, (W, H) in ((1, (512, 512)), (4097, (1600, 1036)), (10 ** 6, (5185, 3359))):
        lay = _capi.binning_layout(R, W, H)
        total = _capi.lib.rgs_binning_bytes(R)
        sizes = dict(keys_unsorted=4 * R, keys_sorted=4 * R, values_unsorted=4 * R, values_sorted=4 * R,
                     sort_temp=_capi.lib.rgs_sort_temp_bytes(R), strip_lists=16 * R)
        spans = sorted((lay[k], lay[k] + sizes[k]) for k in sizes)
        assert all(spans[i][1] <= spans[i + 1][0] for i in range(len(spans) - 1))
        assert spans[-1][1] <= total
    lay = _capi.image_layout(1600, 1036)
    assert lay["n_contrib"] >= 8 * 6500 and lay["n_contrib"] + 4 * 1600 * 1036 <= _capi.lib.rgs_image_bytes(1600, 1036)


def test_entry_points_reject_bad_arguments_without_launching():
    from retinags_amd import _capi
    lib = _capi.lib
    null = ctypes.c_void_p(0)
    assert lib.rgs_mark_visible(-1, null, null, null, null, null) != 0
    assert b"negative" in lib.rgs_last_error()
    assert lib.rgs_mark_visible(0, null, null, null, null, null) == 0
    assert lib.rgs_sort_pairs(null, null, null, null, 10, 0, null, null) != 0
    assert lib.rgs_sort_pairs(null, null, null, null, 0, 40, null, null) == 0
    assert lib.rgs_inclusive_sum(null, null, 0, null, null) == 0
    tbl = (ctypes.c_void_p * 1)()
    assert lib.rgs_composite_forward(0, 4, 4, tbl, tbl, tbl, null, null, null, null, null) != 0
    assert lib.rgs_composite_forward(65, 4, 4, tbl, tbl, tbl, null, null, null, null, null) != 0
    assert b"outside" in lib.rgs_last_error()
    rc = lib.rgs_forward_geom(0, 3, 16, 64, 64, null, null, null, null, null, 1.0, null, null, null, null, null,
                              1.0, 1.0, 0, null, null, 0, null, null, 0)
    assert rc != 0 and b"P must be positive" in lib.rgs_last_error()
    assert lib.rgs_covariance3d(-1, null, 1.0, null, null, null) != 0
    assert lib.rgs_covariance3d(0, null, 1.0, null, null, null) == 0
    # the frame entry points: layer counts outside 1..RGS_MAX_FRAME_LAYERS, null tables
    layers = (_capi.FrameLayer * 1)()
    view = _capi.FrameView()
    for K in (0, _capi.MAX_FRAME_LAYERS + 1):
        assert lib.rgs_frame_forward_geom(K, layers, ctypes.byref(view), null, null, 0) != 0
        assert b"outside" in lib.rgs_last_error()
        assert lib.rgs_frame_forward_raster(K, layers, ctypes.byref(view), null, 0) != 0
        assert lib.rgs_frame_backward(K, layers, ctypes.byref(view), null, 0) != 0
    assert lib.rgs_frame_forward_geom(1, None, ctypes.byref(view), null, null, 0) != 0
    # the sort that allocates nothing refuses more pairs than its array holds, before it touches a device
    assert lib.rgs_sort_pairs_static(null, null, null, null, _capi.STATIC_SORT_MAX_PAIRS + 1, 32, null) != 0
    assert b"pairs" in lib.rgs_last_error()


def test_rasterizer_argument_validation_matches_reference():
    from diff_gaussian_rasterization_half_gaussian import GaussianRasterizationSettings, GaussianRasterizer
    z = torch.zeros
    settings = GaussianRasterizationSettings(
        image_height=32, image_width=32, tanfovx=0.5, tanfovy=0.5, bg=z(3), scale_modifier=1.0, viewmatrix=torch.eye(4),
        projmatrix=torch.eye(4), projmatrix_inv=torch.eye(4), range_low=-torch.ones(3), range_up=torch.ones(3),
        sh_degree=3, campos=z(3), prefiltered=False, debug=False)
    assert settings._fields == ("image_height", "image_width", "tanfovx", "tanfovy", "bg", "scale_modifier",
                                "viewmatrix", "projmatrix", "projmatrix_inv", "range_low", "range_up", "sh_degree",
                                "campos", "prefiltered", "debug")
    r = GaussianRasterizer(settings)
    m = z(5, 3)
    with pytest.raises(Exception, match="SHs or precomputed colors"):
        r(means3D=m, means2D=m, opacities=z(5, 1), scales=z(5, 3), rotations=z(5, 4))
    with pytest.raises(Exception, match="SHs or precomputed colors"):
        r(means3D=m, means2D=m, opacities=z(5, 1), shs=z(5, 16, 3), colors_precomp=z(5, 3), scales=z(5, 3), rotations=z(5, 4))
    with pytest.raises(Exception, match="scale/rotation pair or precomputed 3D covariance"):
        r(means3D=m, means2D=m, opacities=z(5, 1), shs=z(5, 16, 3))
    with pytest.raises(Exception, match="scale/rotation pair or precomputed 3D covariance"):
        r(means3D=m, means2D=m, opacities=z(5, 1), shs=z(5, 16, 3), scales=z(5, 3), rotations=z(5, 4), cov3D_precomp=z(5, 6))
    # wrong rank of means3D is an error (K/rasterize_points.cu:60-62); host tensors cannot be rasterized
    with pytest.raises(RuntimeError, match="num_points, 3"):
        r(means3D=z(5), means2D=m, opacities=z(5, 1), shs=z(5, 16, 3), scales=z(5, 3), rotations=z(5, 4))
    with pytest.raises(RuntimeError, match="GPU"):
        r(means3D=m, means2D=m, opacities=z(5, 1), shs=z(5, 16, 3), scales=z(5, 3), rotations=z(5, 4))


def test_no_shipped_module_touches_the_checker():
    """The product path must not import, load or call anything under oracle/."""
    for base, _, files in os.walk(os.path.join(ROOT, "retinags_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text and "rgs_oracle" not in text, os.path.join(base, f)
    text = open(os.path.join(ROOT, "diff_gaussian_rasterization_half_gaussian", "__init__.py")).read()
    assert "oracle" not in text


def test_partition_and_order_invariants():
    from retinags_amd.harness import scenes, partition
    scene, cam, _ = scenes.make_config("C1", shrink=200)
    n = scene["xyz"].shape[0]
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    assert len(part.leaves) == 4 and [l.path for l in part.leaves] == ["00", "01", "10", "11"]
    # leaves tile the grid without overlap
    cells = np.zeros(part.grid.size, dtype=np.int32)
    for l in part.leaves:
        cells[l.low[0]:l.up[0], l.low[1]:l.up[1], l.low[2]:l.up[2]] += 1
    assert (cells == 1).all()
    # balanced by load within a few percent at this size
    own_counts = np.bincount(part.owner, minlength=4)
    assert own_counts.sum() == n and own_counts.min() > 0.2 * n
    xyz = scene["xyz"].numpy()
    for k in range(4):
        ids = part.members[k]
        own = ids[: own_counts[k]]
        assert (part.owner[own] == k).all() and (np.diff(own) > 0).all()
        assert ((xyz[own] >= part.box_low[k]) & (xyz[own] <= part.box_up[k])).all()
        shared = ids[own_counts[k]:]
        assert (part.owner[shared] != k).all()
        src = part.owner[shared]
        assert (np.diff(src) >= 0).all()  # ascending source submodel
        r = 3.0 * scene["scales"].numpy()[shared].max(axis=1)
        assert ((xyz[shared] + r[:, None] >= part.box_low[k]) & (xyz[shared] - r[:, None] <= part.box_up[k])).all()
    rel = partition.relation_vector(part, cam)
    seen = sorted(v for v in rel if v >= 0)
    assert len(set(seen)) == len(seen)
    # the submodel that contains the camera's (x, y) is composited first
    c = cam.camera_center.numpy()
    inside = [k for k in range(4) if (c[:2] >= part.box_low[k][:2]).all() and (c[:2] <= part.box_up[k][:2]).all()]
    assert inside and rel[inside[0]] == min(seen)


def test_banded_tile_order_is_a_bijection(tmp_path):
    """The blend kernels take tiles in an XCD-banded order; every tile must be taken exactly once."""
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    exe = str(tmp_path / "tile_order_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-I", os.path.join(here, "..", "retinags_amd", "csrc"),
                    os.path.join(here, "tile_order_check.cpp"), "-o", exe], check=True)
    out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "ok"


def test_grad_norm_helper_hands_back_the_screen_space_gradient_length():
    """gaussian_renderer/render_half_gs.py:7-19."""
    from retinags_amd.harness.pipeline import gradNormHelpFunction
    meta = torch.zeros(5, 1, requires_grad=True)
    means2D = gradNormHelpFunction(meta)
    assert means2D.shape == (5, 3) and float(means2D.detach().abs().sum()) == 0.0 and means2D.requires_grad
    g = torch.tensor([[3.0, 4.0, 9.0], [0.0, 0.0, 1.0], [1.0, 0.0, 0.0], [-6.0, 8.0, 0.0], [0.5, 0.5, 0.5]])
    means2D.backward(g)
    assert torch.allclose(meta.grad[:, 0], torch.tensor([5.0, 0.0, 1.0, 10.0, 0.5 * 2 ** 0.5]))
    with pytest.raises(RuntimeError):
        gradNormHelpFunction(torch.zeros(5, 2))


def test_entry_points_refuse_bad_arguments_before_touching_the_gpu():
    """Argument checks come first and report through rgs_last_error; none of these calls launches."""
    import ctypes as C
    from retinags_amd import _capi
    lib = _capi.lib
    null = C.c_void_p(0)
    fp = C.POINTER(C.c_float)
    three = (C.c_float * 3)(0, 0, 0)
    boxes = (C.c_float * 6)(0, 0, 0, 1, 1, 1)
    as_fp = lambda a: C.cast(a, fp)

    def refused(rc, needle):
        assert rc != 0
        message = lib.rgs_last_error().decode()
        assert needle in message, message

    refused(lib.rgs_straddler_select(10, null, null, as_fp(three), as_fp(three), 0, as_fp(boxes), as_fp(boxes), -1,
                                     null, null, 0, null, null), "n_boxes")
    refused(lib.rgs_straddler_select(10, null, null, as_fp(three), as_fp(three), 65, as_fp(boxes), as_fp(boxes), -1,
                                     null, null, 0, null, null), "n_boxes")
    refused(lib.rgs_straddler_select(10, null, null, as_fp(three), as_fp(three), 2, as_fp(boxes), as_fp(boxes), 2,
                                     null, null, 0, null, null), "skip")
    refused(lib.rgs_straddler_select(-1, null, null, as_fp(three), as_fp(three), 2, as_fp(boxes), as_fp(boxes), 0,
                                     null, null, 0, null, null), "negative")
    seg = (_capi.SharedRows * 1)(_capi.SharedRows(None, None, None, None, None, None, 5))
    refused(lib.rgs_merge_rows(1, seg, 0, 48, null, null, null, null, null, null), "null field")
    refused(lib.rgs_merge_rows(1, seg, 0, -3, null, null, null, null, null, null), "sh_floats")
    assert lib.rgs_merge_rows(0, None, 0, 48, null, null, null, null, null, null) == 0       # nothing to do
    grads = (_capi.SharedGrads * 1)(_capi.SharedGrads(None, None, None, None, None, None, None, 5))
    refused(lib.rgs_merge_rows_backward(1, grads, 0, 48, null, null, null, null, null, null, null), "row list")
    refused(lib.rgs_l1_ssim_forward(3, 0, 10, null, null, 0.2, null, null, 1, null), "bad image size")
    refused(lib.rgs_l1_ssim_forward(3, 10, 10, null, null, 0.2, null, null, 1, null), "null pointer")
    refused(lib.rgs_l1_ssim_backward(3, 10, 10, null, null, 0.2, null, null, null, null), "null pointer")
    assert lib.rgs_loss_workspace_bytes(3, 0, 5) == 0 and lib.rgs_loss_workspace_bytes(3, 16, 32) == 4 * (3 * 3 * 16 * 32 + 2 * 3)
    t = (_capi.AdamTensor * 1)(_capi.AdamTensor(None, None, None, None, 8, 0.1, 1))
    refused(lib.rgs_adam_step(1, t, 0.9, 0.999, 1e-8, null), "null array")
    t[0].n, t[0].step = 0, 0
    refused(lib.rgs_adam_step(1, t, 0.9, 0.999, 1e-8, null), "step")
    assert lib.rgs_adam_step(0, None, 0.9, 0.999, 1e-8, null) == 0
    refused(lib.rgs_activate_forward(-1, 15, *([null] * 10)), "bad sizes")
    refused(lib.rgs_activate_forward(8, 15, *([null] * 10)), "null pointer")
    odd = C.c_void_p(0x1004)
    even = C.c_void_p(0x1000)
    refused(lib.rgs_activate_forward(8, 15, even, even, odd, even, even, even, even, even, even, null), "16 bytes")
    refused(lib.rgs_activate_backward(8, 15, null, null, null, even, null, null, null, null, null, null, null, null, null),
            "no room for the SH gradients")
    assert lib.rgs_activate_forward(0, 15, *([null] * 10)) == 0 and lib.rgs_activate_backward(0, 15, *([null] * 13)) == 0
    assert lib.rgs_straddler_scratch_bytes(-1, 4) == 0 and lib.rgs_straddler_scratch_bytes(1025, 3) == 4 * 3 * 3


def test_tensor_expression_branches_of_the_renderer_match_the_checker():
    """The convert_SHs_python and compute_cov3D_python branches of render4BoundedGaussianModel
    (gaussian_renderer/render_half_gs.py:55-77) as the harness restates them: colours and 3D covariances from tensor
    operations against what the checker's preprocess computes in its kernel-order arithmetic, SH degrees 0 to 3,
    a scale modifier, and quaternions that are not normalised (the tensor expression normalises them, the kernel
    uses them as given: equal only for unit quaternions, which is what a model's get_rotation hands out)."""
    from helpers import np32, oracle_settings, scenes
    from retinags_amd.harness import pipeline
    scene, cam, _ = scenes.make_config("C0", shrink=100, resolution_scale=0.25)
    pad = 3.0 * float(scene["scales"].max()) + 1.0
    low, up = scene["xyz"].min(0).values - pad, scene["xyz"].max(0).values + pad
    for degree, mod in ((0, 1.0), (1, 1.0), (2, 1.0), (3, 1.0), (3, 0.7)):
        s = oracle_settings(cam, low, up, torch.zeros(3), sh_degree=degree, scale_modifier=mod)
        st = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]), scales=np32(scene["scales"]),
                         rotations=np32(scene["rotations"]))
        vis = st.radii > 0
        assert vis.sum() > 100
        rgb = pipeline.colours_from_sh(scene["shs"], degree, scene["xyz"], cam.camera_center).numpy()
        cov = pipeline.covariance_from_scaling_rotation(scene["scales"], mod, scene["rotations"]).numpy()
        assert np.abs(rgb[vis] - st.rgb[vis]).max() <= 1e-6
        assert np.abs(cov[vis] - st.cov3D[vis]).max() <= 1e-6 * np.abs(st.cov3D[vis]).max()
        # clamped channels are zero in both
        assert np.array_equal(rgb[vis] == 0.0, st.clamped[vis].astype(bool)) or np.abs((rgb[vis] == 0.0) ^ st.clamped[vis].astype(bool)).mean() < 1e-3
    # the basis itself against scipy's complex harmonics, through the test-side polynomials (sign convention (-1)^m)
    import refmath
    d = torch.randn(64, 3, dtype=torch.float64)
    d = d / d.norm(dim=1, keepdim=True)
    assert torch.allclose(pipeline.sh_basis(3, d), refmath.sh_polynomials(d), atol=1e-12)
    assert np.allclose(pipeline.sh_basis(3, d).numpy(), refmath.real_sh_basis(d.numpy(), 3), atol=1e-12)
    scaled = pipeline.covariance_from_scaling_rotation(scene["scales"], 1.0, 3.0 * scene["rotations"])
    plain = pipeline.covariance_from_scaling_rotation(scene["scales"], 1.0, scene["rotations"])
    assert float((scaled - plain).abs().max()) <= 1e-6 * float(plain.abs().max())


def test_exponent_of_a_conic_staged_pre_scaled_has_the_bits_of_the_reference_expression():
    """The blend kernels keep a conic as (-xx/2, -xy, -yy/2) and evaluate
    (sxx dx) dx + (syy dy) dy + (sxy dx) dy, one multiplication less than the reference's
    -0.5 (xx dx dx + yy dy dy) - xy dx dy (K/cuda_rasterizer_hgs/forward.cu:353).  Scaling by a
    power of two and negation commute with rounding, so both must give the same float32 bits,
    operation by operation; checked here in float32 arithmetic on random conics and offsets,
    the exponents of the same magnitudes the kernels see included."""
    rng = np.random.default_rng(5)
    n = 400_000
    f = np.float32
    xx = rng.uniform(1e-3, 3.3, n).astype(f)
    yy = rng.uniform(1e-3, 3.3, n).astype(f)
    xy = (rng.uniform(-0.99, 0.99, n) * np.sqrt(xx.astype(np.float64) * yy)).astype(f)
    dx = rng.uniform(-40, 40, n).astype(f)
    dy = rng.uniform(-40, 40, n).astype(f)
    # a share of exact zeros and of tiny offsets
    dx[::17] = 0
    dy[::13] = 0
    dx[5::29] *= f(1e-4)
    reference = f(-0.5) * (xx * dx * dx + yy * dy * dy) - xy * dx * dy
    sxx, sxy, syy = f(-0.5) * xx, -xy, f(-0.5) * yy
    staged = (sxx * dx * dx + syy * dy * dy) + sxy * dx * dy
    assert reference.dtype == np.float32 and staged.dtype == np.float32
    assert np.array_equal(reference.view(np.uint32), staged.view(np.uint32))
