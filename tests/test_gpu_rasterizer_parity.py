"""HIP rasterizer vs the CPU checker on identical seeded inputs, stage by stage.

Bit-exact: radii, tile counts, pixel centres, depth bits, clip-w, the depth order of the
Gaussians and their offsets, the sorted (tile, depth) keys (rebuilt from the library's tile
keys and depth bits), per-tile Gaussian lists, tile ranges.  Within 1e-4 max-abs:
rendered colour, depth and alpha planes.  Within 1e-3 relative L2: every gradient.
"""
import ctypes

import numpy as np
import pytest
import torch

from helpers import (check_binning_against, DECISION_MARGIN, GRAD_TOL, IMAGE_TOL, MAX_BORDERLINE_FRACTION, np32, oracle_settings, orc,
                     rel_l2, scenes, view_ws)

pytestmark = pytest.mark.gpu


def _run_gpu_forward(sub, cam, bg, dev, sh_degree=3, scale_modifier=1.0, debug=False):
    from retinags_amd import rasterizer as R
    e = torch.Tensor([])
    return R._rasterize_forward(
        bg.to(dev), sub["xyz"].to(dev), e, sub["opacity"].to(dev), sub["scales"].to(dev), sub["rotations"].to(dev),
        scale_modifier, e, cam.world_view_transform.to(dev), cam.full_proj_transform.to(dev),
        cam.projection_matrix_inv.to(dev), sub["low"].to(dev), sub["up"].to(dev), cam.tanfovx, cam.tanfovy,
        cam.image_height, cam.image_width, sub["shs"].to(dev), sh_degree, cam.camera_center.to(dev), False, debug)


def _check_forward_stages(sub, cam, bg, sh_degree=3, scale_modifier=1.0, max_borderline=MAX_BORDERLINE_FRACTION):
    from retinags_amd import _capi
    dev = torch.device("cuda:0")
    s = oracle_settings(cam, sub["low"], sub["up"], bg, sh_degree, scale_modifier)
    st = orc.forward(s, np32(sub["xyz"]), np32(sub["opacity"]), shs=np32(sub["shs"]), scales=np32(sub["scales"]),
                     rotations=np32(sub["rotations"]), want_margin=True)
    R, color, depth, alpha, radii, geom, binning, img = _run_gpu_forward(sub, cam, bg, dev, sh_degree, scale_modifier)
    torch.cuda.synchronize()
    P, W, H = st.P, cam.image_width, cam.image_height
    T = s.grid[0] * s.grid[1]

    # ---- per-Gaussian geometry: bit-exact
    assert R == st.R
    radii = radii.cpu().numpy()
    assert np.array_equal(radii, st.radii)
    vis = st.radii > 0
    g = _capi.geom_layout(P)
    assert np.array_equal(view_ws(geom, g["tiles_touched"], P, np.uint32), st.tiles_touched)
    assert np.array_equal(view_ws(geom, g["depths"], P, np.uint32)[vis], st.depths.view(np.uint32)[vis])
    # pixel centre, clip w, conic, opacity and colour live in the Gaussian's 64-byte record only
    rec = view_ws(geom, g["blend_record"], 16 * P, np.uint32).reshape(P, 16)[vis]
    assert np.array_equal(rec[:, 0:2], st.xy[vis].view(np.uint32))
    assert np.array_equal(rec[:, 3], st.zw[:, 1].copy().view(np.uint32)[vis])
    assert np.array_equal(rec[:, 4:8], st.conic_opacity[vis].view(np.uint32))
    assert np.array_equal(rec[:, 8:11], st.rgb[vis].view(np.uint32))
    assert np.array_equal(rec[:, 11], st.depths.view(np.uint32)[vis])
    assert np.array_equal(rec[:, 14], st.radii[vis].astype(np.int32).view(np.uint32))
    # the 3D covariance is kept nowhere: forward and backward compute it with the function behind this entry point
    cov = torch.empty((P, 6), device=dev)
    scales_d, rot_d = sub["scales"].to(dev).contiguous(), sub["rotations"].to(dev).contiguous()
    _capi.check(_capi.lib.rgs_covariance3d(P, _capi.ptr(scales_d), scale_modifier, _capi.ptr(rot_d), _capi.ptr(cov),
                                           ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)))
    assert np.array_equal(cov.cpu().numpy()[vis].view(np.uint32), st.cov3D[vis].view(np.uint32))
    clamped = view_ws(geom, g["clamped"], P, np.uint8)
    packed = st.clamped[:, 0] | (st.clamped[:, 1] << 1) | (st.clamped[:, 2] << 2)
    assert np.array_equal(clamped[vis], packed[vis])

    # ---- binning: bit-exact
    check_binning_against(st, geom, binning, P, R, W, H)
    im = _capi.image_layout(W, H)
    assert np.array_equal(view_ws(img, im["ranges"], 2 * T, np.uint32).reshape(T, 2), st.ranges)

    # ---- what the forward blend leaves for the backward: per 16x4 strip the entries it filed, up
    # to the last one blended, and the strips ordered by how many those are
    filed = view_ws(img, im["strip_filed"], 4 * T, np.uint32)
    order = view_ws(img, im["strip_order"], 4 * T, np.uint32)
    assert np.array_equal(np.sort(order), np.arange(4 * T, dtype=np.uint32))
    assert (np.diff(np.minimum(filed[order] >> 3, 255).astype(np.int64)) <= 0).all()
    nc = np.zeros((s.grid[1] * 16, s.grid[0] * 16), np.uint32)
    nc[:H, :W] = view_ws(img, im["n_contrib"], H * W, np.uint32).reshape(H, W)
    span = nc.reshape(s.grid[1], 4, 4, s.grid[0], 16).max(axis=(2, 4)).transpose(0, 2, 1).reshape(-1)
    assert np.array_equal(filed == 0, span == 0)
    if R > 0:
        lists = view_ws(binning, _capi.binning_layout(R, W, H)["strip_lists"], 4 * R, np.uint32)
        ranges = st.ranges.astype(np.int64)
        for sid in np.flatnonzero(filed)[:: max(1, int((filed > 0).sum()) // 200)]:   # a sample of strips
            t, w = sid >> 2, sid & 3
            x, n = ranges[t, 0], ranges[t, 1] - ranges[t, 0]
            mine = lists[4 * x + w * n: 4 * x + w * n + filed[sid]] & 0x7FFFFFFF
            assert (np.diff(mine.astype(np.int64)) > 0).all() and mine[-1] == span[sid] - 1 and mine[-1] < n

    # ---- blend: tolerance, away from decision thresholds
    n_contrib = view_ws(img, im["n_contrib"], H * W, np.uint32)
    safe = (st.margin > DECISION_MARGIN).reshape(H, W)
    assert (~safe).mean() <= max_borderline
    for got, want, unit in ((color, st.color, 1.0), (depth, st.depth, max(1.0, float(np.abs(st.depth).max()))), (alpha, st.alpha, 1.0)):
        # colour and alpha are of order one; the depth plane is in scene units, so its bound is relative to the largest depth
        diff = np.abs(got.cpu().numpy() - want)
        assert diff[:, safe].max() <= IMAGE_TOL * unit
        # a borderline pixel may gain or lose one blended Gaussian, nothing more
        assert diff.max() <= 2e-2 * unit
    assert np.array_equal(n_contrib.reshape(H, W)[safe], st.n_contrib.reshape(H, W)[safe])
    # accumulated alpha and remaining transmittance are complementary
    assert float(alpha.min()) >= 0.0 and float(alpha.max()) <= 1.0 + 1e-5
    return st


def _scene_sub(scene, low=None, up=None):
    xyz = scene["xyz"]
    pad = 3.0 * float(scene["scales"].max()) + 1.0
    low = xyz.min(dim=0).values - pad if low is None else low
    up = xyz.max(dim=0).values + pad if up is None else up
    return dict(xyz=xyz, opacity=scene["opacity"], scales=scene["scales"], rotations=scene["rotations"],
                shs=scene["shs"], low=low.float(), up=up.float())


def test_cube_forward_stages():
    scene, cam, _ = scenes.make_config("C0", shrink=5, resolution_scale=0.5)
    _check_forward_stages(_scene_sub(scene), cam, torch.tensor([0.1, 0.2, 0.3]))


def test_cube_at_full_size_forward_and_backward():
    """Config C0 whole: 100 000 Gaussians at 512x512, one submodel, every stage and every gradient."""
    import os
    scene, cam, cfg = scenes.make_config("C0")
    assert cfg["n"] == 100_000 and (cam.image_width, cam.image_height) == (512, 512)
    orc.set_threads(min(16, orc.max_threads(), os.cpu_count() or 1))
    try:
        # a pixel walks some 500 list entries here, each a chance to sit within 2e-5 of a threshold
        st = _check_forward_stages(_scene_sub(scene), cam, torch.tensor([0.1, 0.2, 0.3]), max_borderline=1e-3)
        assert st.R > 400_000
        _check_backward(_scene_sub(scene), cam, torch.tensor([0.1, 0.2, 0.3]), seed=21, with_depth_alpha=True)
    finally:
        orc.set_threads(1)


def test_cube_forward_lower_sh_degrees_and_scale_modifier():
    scene, cam, _ = scenes.make_config("C0", shrink=50, resolution_scale=0.25)
    for deg, mod in ((0, 1.0), (1, 0.7), (2, 1.5)):
        _check_forward_stages(_scene_sub(scene), cam, torch.zeros(3), sh_degree=deg, scale_modifier=mod)


def test_cube_half_box_clips():
    """A box that ends in the middle of the cube: the per-pixel test must clip exactly like the checker."""
    scene, cam, _ = scenes.make_config("C0", shrink=20, resolution_scale=0.5)
    sub = _scene_sub(scene, up=torch.tensor([0.13, 0.4, 4.2]))
    st = _check_forward_stages(sub, cam, torch.zeros(3))
    assert st.counters[3] < st.counters[2]  # some samples were clipped by the box


def test_depths_beyond_the_range_of_three_sort_passes():
    """The depth sort looks at 27 bits of the depth's bit pattern in three passes, which tells depths below 8192
    apart; a scene with Gaussians beyond that makes it run its fourth pass over the remaining bits.  Half of the cube
    is pushed out along the viewing direction, scaled so that it covers the same pixels, to depths of 12 000 to 20 000
    (among them keys that differ only above bit 27 from keys of the near half); the depth order, the lists and the images
    must still be the checker's bit for bit / within tolerance, with the near half alone, the far half alone and both."""
    from retinags_amd import _capi
    scene, cam, _ = scenes.make_config("C0", shrink=30, resolution_scale=0.25)
    n = scene["xyz"].shape[0]
    far = torch.arange(n) % 2 == 1
    eye = cam.camera_center.clone()
    for which in ("both", "far", "near"):
        moved = {k: v.clone() for k, v in scene.items()}
        pick = far if which == "both" else torch.ones(n, dtype=torch.bool) if which == "far" else torch.zeros(n, dtype=torch.bool)
        moved["xyz"][pick] = eye + (scene["xyz"][pick] - eye) * 4000.0
        moved["scales"][pick] = scene["scales"][pick] * 4000.0
        st = _check_forward_stages(_scene_sub(moved), cam, torch.tensor([0.1, 0.2, 0.3]), max_borderline=2e-3)
        if which != "near":
            assert float(st.depths[st.radii > 0].max()) > 8192.0
        assert (st.radii > 0).sum() > n // 2


def test_garden_odd_resolution():
    """Garden-like scene at a resolution that is not a multiple of the tile size."""
    scene, cam, _ = scenes.make_config("C1", shrink=200, resolution_scale=0.2)
    assert cam.image_width % 16 != 0 or cam.image_height % 16 != 0
    _check_forward_stages(_scene_sub(scene), cam, torch.tensor([1.0, 1.0, 1.0]))


def _check_backward(sub, cam, bg, seed, with_depth_alpha, sh_degree=3, scale_modifier=1.0):
    from retinags_amd import GaussianRasterizationSettings, GaussianRasterizer
    dev = torch.device("cuda:0")
    H, W = cam.image_height, cam.image_width
    gen = torch.Generator().manual_seed(seed)
    g_color = torch.randn(3, H, W, generator=gen) * 1e-2
    g_depth = torch.randn(1, H, W, generator=gen) * 1e-2 if with_depth_alpha else None
    g_alpha = torch.randn(1, H, W, generator=gen) * 1e-2 if with_depth_alpha else None

    s = oracle_settings(cam, sub["low"], sub["up"], bg, sh_degree, scale_modifier)
    st = orc.forward(s, np32(sub["xyz"]), np32(sub["opacity"]), shs=np32(sub["shs"]), scales=np32(sub["scales"]),
                     rotations=np32(sub["rotations"]))
    want = orc.backward(s, st, np32(g_color), None if g_depth is None else np32(g_depth),
                        None if g_alpha is None else np32(g_alpha))

    leaf = {k: sub[k].to(dev).clone().requires_grad_(True) for k in ("xyz", "opacity", "scales", "rotations", "shs")}
    means2D = torch.zeros_like(leaf["xyz"], requires_grad=True)
    settings = GaussianRasterizationSettings(
        image_height=H, image_width=W, tanfovx=cam.tanfovx, tanfovy=cam.tanfovy, bg=bg.to(dev),
        scale_modifier=scale_modifier,
        viewmatrix=cam.world_view_transform.to(dev), projmatrix=cam.full_proj_transform.to(dev),
        projmatrix_inv=cam.projection_matrix_inv.to(dev), range_low=sub["low"].to(dev), range_up=sub["up"].to(dev),
        sh_degree=sh_degree, campos=cam.camera_center.to(dev), prefiltered=False, debug=False)
    color, radii, depth, alpha = GaussianRasterizer(settings)(
        means3D=leaf["xyz"], means2D=means2D, opacities=leaf["opacity"], shs=leaf["shs"], scales=leaf["scales"],
        rotations=leaf["rotations"])
    loss = (color * g_color.to(dev)).sum()
    if with_depth_alpha:
        loss = loss + (depth * g_depth.to(dev)).sum() + (alpha * g_alpha.to(dev)).sum()
    loss.backward()
    torch.cuda.synchronize()
    got = dict(means3D=leaf["xyz"].grad, means2D=means2D.grad, sh=leaf["shs"].grad, opacity=leaf["opacity"].grad,
               scales=leaf["scales"].grad, rotations=leaf["rotations"].grad)
    for k, v in got.items():
        err = rel_l2(v.cpu().numpy(), want[k])
        assert err <= GRAD_TOL, f"gradient {k}: relative L2 {err:.3e}"
    # Gaussians that were not rendered get exactly zero
    dead = torch.from_numpy(st.radii <= 0).to(dev)
    for k in ("means3D", "sh", "scales", "rotations", "opacity", "means2D"):
        assert float(got[k][dead].abs().sum()) == 0.0


def test_cube_backward_colour_only():
    scene, cam, _ = scenes.make_config("C0", shrink=10, resolution_scale=0.5)
    _check_backward(_scene_sub(scene), cam, torch.zeros(3), seed=7, with_depth_alpha=False)


def test_cube_backward_all_outputs_with_background_and_box():
    scene, cam, _ = scenes.make_config("C0", shrink=20, resolution_scale=0.5)
    sub = _scene_sub(scene, up=torch.tensor([0.3, 2.0, 4.5]))
    _check_backward(sub, cam, torch.tensor([0.3, 0.6, 0.9]), seed=8, with_depth_alpha=True)


def test_garden_backward():
    scene, cam, _ = scenes.make_config("C1", shrink=400, resolution_scale=0.2)
    _check_backward(_scene_sub(scene), cam, torch.zeros(3), seed=9, with_depth_alpha=True)


@pytest.mark.parametrize("degree,stored", [(0, 16), (1, 16), (2, 16), (1, 4), (0, 1), (2, 9)])
def test_backward_at_lower_sh_degrees_and_fewer_stored_coefficients(degree, stored):
    """The active SH degree may be below 3 (the reference raises it during training,
    scene/gaussian_nn_module.py:399-401) and the SH tensor may hold fewer than 16 coefficients
    (M = sh.size(1), K/rasterize_points.cu:85-89); coefficients beyond the active degree get no gradient."""
    scene, cam, _ = scenes.make_config("C0", shrink=40, resolution_scale=0.4)
    sub = _scene_sub(scene)
    sub["shs"] = sub["shs"][:, :stored].contiguous()
    _check_backward(sub, cam, torch.tensor([0.1, 0.2, 0.3]), seed=10 + degree, with_depth_alpha=True, sh_degree=degree,
                    scale_modifier=0.8)


@pytest.mark.parametrize("width,height,n", [(9, 7, 50), (16, 16, 1), (17, 33, 300), (1, 1, 20), (130, 5, 200)])
def test_tiny_images_and_few_gaussians(width, height, n):
    """One tile, one pixel, one Gaussian, a strip of tiles: every stage and every gradient as at full size."""
    scene = scenes.cube_scene(n, seed=width * 100 + height)
    scene["scales"] = scene["scales"] * 6.0      # wide enough to be seen at these sizes
    cam = scenes.look_at_camera((0.0, 0.0, 0.0), (0.0, 0.0, 4.0), (0, -1, 0), width, height, 60.0)
    sub = _scene_sub(scene)
    _check_forward_stages(sub, cam, torch.tensor([0.2, 0.1, 0.05]))
    _check_backward(sub, cam, torch.tensor([0.2, 0.1, 0.05]), seed=3, with_depth_alpha=True)


@pytest.mark.parametrize("width,height", [(400, 272), (1040, 784)])
def test_gaussians_that_cover_the_whole_image(width, height):
    """Footprints of hundreds of tiles each (one Gaussian keeps a wavefront of the key duplication busy),
    mixed with small ones; faint enough that the lists are walked to the end.  At the larger size a footprint
    has more tiles than one workgroup of the key duplication writes, so several workgroups start inside the
    same Gaussian."""
    scene = scenes.cube_scene(400, seed=77)
    with torch.no_grad():
        scene["scales"][:40] = scene["scales"][:40] * 150.0
        scene["opacity"][:40] = 0.02
    cam = scenes.look_at_camera((0.0, 0.0, 0.0), (0.0, 0.0, 4.0), (0, -1, 0), width, height, 60.0)
    sub = _scene_sub(scene)
    st = _check_forward_stages(sub, cam, torch.tensor([0.0, 0.0, 0.0]))
    tiles = (width // 16) * (height // 16)
    assert (st.tiles_touched[:40] >= tiles // 2).sum() >= 20
    _check_backward(sub, cam, torch.zeros(3), seed=5, with_depth_alpha=True)
