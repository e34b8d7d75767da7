"""Pins the CPU checker (oracle/) against mathematics that does not share its formulas:
float64 matrix algebra, scipy's spherical harmonics, brute-force enumeration, numpy's stable
sort, closed forms, and autograd through an independent differentiable renderer.  The
reference ships no tests or golden vectors for this path, so these pins are what makes the
checker trustworthy; each test names the reference routine it pins."""
import math

import numpy as np
import pytest
import torch

import refmath
from helpers import np32, oracle_settings, orc, rel_l2, scenes

K = "rasterization_kernels/diff-gaussian-rasterization-half-gaussian"


def tiny_scene(n=40, seed=0, W=48, H=40, spread=0.8, log_scale=-1.9, opacity_shift=0.0):
    g = torch.Generator().manual_seed(seed)
    xyz = (torch.rand(n, 3, generator=g) * 2 - 1) * spread
    xyz[:, 2] = xyz[:, 2] * 0.5 + 4.0
    scales = torch.exp(torch.randn(n, 3, generator=g) * 0.3 + log_scale)
    rot = torch.randn(n, 4, generator=g)
    rot = rot / rot.norm(dim=1, keepdim=True)
    opacity = torch.sigmoid(torch.randn(n, 1, generator=g) + opacity_shift)
    shs = torch.randn(n, 16, 3, generator=g) * 0.2
    shs[:, 0] += 0.5
    cam = scenes.look_at_camera((0.1, -0.2, 0.0), (0.0, 0.0, 4.0), (0, -1, 0), W, H, 60.0)
    return dict(xyz=xyz, scales=scales, rotations=rot, opacity=opacity, shs=shs), cam


def cam64(cam):
    d = lambda t: t.double()
    return dict(view_t=d(cam.world_view_transform), proj_t=d(cam.full_proj_transform),
                c2w_t=d(cam.projection_matrix_inv), campos=d(cam.camera_center), tanx=cam.tanfovx, tany=cam.tanfovy)


def big_box():
    return torch.tensor([-50.0, -50.0, -50.0]), torch.tensor([50.0, 50.0, 50.0])


def run_oracle(scene, cam, low, up, bg, **kw):
    s = oracle_settings(cam, low, up, bg, kw.pop("sh_degree", 3), kw.pop("scale_modifier", 1.0))
    st = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]),
                     scales=np32(scene["scales"]), rotations=np32(scene["rotations"]), **kw)
    return s, st


# ---- getHigherMsb (K/cuda_rasterizer_hgs/rasterizer_impl.cu:35-50) ---------------------------

def test_higher_msb_table_and_bruteforce():
    for n, want in ((1024, 11), (6500, 13), (8160, 13), (68250, 17)):
        assert orc.get_higher_msb(n) == want
    for n in list(range(1, 5000)) + [2 ** k + d for k in range(12, 31) for d in (-1, 0, 1)]:
        assert orc.get_higher_msb(n) == n.bit_length()


# ---- projection and near cull (K/cuda_rasterizer_hgs/auxiliary.h:63-82,155-180) ----------------

def test_projection_and_cull_against_float64_matmul():
    scene, cam = tiny_scene(200, seed=1, spread=3.0)
    scene["xyz"][:50, 2] -= 5.0  # push some behind the camera
    low, up = big_box()
    s, st = run_oracle(scene, cam, low, up, torch.zeros(3))
    p_view, p_clip = refmath.project(scene["xyz"].double(), cam.world_view_transform.double(),
                                     cam.full_proj_transform.double())
    vis = st.radii > 0
    assert np.array_equal(orc.mark_visible(s, np32(scene["xyz"])), (p_view[:, 2] > 0.2).numpy())
    assert not vis[(p_view[:, 2] <= 0.2).numpy()].any()
    assert np.allclose(st.depths[vis], p_view[:, 2].numpy()[vis], rtol=1e-6, atol=1e-6)
    assert np.allclose(st.zw[vis], p_clip[:, 2:].numpy()[vis], rtol=1e-6, atol=1e-5)
    ndc = (p_clip[:, :2] / (p_clip[:, 3:] + 1e-7)).numpy()
    pix = np.stack([((ndc[:, 0] + 1) * cam.image_width - 1) / 2, ((ndc[:, 1] + 1) * cam.image_height - 1) / 2], 1)
    assert np.allclose(st.xy[vis], pix[vis], rtol=0, atol=2e-4)


def test_cull_threshold_is_strict():
    cam = scenes.look_at_camera((0, 0, 0), (0, 0, 1), (0, -1, 0), 32, 32, 60.0)
    s = oracle_settings(cam, *big_box(), torch.zeros(3))
    z = np.float32(0.2)
    pts = np.array([[0, 0, z], [0, 0, np.nextafter(z, np.float32(1))], [0, 0, np.nextafter(z, np.float32(0))]], np.float32)
    assert orc.mark_visible(s, pts).tolist() == [False, True, False]


# ---- 3D covariance (K/cuda_rasterizer_hgs/forward.cu:118-152) -----------------------------------

def test_cov3d_closed_form_symmetry_and_identity():
    scene, cam = tiny_scene(100, seed=2)
    scene["rotations"][0] = torch.tensor([1.0, 0, 0, 0])
    _, st = run_oracle(scene, cam, *big_box(), torch.zeros(3), scale_modifier=1.3)
    want = refmath.covariance3d(scene["scales"].double(), scene["rotations"].double(), 1.3).numpy()
    got = st.cov3D
    full = np.stack([got[:, [0, 1, 2]], got[:, [1, 3, 4]], got[:, [2, 4, 5]]], 1)
    vis = st.radii > 0
    assert vis.all()
    assert np.allclose(full, want, rtol=2e-5, atol=2e-8)  # entries are O(1e-2); off-diagonals cancel
    s0 = (1.3 * scene["scales"][0].numpy().astype(np.float32)) ** 2
    assert np.allclose(full[0], np.diag(s0), rtol=1e-6, atol=0)
    assert (np.linalg.eigvalsh(full.astype(np.float64)) > -1e-9).all()


# ---- EWA covariance, conic, radius (K/cuda_rasterizer_hgs/forward.cu:74-113,216-233) -------------

def test_cov2d_conic_radius_against_float64():
    scene, cam = tiny_scene(150, seed=3, spread=1.5)
    W, H = cam.image_width, cam.image_height
    _, st = run_oracle(scene, cam, *big_box(), torch.zeros(3))
    cov3 = refmath.covariance3d(scene["scales"].double(), scene["rotations"].double())
    cov2 = refmath.ewa_cov2d(scene["xyz"].double(), cov3, cam.world_view_transform.double(), W, H, cam.tanfovx,
                             cam.tanfovy).numpy()
    vis = st.radii > 0
    con = st.conic_opacity
    conic = np.stack([con[:, [0, 1]], con[:, [1, 2]]], 1).astype(np.float64)
    eye = conic[vis] @ cov2[vis]
    assert np.allclose(eye, np.eye(2)[None], atol=5e-4)
    assert np.array_equal(con[vis, 3], np32(scene["opacity"])[vis, 0])
    # extent rule: larger eigenvalue with the half-gap between the eigenvalues floored at sqrt(0.1)
    ev = np.linalg.eigvalsh(cov2)
    lam = 0.5 * (ev[:, 0] + ev[:, 1]) + np.sqrt(np.maximum(0.1, (0.5 * (ev[:, 1] - ev[:, 0])) ** 2))
    assert ((0.5 * (ev[:, 1] - ev[:, 0])) ** 2 > 0.1).any() and ((0.5 * (ev[:, 1] - ev[:, 0])) ** 2 < 0.1).any()
    r = np.ceil(3 * np.sqrt(lam))
    # the radius is an integer; float32 vs float64 may differ only where 3*sqrt(lambda) is within rounding of an integer
    frac = np.abs(3 * np.sqrt(lam) - np.round(3 * np.sqrt(lam)))
    sure = vis & (frac > 1e-3)
    assert np.array_equal(st.radii[sure], r[sure].astype(np.int32))


def test_isotropic_gaussian_on_axis_closed_form():
    cam = scenes.look_at_camera((0, 0, 0), (0, 0, 1), (0, -1, 0), 64, 64, 60.0)
    z, s_ = 5.0, 0.2
    scene = dict(xyz=torch.tensor([[0.0, 0.0, z]]), scales=torch.full((1, 3), s_),
                 rotations=torch.tensor([[0.6, 0.0, 0.8, 0.0]]), opacity=torch.tensor([[0.5]]),
                 shs=torch.zeros(1, 16, 3))
    _, st = run_oracle(scene, cam, *big_box(), torch.zeros(3))
    f = 64 / (2 * math.tan(math.radians(30)))
    var = (s_ * f / z) ** 2 + 0.3
    assert np.allclose(st.conic_opacity[0, [0, 2]], 1 / var, rtol=1e-5)
    assert abs(st.conic_opacity[0, 1]) < 1e-6
    # equal eigenvalues: the extent rule floors their half-gap at sqrt(0.1)
    assert st.radii[0] == math.ceil(3 * math.sqrt(var + math.sqrt(0.1))) == 8
    assert np.allclose(st.xy[0], [31.5, 31.5], atol=1e-5)


# ---- spherical harmonics (K/cuda_rasterizer_hgs/auxiliary.h:22-39, forward.cu:20-71) --------------

def test_sh_basis_matches_scipy_harmonics():
    g = np.random.default_rng(0)
    dirs = g.normal(size=(24, 3))
    dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
    want = refmath.real_sh_basis(dirs, 3)
    # a negative basis value is clamped to 0 by the colour stage: offset by a DC term instead
    n = dirs.shape[0]
    cam = scenes.look_at_camera((0, 0, 0), (0, 0, 1), (0, -1, 0), 64, 64, 60.0)
    s = oracle_settings(cam, *big_box(), torch.zeros(3), sh_degree=3)
    pts = np.tile(np.array([[0.0, 0.0, 3.0]], np.float32), (n, 1))
    c0 = 0.28209479177387814
    for k in range(1, 16):
        for i in range(n):
            shs = np.zeros((1, 16, 3), np.float32)
            shs[0, 0, :] = 4.0          # +4*C0 keeps every channel positive
            shs[0, k, 0] = 1.0
            s.campos = (pts[i] - dirs[i].astype(np.float32) * 2.0).astype(np.float32)
            pre = orc.preprocess(s, pts[i:i + 1], np.ones(1, np.float32), shs=shs,
                                 scales=np.full((1, 3), 0.05, np.float32),
                                 rotations=np.array([[1, 0, 0, 0]], np.float32))
            assert not pre["clamped"].any()
            d = (pts[i] - s.campos).astype(np.float64)
            d /= np.linalg.norm(d)
            basis = refmath.real_sh_basis(d[None], 3)[0]
            got = float(pre["rgb"][0, 0]) - 0.5 - 4.0 * c0
            assert abs(got - basis[k]) < 5e-6, (k, i, got, basis[k])
            assert abs(float(pre["rgb"][0, 1]) - 0.5 - 4.0 * c0) < 5e-7


def test_sh_basis_is_orthonormal_under_quadrature():
    """Every constant of the table is pinned by <Y_i, Y_j> = delta_ij on the sphere."""
    nodes, weights = np.polynomial.legendre.leggauss(12)
    phis = (np.arange(24) + 0.5) * (2 * np.pi / 24)
    dirs, w = [], []
    for ct, wt in zip(nodes, weights):
        st_ = math.sqrt(1 - ct * ct)
        for ph in phis:
            dirs.append([st_ * math.cos(ph), st_ * math.sin(ph), ct])
            w.append(wt * 2 * np.pi / 24)
    dirs, w = np.array(dirs), np.array(w)
    B = refmath.sh_polynomials(torch.from_numpy(dirs)).numpy()
    gram = (B * w[:, None]).T @ B
    assert np.allclose(gram, np.eye(16), atol=1e-10)
    assert np.allclose(B, refmath.real_sh_basis(dirs, 3), atol=1e-12)


def test_sh_degree0_and_clamp_flags():
    scene, cam = tiny_scene(60, seed=4)
    scene["shs"][:30, 0, :] = -3.0  # strongly negative DC -> clamped to 0
    _, st = run_oracle(scene, cam, *big_box(), torch.zeros(3), sh_degree=0)
    want = 0.28209479177387814 * np32(scene["shs"])[:, 0, :] + 0.5
    assert np.allclose(st.rgb, np.maximum(want, 0), atol=1e-6)
    assert np.array_equal(st.clamped.astype(bool), want < 0)
    assert st.clamped[:30].all() and (st.rgb[:30] == 0).all()


# ---- tile rectangles, keys, sort, ranges (K/cuda_rasterizer_hgs/auxiliary.h:51-61,
#      rasterizer_impl.cu:70-138,283,309-323) ---------------------------------------------------------

def test_tile_rects_keys_sort_and_ranges_bruteforce():
    scene, cam = tiny_scene(80, seed=5, W=70, H=52, spread=1.6, log_scale=-1.6)
    W, H = cam.image_width, cam.image_height
    s, st = run_oracle(scene, cam, *big_box(), torch.zeros(3))
    gx, gy = s.grid
    T = gx * gy
    vis = np.nonzero(st.radii > 0)[0]
    # independent enumeration of the tiles of every visible Gaussian
    expect_keys, expect_vals = [], []
    for i in range(st.P):
        if st.radii[i] <= 0:
            assert st.tiles_touched[i] == 0
            continue
        x0, y0, x1, y1 = refmath.tile_rect_bruteforce(float(st.xy[i, 0]), float(st.xy[i, 1]), int(st.radii[i]), W, H)
        assert st.tiles_touched[i] == (x1 - x0) * (y1 - y0) > 0
        dbits = int(st.depths[i:i + 1].view(np.uint32)[0])
        for y in range(y0, y1):
            for x in range(x0, x1):
                expect_keys.append(((y * gx + x) << 32) | dbits)
                expect_vals.append(i)
    assert len(vis) > 10
    assert np.array_equal(st.point_offsets, np.cumsum(st.tiles_touched.astype(np.uint64)).astype(np.uint32))
    assert st.R == len(expect_keys) == int(st.tiles_touched.sum())
    assert np.array_equal(st.keys_unsorted, np.array(expect_keys, np.uint64))
    assert np.array_equal(st.values_unsorted, np.array(expect_vals, np.uint32))
    order = np.argsort(st.keys_unsorted, kind="stable")
    assert np.array_equal(st.keys, st.keys_unsorted[order])
    assert np.array_equal(st.point_list, st.values_unsorted[order])
    # ranges partition [0, R) in tile order; untouched tiles stay (0, 0)
    tiles = (st.keys >> np.uint64(32)).astype(np.int64)
    cursor = 0
    for t in range(T):
        cnt = int((tiles == t).sum())
        if cnt == 0:
            assert tuple(st.ranges[t]) == (0, 0)
        else:
            assert tuple(st.ranges[t]) == (cursor, cursor + cnt)
            cursor += cnt
            seg = st.point_list[st.ranges[t, 0]:st.ranges[t, 1]]
            d = st.depths[seg]
            assert (np.diff(d) >= 0).all()
    assert cursor == st.R


def test_sort_pairs_is_stable_and_masks_high_bits():
    g = np.random.default_rng(1)
    for n, end_bit in ((0, 40), (1, 40), (1000, 43), (5000, 45), (4097, 49), (3000, 8), (3000, 1), (2000, 64)):
        keys = g.integers(0, 2 ** 63, size=n, dtype=np.uint64)
        keys[: n // 2] &= np.uint64(0xFFFF)  # many ties in the compared bits
        vals = np.arange(n, dtype=np.uint32)
        ko, vo = orc.sort_pairs(keys, vals, end_bit)
        mask = np.uint64((1 << end_bit) - 1) if end_bit < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
        order = np.argsort(keys & mask, kind="stable")
        assert np.array_equal(ko, keys[order]) and np.array_equal(vo, vals[order])


def test_inclusive_sum_wraps_like_uint32():
    x = np.array([4000000000, 500000000, 7, 0, 1], np.uint32)
    assert np.array_equal(orc.inclusive_sum(x), np.cumsum(x.astype(np.uint64)).astype(np.uint32))


# ---- forward blend (K/cuda_rasterizer_hgs/forward.cu:263-405) -----------------------------------------

def _reference_render(scene, cam, low, up, bg, grad=False):
    p = {k: v.double().clone().requires_grad_(grad) for k, v in scene.items()}
    out = refmath.render_reference(p, cam64(cam), cam.image_width, cam.image_height, low.double(), up.double(),
                                   bg.double())
    return p, out


def test_forward_blend_matches_independent_float64_renderer():
    scene, cam = tiny_scene(40, seed=6)
    low, up = big_box()
    bg = torch.tensor([0.2, 0.5, 0.7])
    _, st = run_oracle(scene, cam, low, up, bg)
    _, (color, depth, alpha, aux) = _reference_render(scene, cam, low, up, bg)
    assert np.array_equal(st.radii, aux["radius"].numpy().astype(np.int32) * aux["visible"].numpy())
    assert np.abs(st.color - color.numpy()).max() < 2e-5
    assert np.abs(st.depth - depth.numpy()).max() < 1e-4
    assert np.abs(st.alpha - alpha.numpy()).max() < 2e-5
    assert st.alpha.max() > 0.5  # the scene really covers pixels


def test_half_gaussian_box_clips_like_independent_renderer():
    scene, cam = tiny_scene(40, seed=7)
    low, up = torch.tensor([-50.0, -50.0, -50.0]), torch.tensor([0.07, 50.0, 4.1])
    bg = torch.zeros(3)
    _, st = run_oracle(scene, cam, low, up, bg)
    _, (color, depth, alpha, _) = _reference_render(scene, cam, low, up, bg)
    assert np.abs(st.color - color.numpy()).max() < 2e-5
    assert np.abs(st.alpha - alpha.numpy()).max() < 2e-5
    assert 0 < st.counters[3] < st.counters[2]
    # a box that contains no ray sample at all leaves only the background
    _, st0 = run_oracle(scene, cam, torch.tensor([60.0, 60, 60]), torch.tensor([70.0, 70, 70]), torch.tensor([0.3, 0.2, 0.1]))
    assert st0.counters[3] == 0 and (st0.alpha == 0).all() and (st0.n_contrib == 0).all()
    assert np.allclose(st0.color, np.array([0.3, 0.2, 0.1], np.float32)[:, None, None])


def test_two_complementary_boxes_compose_to_the_unclipped_image():
    """The property the half-Gaussian test exists for: partial images of a split scene,
    composited front to back, reproduce the unsplit render (up to the per-image
    early-termination threshold)."""
    scene, cam = tiny_scene(40, seed=8, opacity_shift=-1.0)
    bg = torch.zeros(3)
    cut = 4.0
    _, whole = run_oracle(scene, cam, *big_box(), bg)
    near_ids = (scene["xyz"][:, 2] <= cut).numpy()
    pad = 3.0 * float(scene["scales"].max())
    reach_far = (scene["xyz"][:, 2] + pad > cut).numpy()
    reach_near = (scene["xyz"][:, 2] - pad <= cut).numpy()
    sub = lambda m: {k: v[torch.from_numpy(m)] for k, v in scene.items()}
    _, a = run_oracle(sub(near_ids | reach_near), cam, torch.tensor([-50.0, -50, -50]), torch.tensor([50.0, 50, cut]), bg)
    _, b = run_oracle(sub(~near_ids | reach_far), cam, torch.tensor([-50.0, -50, cut]), torch.tensor([50.0, 50, 50]), bg)
    img, dep, alp = orc.composite_forward([a.color, b.color], [a.depth, b.depth], [a.alpha, b.alpha], np.zeros(3))
    assert np.abs(img - whole.color).max() < 2e-3
    assert np.abs(alp - whole.alpha).max() < 2e-3


def test_single_gaussian_closed_form_and_alpha_transmittance_identity():
    cam = scenes.look_at_camera((0, 0, 0), (0, 0, 1), (0, -1, 0), 33, 33, 60.0)
    # pixel (16,16) is the exact image centre of a 33x33 image
    scene = dict(xyz=torch.tensor([[0.0, 0.0, 3.0]]), scales=torch.full((1, 3), 0.3),
                 rotations=torch.tensor([[1.0, 0, 0, 0]]), opacity=torch.tensor([[0.7]]), shs=torch.zeros(1, 16, 3))
    scene["shs"][0, 0] = torch.tensor([1.0, 0.5, -0.5])
    bg = torch.tensor([0.1, 0.2, 0.3])
    _, st = run_oracle(scene, cam, *big_box(), bg)
    c = np.maximum(0.28209479177387814 * np.array([1.0, 0.5, -0.5]) + 0.5, 0)
    want = 0.7 * c + 0.3 * bg.numpy()
    assert np.allclose(st.color[:, 16, 16], want, atol=1e-6)
    assert abs(st.alpha[0, 16, 16] - 0.7) < 1e-6
    assert abs(st.depth[0, 16, 16] - 0.7 * 3.0) < 1e-5
    # opacity 1.0 is clamped to 0.99 at the centre
    scene["opacity"][0, 0] = 1.0
    _, st = run_oracle(scene, cam, *big_box(), bg)
    assert abs(st.alpha[0, 16, 16] - 0.99) < 1e-6
    # accumulated alpha + product of (1 - alpha) = 1
    scene2, cam2 = tiny_scene(30, seed=9)
    _, st2 = run_oracle(scene2, cam2, *big_box(), torch.ones(3))
    s2 = oracle_settings(cam2, *big_box(), torch.zeros(3))
    st0 = orc.forward(s2, np32(scene2["xyz"]), np32(scene2["opacity"]), shs=np32(scene2["shs"]),
                      scales=np32(scene2["scales"]), rotations=np32(scene2["rotations"]))
    # with a white background colour = C + T, with black colour = C: their difference is T
    assert np.allclose((st2.color - st0.color)[0] + st0.alpha[0], 1.0, atol=1e-5)


# ---- backward (K/cuda_rasterizer_hgs/backward.cu:144-622) -------------------------------------------------

def _oracle_vs_autograd(scene, cam, low, up, bg, seed, with_aux_outputs):
    H, W = cam.image_height, cam.image_width
    g = torch.Generator().manual_seed(seed)
    g_color = torch.randn(3, H, W, generator=g, dtype=torch.float64)
    g_depth = torch.randn(1, H, W, generator=g, dtype=torch.float64) if with_aux_outputs else None
    g_alpha = torch.randn(1, H, W, generator=g, dtype=torch.float64) if with_aux_outputs else None
    s, st = run_oracle(scene, cam, low, up, bg)
    got = orc.backward(s, st, np32(g_color), None if g_depth is None else np32(g_depth),
                       None if g_alpha is None else np32(g_alpha))
    p, (color, depth, alpha, aux) = _reference_render(scene, cam, low, up, bg, grad=True)
    loss = (color * g_color).sum()
    if with_aux_outputs:
        loss = loss + (depth * g_depth).sum() + (alpha * g_alpha).sum()
    loss.backward()
    pairs = (("means3D", "xyz"), ("opacity", "opacity"), ("scales", "scales"), ("rotations", "rotations"), ("sh", "shs"))
    errs = {a: rel_l2(got[a], p[b].grad.numpy()) for a, b in pairs}
    # The screen-space gradient the rasterizer hands back is taken with respect to the NDC position through the blend
    # alone (K/cuda_rasterizer_hgs/backward.cu:496-497, 610-611: dL/ddelta times 0.5 W, 0.5 H); the independent
    # renderer's pixel centre is (ndc + 1) * 0.5 * (W, H) - 0.5 and only its blend reads it, so dL/dmean2D =
    # 0.5 (W, H) dL/dpixel-centre, and the third column stays zero.
    H, W = cam.image_height, cam.image_width
    d_pix = aux["pix_node"].grad.numpy()
    want_2d = np.concatenate([d_pix * np.array([0.5 * W, 0.5 * H]), np.zeros((d_pix.shape[0], 1))], axis=1)
    errs["means2D"] = rel_l2(got["means2D"], want_2d)
    return errs, got, st


def test_backward_matches_autograd_colour_only():
    scene, cam = tiny_scene(30, seed=10)
    errs, got, st = _oracle_vs_autograd(scene, cam, *big_box(), torch.zeros(3), 1, False)
    assert max(errs.values()) < 1e-3, errs
    assert np.abs(got["means3D"]).sum() > 0 and np.abs(got["rotations"]).sum() > 0


def test_backward_matches_autograd_all_outputs_background_and_box():
    scene, cam = tiny_scene(30, seed=11)
    low, up = torch.tensor([-50.0, -50.0, -50.0]), torch.tensor([0.2, 50.0, 4.2])
    errs, got, st = _oracle_vs_autograd(scene, cam, low, up, torch.tensor([0.9, 0.1, 0.4]), 2, True)
    assert max(errs.values()) < 1e-3, errs


def test_backward_straight_through_clamp():
    """alpha = min(0.99, o G) passes gradients as if it were not clamped
    (K/cuda_rasterizer_hgs/backward.cu:537,603-619); the independent renderer models it with
    a straight-through estimator."""
    scene, cam = tiny_scene(12, seed=12, log_scale=-1.2)
    scene["opacity"][:] = 0.9999
    errs, got, st = _oracle_vs_autograd(scene, cam, *big_box(), torch.zeros(3), 3, True)
    assert st.alpha.max() > 0.98
    assert max(errs.values()) < 1e-3, errs


def test_backward_outside_the_guard_frustum():
    """Gaussians whose centre lies beyond 1.3 x the field of view but whose footprint still reaches
    the image: the forward clamps the view-space x / y it linearises around, and the backward treats
    the clamped value as a constant (K/cuda_rasterizer_hgs/backward.cu:168-176, 262-264).  The
    independent renderer models exactly that with a detached clamp."""
    scene, cam = tiny_scene(24, seed=13, log_scale=-1.0)
    with torch.no_grad():
        z = scene["xyz"][:, 2]
        # half of them far off to the sides and above / below, large enough to be seen
        scene["xyz"][0:6, 0] = 1.6 * cam.tanfovx * z[0:6] * torch.tensor([1, -1, 1, -1, 1, -1.0])
        scene["xyz"][6:12, 1] = 1.5 * cam.tanfovy * z[6:12] * torch.tensor([1, -1, 1, -1, 1, -1.0])
        scene["scales"][0:12] = scene["scales"][0:12] * 2.5
    view = np32(scene["xyz"]) @ cam.world_view_transform.numpy()[:3, :3] + cam.world_view_transform.numpy()[3, :3]
    outside = (np.abs(view[:, 0] / view[:, 2]) > 1.3 * cam.tanfovx) | (np.abs(view[:, 1] / view[:, 2]) > 1.3 * cam.tanfovy)
    errs, got, st = _oracle_vs_autograd(scene, cam, *big_box(), torch.tensor([0.2, 0.2, 0.2]), 4, True)
    seen_outside = outside & (st.radii > 0)
    assert seen_outside.sum() >= 6
    # they do take part: their gradients are not zero
    assert np.abs(got["means3D"][seen_outside]).sum() > 0 and np.abs(got["scales"][seen_outside]).sum() > 0
    assert max(errs.values()) < 1e-3, errs


# ---- compositor (parallel_utils/basic_parallel_trainer/result_aggregator.py:244-259) -------------------

def _torch_composite(images, depths, alphas, bg):
    """The reference expression, rewritten in float64: transmittance by cumulative product."""
    a = torch.stack([torch.zeros_like(alphas[0])] + list(alphas), 0)
    T = torch.cumprod(1 - a, 0)
    img = (T[:-1] * torch.stack(list(images), 0)).sum(0) + bg.view(3, 1, 1) * T[-1]
    dep = (T[:-1] * torch.stack(list(depths), 0)).sum(0)
    return img, dep, 1 - T[-1]


@pytest.mark.parametrize("Kn", [1, 2, 4, 16, 33])
def test_composite_forward_backward_against_autograd(Kn):
    g = torch.Generator().manual_seed(Kn)
    H, W = 9, 13
    imgs = [torch.rand(3, H, W, generator=g, dtype=torch.float64).requires_grad_(True) for _ in range(Kn)]
    deps = [torch.rand(1, H, W, generator=g, dtype=torch.float64).requires_grad_(True) for _ in range(Kn)]
    alps = [torch.rand(1, H, W, generator=g, dtype=torch.float64).requires_grad_(True) for _ in range(Kn)]
    alps[0].data[0, 0, 0] = 1.0  # fully opaque first layer at one pixel
    bg = torch.tensor([0.3, 0.6, 0.9], dtype=torch.float64)
    img, dep, alp = _torch_composite(imgs, deps, alps, bg)
    gi, gd, ga = (torch.randn_like(t) for t in (img, dep, alp))
    (img * gi).sum().add((dep * gd).sum()).add((alp * ga).sum()).backward()
    n = lambda ts: [np32(t) for t in ts]
    oi, od, oa = orc.composite_forward(n(imgs), n(deps), n(alps), np32(bg))
    assert np.abs(oi - img.detach().numpy()).max() < 1e-5
    assert np.abs(od - dep.detach().numpy()).max() < 1e-5
    assert np.abs(oa - alp.detach().numpy()).max() < 1e-5
    di, dd, da = orc.composite_backward(n(imgs), n(deps), n(alps), np32(bg), np32(gi), np32(gd), np32(ga))
    for k in range(Kn):
        assert rel_l2(di[k], imgs[k].grad.numpy()) < 1e-5
        assert rel_l2(dd[k], deps[k].grad.numpy()) < 1e-5
        assert rel_l2(da[k], alps[k].grad.numpy()) < 1e-5


def test_composite_single_layer_is_identity_and_grouping_is_associative():
    g = np.random.default_rng(3)
    H, W = 6, 7
    mk = lambda c: g.random((c, H, W), dtype=np.float32)
    A, B, Cc = [(mk(3), mk(1), mk(1)) for _ in range(3)]
    z = np.zeros(3, np.float32)
    i1, d1, a1 = orc.composite_forward([A[0]], [A[1]], [A[2]], z)
    assert np.array_equal(i1, A[0]) and np.array_equal(d1, A[1]) and np.allclose(a1, A[2], atol=1e-7)
    full = orc.composite_forward([A[0], B[0], Cc[0]], [A[1], B[1], Cc[1]], [A[2], B[2], Cc[2]], z)
    bc = orc.composite_forward([B[0], Cc[0]], [B[1], Cc[1]], [B[2], Cc[2]], z)
    nested = orc.composite_forward([A[0], bc[0]], [A[1], bc[1]], [A[2], bc[2]], z)
    for x, y in zip(full, nested):
        assert np.abs(x - y).max() < 1e-6
