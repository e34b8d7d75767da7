"""Size-independent properties of the HIP path at the full benchmark shapes, where the CPU
checker would take too long: structure of the binning output (sortedness, stability,
range partition, counts), determinism, and exact linearity of the rendered loss in the SH
DC coefficients (a finite-difference check of dL/dSH that needs no oracle).  Config names are
those of retinags_amd.harness.scenes.CONFIGS."""
import numpy as np
import pytest
import torch

from helpers import check_binning_against, scenes, view_ws

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _forward_raw(sub, cam_d, cam, bg):
    from retinags_amd import rasterizer as R
    e = torch.Tensor([])
    return R._rasterize_forward(bg, sub.means3D.detach(), e, sub.opacity.detach(), sub.scales.detach(),
                                sub.rotations.detach(), 1.0, e, cam_d.world_view_transform, cam_d.full_proj_transform,
                                cam_d.projection_matrix_inv, sub.range_low, sub.range_up, cam.tanfovx, cam.tanfovy,
                                cam.image_height, cam.image_width, sub.shs.detach(), 3, cam_d.camera_center, False, False)


def _check_binning_structure(outs, P, W, H):
    """Sorted keys, stable ties, ranges that partition [0, R), counts that add up."""
    from retinags_amd import _capi
    Rn, color, depth, alpha, radii, geom, binning, img = outs
    gx, gy = (W + 15) // 16, (H + 15) // 16
    T = gx * gy
    g = _capi.geom_layout(P)
    radii = radii.cpu().numpy()
    touched = view_ws(geom, g["tiles_touched"], P, np.uint32)
    n_vis = int(view_ws(geom, g["visible_count"], 1, np.uint32)[0])
    offsets = view_ws(geom, g["point_offsets"], P, np.uint32)[:n_vis]
    order = view_ws(geom, g["depth_order"], P, np.uint32)[:n_vis]
    depth_bits = view_ws(geom, g["depths"], P, np.uint32)
    assert int(touched.astype(np.int64).sum()) == Rn
    assert np.array_equal(np.sort(order), np.flatnonzero(touched != 0).astype(np.uint32))   # the visible ones, once each
    assert (np.diff(depth_bits[order].astype(np.int64)) >= 0).all()                         # by depth
    assert np.array_equal(offsets, np.cumsum(touched[order].astype(np.uint64)).astype(np.uint32))
    assert np.array_equal(radii > 0, touched > 0)
    if Rn == 0:
        return
    b = _capi.binning_layout(Rn, W, H)
    vals = view_ws(binning, b["values_sorted"], Rn, np.uint32)
    # the reference's 64-bit keys, rebuilt: the tile the sort used and the Gaussian's depth bits
    keys = (view_ws(binning, b["keys_sorted"], Rn, np.uint32).astype(np.uint64) << np.uint64(32)) | \
        depth_bits[vals].astype(np.uint64)
    assert (np.diff(keys.astype(np.uint64).view(np.int64)) >= 0).all()          # sorted (keys < 2^63)
    same = keys[1:] == keys[:-1]
    assert (vals[1:][same] > vals[:-1][same]).all()                             # ties keep emission order
    assert int(vals.max()) < P and (radii[vals] > 0).all()
    depths = view_ws(geom, g["depths"], P, np.uint32)
    assert np.array_equal((keys & np.uint64(0xFFFFFFFF)).astype(np.uint32), depths[vals])
    tiles = (keys >> np.uint64(32)).astype(np.int64)
    assert tiles.max() < T
    per_gaussian = np.bincount(vals, minlength=P)
    assert np.array_equal(per_gaussian.astype(np.uint32), touched)
    im = _capi.image_layout(W, H)
    ranges = view_ws(img, im["ranges"], 2 * T, np.uint32).reshape(T, 2).astype(np.int64)
    counts = np.bincount(tiles, minlength=T)
    nz = counts > 0
    assert np.array_equal(ranges[nz, 1] - ranges[nz, 0], counts[nz])
    assert (ranges[~nz] == 0).all()
    starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
    assert np.array_equal(ranges[nz, 0], starts[nz])
    n_contrib = view_ws(img, im["n_contrib"], W * H, np.uint32).reshape(H, W)
    tile_len = (ranges[:, 1] - ranges[:, 0]).reshape(gy, gx)
    cap = np.repeat(np.repeat(tile_len, 16, axis=0), 16, axis=1)[:H, :W]
    assert (n_contrib <= cap).all()
    a = alpha.cpu().numpy()
    assert np.isfinite(color.cpu().numpy()).all() and a.min() >= 0.0 and a.max() <= 1.0 + 1e-5
    assert ((n_contrib == 0) == (a[0] == 0)).all()


def _frame_setup(name, shrink, resolution_scale=1.0):
    from retinags_amd.harness import partition, pipeline
    scene, cam, cfg = scenes.make_config(name, "cpu", shrink, resolution_scale)
    if cfg["bvh_depth"] > 0:
        part = partition.partition_scene(scene["xyz"], scene["scales"], cfg["bvh_depth"])
        rel = partition.relation_vector(part, cam)
        subs = pipeline.submodels_from_partition(scene, part, DEV)
    else:
        rel = np.zeros(1, dtype=np.int64)
        subs = [pipeline.whole_scene_submodel(scene, DEV)]
    return scene, cam, cfg, subs, rel


def _sh_linearity(cam, subs, rel, which, seed):
    """The rendered loss <image, g> is exactly linear in the DC SH coefficients of Gaussians
    whose colour stays positive, so a plain difference of two renders must equal the
    directional derivative given by dL/dSH."""
    from retinags_amd.harness import pipeline
    cam_d = cam.to(DEV)
    H, W = cam.image_height, cam.image_width
    gen = torch.Generator().manual_seed(seed)
    g = (torch.randn(3, H, W, generator=gen) * 1e-2).to(DEV)
    bg = torch.zeros(3, device=DEV)
    for s_ in subs:
        s_.requires_grad_(True)
    out = pipeline.render_frame(cam_d, subs, rel, bg)
    loss0 = (out["render"].detach().double() * g.double()).sum()
    torch.autograd.backward([out["render"]], [g])
    if which is None:  # the submodel with the most rendered Gaussians
        which = max(out["partial"], key=lambda m: int((out["partial"][m]["radii"] > 0).sum()))
    sub = subs[which]
    rendered = out["partial"][which]["radii"] > 0
    grad = sub.shs.grad.clone()
    # Gaussians whose three colour channels are clearly positive are not clamped, and a positive DC
    # offset keeps them so; their colour is then exactly affine in the DC coefficients.
    from retinags_amd import _capi
    P = sub.means3D.shape[0]
    raw = _forward_raw(sub, cam_d, cam, bg)
    rgb = torch.from_numpy(view_ws(raw[5], _capi.geom_layout(P)["rgb"], 3 * P, np.float32).reshape(P, 3).copy()).to(DEV)
    safe = rendered & (rgb.min(dim=1).values > 0.05)
    del raw
    assert int(safe.sum()) > 100
    v = torch.zeros_like(sub.shs)
    v[safe, 0, :] = torch.rand(int(safe.sum()), 3, generator=gen).to(DEV) * 0.5
    with torch.no_grad():
        sub.shs += v
        out1 = pipeline.render_frame(cam_d, subs, rel, bg)
        loss1 = (out1["render"].detach().double() * g.double()).sum()
        sub.shs -= v
    predicted = (grad.double() * v.double()).sum()
    measured = loss1 - loss0
    # The backward recovers each pixel's transmittance from 1 - sum(alpha T) by repeated division
    # (K/cuda_rasterizer_hgs/backward.cu:469,555); on saturated pixels that difference has only a
    # few significant bits, so the property holds to about a percent, not to rounding.
    assert abs(float(measured)) > 1e-6
    assert abs(float(measured - predicted)) <= 2e-2 * abs(float(measured)) + 1e-7
    for s in subs:
        s.requires_grad_(False)
        for t in s.parameters():
            t.grad = None


def test_garden_full_size_structure_determinism_and_sh_linearity():
    """Config C1 at full size: 5.6 M Gaussians, 1600x1036, 4 submodels."""
    scene, cam, cfg, subs, rel = _frame_setup("C1", 1.0)
    cam_d = cam.to(DEV)
    bg = torch.zeros(3, device=DEV)
    total = 0
    for m, sub in enumerate(subs):
        if rel[m] < 0:
            continue
        outs = _forward_raw(sub, cam_d, cam, bg)
        _check_binning_structure(outs, sub.means3D.shape[0], cam.image_width, cam.image_height)
        again = _forward_raw(sub, cam_d, cam, bg)
        assert outs[0] == again[0]
        for k in (1, 2, 3, 4):
            assert torch.equal(outs[k], again[k])          # the forward is deterministic, bit for bit
        total += outs[0]
    assert total > 5_000_000
    _sh_linearity(cam, subs, rel, which=None, seed=3)


def test_garden_full_size_against_checker():
    """Config C1 at full size, the two heaviest kinds of submodel, against the CPU checker
    (OpenMP makes it fast enough): bit-exact binning, images, every gradient."""
    from helpers import DECISION_MARGIN, GRAD_TOL, IMAGE_TOL, np32, orc, rel_l2
    from retinags_amd.harness import partition, pipeline
    from retinags_amd import _capi
    import os
    scene, cam, cfg = scenes.make_config("C1", "cpu", 1.0)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    subs = pipeline.submodels_from_partition(scene, part, DEV)
    H, W = cam.image_height, cam.image_width
    g = (torch.randn(3, H, W, generator=torch.Generator().manual_seed(11)) * 1e-2)
    xyz, opa, sc, rot, shs = (np32(scene[k]) for k in ("xyz", "opacity", "scales", "rotations", "shs"))
    orc.set_threads(min(16, orc.max_threads(), os.cpu_count() or 1))
    try:
        for m in (0, 2):
            ids = part.members[m]
            s = orc.settings_from_camera(cam, part.box_low[m], part.box_up[m], torch.zeros(3))
            st = orc.forward(s, xyz[ids], opa[ids], shs=shs[ids], scales=sc[ids], rotations=rot[ids], want_margin=True)
            want = orc.backward(s, st, np32(g))
            sub = subs[m].requires_grad_(True)
            raw = _forward_raw(sub, cam.to(DEV), cam, torch.zeros(3, device=DEV))
            assert raw[0] == st.R
            check_binning_against(st, raw[5], raw[6], st.P, st.R, W, H)
            assert np.array_equal(view_ws(raw[7], _capi.image_layout(W, H)["ranges"], 2 * len(st.ranges), np.uint32),
                                  st.ranges.ravel())
            del raw
            out = pipeline.render_submodel(cam.to(DEV), sub, torch.zeros(3, device=DEV))
            torch.autograd.backward([out["render"]], [g.to(DEV)])
            assert np.array_equal(out["radii"].cpu().numpy(), st.radii)
            safe = (st.margin > DECISION_MARGIN).reshape(H, W)
            assert (~safe).mean() < 1e-3
            assert np.abs(out["render"].detach().cpu().numpy() - st.color)[:, safe].max() <= IMAGE_TOL
            assert np.abs(out["alpha"].detach().cpu().numpy() - st.alpha)[:, safe].max() <= IMAGE_TOL
            for key, t in (("means3D", sub.means3D), ("sh", sub.shs), ("opacity", sub.opacity), ("scales", sub.scales),
                           ("rotations", sub.rotations)):
                assert rel_l2(t.grad.cpu().numpy(), want[key]) <= GRAD_TOL, (m, key)
            sub.requires_grad_(False)
            for t in sub.parameters():
                t.grad = None
    finally:
        orc.set_threads(1)


def test_high_resolution_seven_pass_sort():
    """Config C2's image (5185x3359: 68 250 tiles, 49-bit keys, 7 radix passes) with a tenth of the Gaussians."""
    from retinags_amd import _capi
    scene, cam, cfg, subs, rel = _frame_setup("C2", 10.0)
    assert _capi.lib.rgs_get_higher_msb(((cam.image_width + 15) // 16) * ((cam.image_height + 15) // 16)) == 17
    cam_d = cam.to(DEV)
    bg = torch.zeros(3, device=DEV)
    for m, sub in enumerate(subs):
        if rel[m] >= 0:
            _check_binning_structure(_forward_raw(sub, cam_d, cam, bg), sub.means3D.shape[0], cam.image_width,
                                     cam.image_height)
    _sh_linearity(cam, subs, rel, which=None, seed=4)


def test_sixteen_submodels_dense_scene():
    """Config C3's partition (bvh_depth 4, 16 submodels, shrunk scales) with a twentieth of the Gaussians."""
    from retinags_amd.harness import pipeline
    scene, cam, cfg, subs, rel = _frame_setup("C3", 20.0)
    assert len(subs) == 16
    cam_d = cam.to(DEV)
    bg = torch.tensor([0.1, 0.2, 0.3], device=DEV)
    for m in (0, 7, 15):
        if rel[m] >= 0:
            _check_binning_structure(_forward_raw(subs[m], cam_d, cam, torch.zeros(3, device=DEV)),
                                     subs[m].means3D.shape[0], cam.image_width, cam.image_height)
    out = pipeline.render_frame(cam_d, subs, rel, bg)
    a = out["alpha"]
    assert torch.isfinite(out["render"]).all() and float(a.min()) >= 0 and float(a.max()) <= 1 + 1e-5
    # transmittance left after all layers shows the background: image = sum + bg * (1 - alpha)
    partial = [out["partial"][m] for m in sorted((m for m in range(16) if rel[m] >= 0), key=lambda m: rel[m])]
    T = torch.ones_like(a)
    acc = torch.zeros_like(out["render"])
    for pk in partial:
        acc += T * pk["render"]
        T = T * (1 - pk["alpha"])
    assert torch.allclose(out["render"], acc + bg.view(3, 1, 1) * T, atol=1e-5)
    assert torch.allclose(a, 1 - T, atol=1e-6)
    _sh_linearity(cam, subs, rel, which=None, seed=5)


def test_city_forward_only_thirty_two_submodels():
    """Config C4's partition (bvh_depth 5, 32 submodels, 1920x1080, forward only) with 2 % of the Gaussians."""
    from retinags_amd.harness import pipeline
    scene, cam, cfg, subs, rel = _frame_setup("C4", 50.0)
    assert len(subs) == 32 and not cfg["backward"]
    cam_d = cam.to(DEV)
    bg = torch.zeros(3, device=DEV)
    seen = [m for m in range(32) if rel[m] >= 0]
    assert len(seen) >= 4   # the camera's frustum meets 6 of the 32 boxes (exact test, as the reference's)
    for m in seen[:3]:
        _check_binning_structure(_forward_raw(subs[m], cam_d, cam, bg), subs[m].means3D.shape[0], cam.image_width,
                                 cam.image_height)
    with torch.no_grad():
        out = pipeline.render_frame(cam_d, subs, rel, bg)
    assert torch.isfinite(out["render"]).all() and float(out["alpha"].max()) <= 1 + 1e-5
    assert float(out["alpha"].mean()) > 0.01
