"""Every benchmark configuration at its full size.  Where the CPU checker finishes in seconds
(C0, C1, the heaviest submodel of C2) the HIP path is compared with it; everywhere it is held
to size-independent properties: structure of the binning output (sortedness, stability, range
partition, counts), bit-for-bit determinism, the compositing identity, and exact linearity of
the rendered loss in the SH DC coefficients (a finite-difference check of dL/dSH that needs no
oracle).  The scenes of C3 (62.9 M Gaussians) and C4 (217.3 M) are generated and partitioned
on the device.  Config names are those of retinags_amd.harness.scenes.CONFIGS.

Every configuration is rendered both ways the library offers: one call per submodel
(rgs_forward_geom / rgs_forward_raster / rgs_backward, the reference's call pattern) and all
submodels of the frame through rgs_frame_forward_geom / _raster / rgs_frame_backward (one launch
per stage for the whole frame, which is what bench.py times).  The two must agree bit for bit in
everything but the atomically summed gradients, and the comparisons with the CPU checker are
taken from the frame path's outputs."""
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
    keys = ((view_ws(binning, b["keys_sorted"], Rn, np.uint32) & np.uint32(0xFFFFFF)).astype(np.uint64) << np.uint64(32)) | \
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


def _frame_setup_on_device(name):
    """The full-size scene generated, partitioned and split into submodels on the GPU."""
    from retinags_amd.harness import partition, pipeline
    scene, cam, cfg = scenes.make_config(name, DEV)
    part = partition.partition_scene_on_device(scene["xyz"], scene["scales"], cfg["bvh_depth"])
    rel = partition.relation_vector(part, cam)
    subs = pipeline.submodels_from_partition(scene, part, DEV)
    owned = [int((part.owner == k).sum()) for k in range(len(subs))]
    assert sum(owned) == cfg["n"]
    del scene
    torch.cuda.empty_cache()
    return cam, cfg, subs, rel, part


# Relative L2 between the two paths' gradients: the same terms added atomically in another order (a frame rendered twice
# the same way differs from itself as much: a few 1e-5 at most where a Gaussian's sum has thousands of terms of both signs)
FRAME_GRAD_TOL = 1e-4


def _frame_against_calls_per_submodel(cam, subs, rel, bg, with_backward, seed, grads_on_layers=False):
    """Renders the frame through rasterize_frame (pipeline.render_frame(together=True)) and again with one call per
    submodel, and holds the former to the latter: instance counts, radii, the sorted lists, tile ranges, n_contrib and
    the images bit for bit; with_backward every gradient to FRAME_GRAD_TOL.  The upstream gradient is put on the
    composited image, or (grads_on_layers) directly on every layer's image.  Returns the frame path's output (with
    its workspaces) and, with_backward, {submodel: {field: gradient}} of the frame path, and the upstream gradient."""
    from retinags_amd import _capi
    from retinags_amd.harness import pipeline
    cam_d = cam.to(DEV)
    H, W = cam.image_height, cam.image_width
    related = [m for m in range(len(subs)) if rel[m] >= 0]
    g = (torch.randn(3, H, W, generator=torch.Generator().manual_seed(seed)) * 1e-2).to(DEV)
    fields = ("means3D", "opacity", "scales", "rotations", "shs")

    def take_grads():
        out = {}
        for m in related:
            out[m] = {f: getattr(subs[m], f).grad for f in fields}
            out[m]["means2D"] = subs[m].means2D.grad
            for t in subs[m].parameters():
                t.grad = None
            subs[m].means2D = None
        return out

    def prepare():
        for m in related:
            subs[m].requires_grad_(with_backward)
            subs[m].means2D = torch.zeros_like(subs[m].means3D, requires_grad=True) if with_backward else None

    def send_back(out):
        if grads_on_layers:
            torch.autograd.backward([out["partial"][m]["render"] for m in related], [g for _ in related])
        else:
            torch.autograd.backward([out["render"]], [g])

    prepare()
    frame = pipeline.render_frame(cam_d, subs, rel, bg, together=True, keep_workspaces=True)
    frame_grads = None
    if with_backward:
        send_back(frame)
        frame_grads = take_grads()
    prepare()
    zero = torch.zeros(3, device=DEV)
    im = _capi.image_layout(W, H)
    T = ((W + 15) // 16) * ((H + 15) // 16)
    piece = lambda buf, off, nbytes: buf[off:off + nbytes]
    for m in related:
        Rn, geom, binning, img = frame["workspaces"][m]
        raw = _forward_raw(subs[m], cam_d, cam, zero)
        assert raw[0] == Rn, m
        layer = frame["partial"][m]
        assert torch.equal(raw[4], layer["radii"]), m
        for k, key in ((1, "render"), (2, "depth"), (3, "alpha")):
            assert torch.equal(raw[k], layer[key].detach()), (m, key)          # the images, bit for bit
        assert torch.equal(piece(raw[7], im["n_contrib"], 4 * W * H), piece(img, im["n_contrib"], 4 * W * H)), m
        assert torch.equal(piece(raw[7], im["ranges"], 8 * T), piece(img, im["ranges"], 8 * T)), m
        if Rn:
            b = _capi.binning_layout(Rn, W, H)
            for name in ("keys_sorted", "values_sorted"):
                assert torch.equal(piece(raw[6], b[name], 4 * Rn), piece(binning, b[name], 4 * Rn)), (m, name)
        del raw
    if with_backward:
        again = pipeline.render_frame(cam_d, subs, rel, bg)   # one call per submodel
        assert torch.equal(again["render"], frame["render"]) and torch.equal(again["alpha"], frame["alpha"])
        send_back(again)
        call_grads = take_grads()
        from helpers import rel_l2
        for m in related:
            for f, want in call_grads[m].items():
                got = frame_grads[m][f]
                assert (got is None) == (want is None), (m, f)
                if want is not None:
                    assert rel_l2(got.cpu().numpy(), want.cpu().numpy()) <= FRAME_GRAD_TOL, (m, f)
        del again, call_grads
    for m in related:
        subs[m].requires_grad_(False)
        subs[m].means2D = None
    return frame, frame_grads, g


def _frame_layer_against_checker(frame, frame_grads, m, sub, cam, low, up, g_layer):
    """Submodel m of a frame rendered through rasterize_frame against the CPU checker (OpenMP): instance count,
    radii, binning bit for bit, images, and (with frame_grads: gradients taken with g_layer on this layer's image)
    every gradient."""
    import os
    from helpers import DECISION_MARGIN, GRAD_TOL, IMAGE_TOL, np32, orc, rel_l2
    H, W = cam.image_height, cam.image_width
    xyz, opa, sc, rot, shs = (np32(t) for t in (sub.means3D, sub.opacity, sub.scales, sub.rotations, sub.shs))
    orc.set_threads(min(16, orc.max_threads(), os.cpu_count() or 1))
    try:
        s = orc.settings_from_camera(cam, low, up, torch.zeros(3))
        st = orc.forward(s, xyz, opa, shs=shs, scales=sc, rotations=rot, want_margin=True)
        want = orc.backward(s, st, np32(g_layer)) if frame_grads is not None else None
    finally:
        orc.set_threads(1)
    Rn, geom, binning, img = frame["workspaces"][m]
    assert Rn == st.R
    check_binning_against(st, geom, binning, st.P, st.R, W, H)
    layer = frame["partial"][m]
    assert np.array_equal(layer["radii"].cpu().numpy(), st.radii)
    safe = (st.margin > DECISION_MARGIN).reshape(H, W)
    assert (~safe).mean() < 1e-3
    for key, want_plane in (("render", st.color), ("alpha", st.alpha), ("depth", st.depth)):
        tol = IMAGE_TOL * (max(1.0, float(np.abs(want_plane).max())) if key == "depth" else 1.0)
        assert np.abs(layer[key].detach().cpu().numpy() - want_plane)[:, safe].max() <= tol, key
    if frame_grads is not None:
        for key, f in (("means3D", "means3D"), ("means2D", "means2D"), ("sh", "shs"), ("opacity", "opacity"), ("scales", "scales"),
                       ("rotations", "rotations")):
            assert rel_l2(frame_grads[m][f].cpu().numpy(), want[key]) <= GRAD_TOL, (m, key)
    return st


def _check_compositing_identity(out, rel, bg):
    """image = sum_k T_k image_k + bg T_K, alpha = 1 - T_K, with T_k the product of (1 - alpha_j) over
    the layers in front (parallel_utils/basic_parallel_trainer/result_aggregator.py:244-259)."""
    a = out["alpha"]
    assert torch.isfinite(out["render"]).all() and float(a.min()) >= 0 and float(a.max()) <= 1 + 1e-5
    layers = [out["partial"][m] for m in sorted((m for m in range(len(rel)) if rel[m] >= 0), key=lambda m: rel[m])]
    T = torch.ones_like(a)
    acc = torch.zeros_like(out["render"])
    for layer in layers:
        acc += T * layer["render"]
        T = T * (1 - layer["alpha"])
    assert torch.allclose(out["render"], acc + bg.view(3, 1, 1) * T, atol=1e-5)
    assert torch.allclose(a, 1 - T, atol=1e-6)


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
    rgb = torch.from_numpy(view_ws(raw[5], _capi.geom_layout(P)["blend_record"], 16 * P, np.float32).reshape(P, 16)[:, 8:11].copy()).to(DEV)
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
    # few significant bits, so every term of the prediction holds to a fraction of a percent, not to
    # rounding (the CPU checker shows the same deviation).  The terms have both signs, so the bound
    # is taken against their absolute sum, not against the net change.
    mass = (grad.double() * v.double()).abs().sum()
    assert abs(float(measured)) > 1e-6
    assert abs(float(measured - predicted)) <= 5e-3 * float(mass) + 1e-7
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
    """Config C1 at full size against the CPU checker (OpenMP makes it fast enough), rendered the way bench.py times
    it: all four submodels through rasterize_frame (rgs_frame_forward_geom / _raster / rgs_frame_backward).  Every
    submodel's binning bit for bit, its images and every gradient, the screen-space gradient included, with the
    upstream gradients that the compositor's backward hands each layer; then the composited frame.  The same frame
    with one call per submodel must give the same bits (gradients: the same sums in another order)."""
    from helpers import DECISION_MARGIN, GRAD_TOL, IMAGE_TOL, np32, orc, rel_l2
    from retinags_amd.harness import partition, pipeline
    from retinags_amd import _capi
    import os
    scene, cam, cfg = scenes.make_config("C1", "cpu", 1.0)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    rel = partition.relation_vector(part, cam)
    assert (rel >= 0).all()
    subs = pipeline.submodels_from_partition(scene, part, DEV)
    H, W = cam.image_height, cam.image_width
    bg = torch.tensor([0.1, 0.3, 0.2])
    frame, grads, g = _frame_against_calls_per_submodel(cam, subs, rel, bg.to(DEV), with_backward=True, seed=11)
    g = g.cpu()
    xyz, opa, sc, rot, shs = (np32(scene[k]) for k in ("xyz", "opacity", "scales", "rotations", "shs"))
    orc.set_threads(min(16, orc.max_threads(), os.cpu_count() or 1))
    try:
        order = sorted(range(4), key=lambda m: rel[m])
        states, sets = {}, {}
        for m in order:
            ids = part.members[m]
            sets[m] = orc.settings_from_camera(cam, part.box_low[m], part.box_up[m], torch.zeros(3))
            states[m] = orc.forward(sets[m], xyz[ids], opa[ids], shs=shs[ids], scales=sc[ids], rotations=rot[ids],
                                    want_margin=True)
        for m in order:   # binning of the frame path, bit for bit
            st = states[m]
            Rn, geom, binning, img = frame["workspaces"][m]
            assert Rn == st.R
            check_binning_against(st, geom, binning, st.P, st.R, W, H)
            assert np.array_equal(view_ws(img, _capi.image_layout(W, H)["ranges"], 2 * len(st.ranges), np.uint32),
                                  st.ranges.ravel())
        out = frame
        imgs, deps, alps = ([states[m].color for m in order], [states[m].depth for m in order],
                            [states[m].alpha for m in order])
        want_img, want_dep, want_alpha = orc.composite_forward(imgs, deps, alps, np32(bg))
        d_img, d_dep, d_alp = orc.composite_backward(imgs, deps, alps, np32(bg), np32(g))
        safe_all = np.ones((H, W), dtype=bool)
        for k, m in enumerate(order):
            st, layer = states[m], out["partial"][m]
            want = orc.backward(sets[m], st, d_img[k], d_dep[k], d_alp[k])
            assert np.array_equal(layer["radii"].cpu().numpy(), st.radii)
            safe = (st.margin > DECISION_MARGIN).reshape(H, W)
            assert (~safe).mean() < 1e-3
            safe_all &= safe
            assert np.abs(layer["render"].detach().cpu().numpy() - st.color)[:, safe].max() <= IMAGE_TOL
            assert np.abs(layer["alpha"].detach().cpu().numpy() - st.alpha)[:, safe].max() <= IMAGE_TOL
            assert np.abs(layer["depth"].detach().cpu().numpy() - st.depth)[:, safe].max() <= IMAGE_TOL
            for key, f in (("means3D", "means3D"), ("means2D", "means2D"), ("sh", "shs"), ("opacity", "opacity"),
                           ("scales", "scales"), ("rotations", "rotations")):
                assert rel_l2(grads[m][f].cpu().numpy(), want[key]) <= GRAD_TOL, (m, key)
        assert np.abs(out["render"].detach().cpu().numpy() - want_img)[:, safe_all].max() <= IMAGE_TOL
        assert np.abs(out["alpha"].detach().cpu().numpy() - want_alpha)[:, safe_all].max() <= IMAGE_TOL
        assert np.abs(out["depth"].detach().cpu().numpy() - want_dep)[:, safe_all].max() <= IMAGE_TOL
    finally:
        orc.set_threads(1)


def test_high_resolution_full_size():
    """Config C2 at full size: the 5.6 M Gaussians of C1 at 5185x3359 (68 250 tiles: 17-bit tile keys, sorted in two
    passes of 9 and 8 bits where C1's 13 bits take 7 and 6), about 71 M instances.  Structure and determinism of every submodel, the compositing identity, SH linearity, the frame through
    rasterize_frame against one call per submodel, and the submodel with the most instances against the CPU checker."""
    from helpers import DECISION_MARGIN, GRAD_TOL, IMAGE_TOL, np32, orc, rel_l2
    from retinags_amd.harness import partition, pipeline
    from retinags_amd import _capi
    import os
    scene, cam, cfg = scenes.make_config("C2", "cpu", 1.0)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    rel = partition.relation_vector(part, cam)
    subs = pipeline.submodels_from_partition(scene, part, DEV)
    H, W = cam.image_height, cam.image_width
    assert (W, H) == (5185, 3359) and _capi.lib.rgs_get_higher_msb(((W + 15) // 16) * ((H + 15) // 16)) == 17
    cam_d = cam.to(DEV)
    bg = torch.zeros(3, device=DEV)
    counts = {}
    for m, sub in enumerate(subs):
        if rel[m] < 0:
            continue
        outs = _forward_raw(sub, cam_d, cam, bg)
        _check_binning_structure(outs, sub.means3D.shape[0], W, H)
        again = _forward_raw(sub, cam_d, cam, bg)
        assert outs[0] == again[0] and all(torch.equal(outs[k], again[k]) for k in (1, 2, 3, 4))
        counts[m] = outs[0]
        del outs, again
    assert sum(counts.values()) > 50_000_000
    with torch.no_grad():
        _check_compositing_identity(pipeline.render_frame(cam_d, subs, rel, torch.tensor([0.1, 0.2, 0.3], device=DEV)),
                                    rel, torch.tensor([0.1, 0.2, 0.3], device=DEV))
    _sh_linearity(cam, subs, rel, which=None, seed=4)

    # the whole frame through rasterize_frame against one call per submodel, forward and backward; then the submodel
    # with the most instances, as the frame path rendered it, against the CPU checker
    bg = torch.zeros(3, device=DEV)
    frame, grads, g = _frame_against_calls_per_submodel(cam, subs, rel, bg, with_backward=True, seed=12, grads_on_layers=True)
    m = max(counts, key=counts.get)
    _frame_layer_against_checker(frame, grads, m, subs[m], cam, part.box_low[m], part.box_up[m], g)


def test_dense_scene_full_size_sixteen_submodels():
    """Config C3 at full size: 62.9 M Gaussians with scales shrunk by sqrt(11), bvh_depth 4, every submodel that
    the camera sees rendered and composited, forward and backward."""
    from retinags_amd.harness import pipeline
    cam, cfg, subs, rel, part = _frame_setup_on_device("C3")
    assert len(subs) == 16 and cfg["n"] == 62_900_000
    cam_d = cam.to(DEV)
    seen = [m for m in range(16) if rel[m] >= 0]
    assert len(seen) >= 8
    counts = {}
    for m in seen:
        outs = _forward_raw(subs[m], cam_d, cam, torch.zeros(3, device=DEV))
        _check_binning_structure(outs, subs[m].means3D.shape[0], cam.image_width, cam.image_height)
        again = _forward_raw(subs[m], cam_d, cam, torch.zeros(3, device=DEV))
        assert outs[0] == again[0] and all(torch.equal(outs[k], again[k]) for k in (1, 2, 3, 4))
        counts[m] = outs[0]
        del outs, again
    assert sum(counts.values()) > 20_000_000
    # the whole frame (every submodel the camera sees, one launch per stage) against one call per submodel, forward
    # and backward; then the two submodels with the most instances, as the frame path rendered them, against the
    # CPU checker, forward and backward
    frame, grads, g = _frame_against_calls_per_submodel(cam, subs, rel, torch.zeros(3, device=DEV), with_backward=True, seed=40,
                                                        grads_on_layers=True)
    for m in sorted(counts, key=counts.get)[-2:]:
        _frame_layer_against_checker(frame, grads, m, subs[m], cam, part.box_low[m], part.box_up[m], g)
    del frame, grads
    torch.cuda.empty_cache()
    bg = torch.tensor([0.1, 0.2, 0.3], device=DEV)
    with torch.no_grad():
        _check_compositing_identity(pipeline.render_frame(cam_d, subs, rel, bg), rel, bg)
    _sh_linearity(cam, subs, rel, which=None, seed=5)


def test_city_full_size_forward_only_thirty_two_submodels():
    """Config C4 at full size: 217.3 M Gaussians, bvh_depth 5, 1920x1080, forward only."""
    from retinags_amd.harness import pipeline
    cam, cfg, subs, rel, part = _frame_setup_on_device("C4")
    assert len(subs) == 32 and cfg["n"] == 217_300_000 and not cfg["backward"]
    cam_d = cam.to(DEV)
    bg = torch.zeros(3, device=DEV)
    seen = [m for m in range(32) if rel[m] >= 0]
    assert len(seen) >= 4   # the camera's frustum meets few of the 32 boxes (exact test, as the reference's)
    counts = {}
    for m in seen:
        outs = _forward_raw(subs[m], cam_d, cam, bg)
        _check_binning_structure(outs, subs[m].means3D.shape[0], cam.image_width, cam.image_height)
        again = _forward_raw(subs[m], cam_d, cam, bg)
        assert outs[0] == again[0] and all(torch.equal(outs[k], again[k]) for k in (1, 2, 3, 4))
        counts[m] = outs[0]
        del outs, again
    # the frame through rasterize_frame against one call per submodel, then the submodel with the most instances,
    # as the frame path rendered it, against the CPU checker
    with torch.no_grad():
        frame, _, _ = _frame_against_calls_per_submodel(cam, subs, rel, bg, with_backward=False, seed=50)
    m = max(counts, key=counts.get)
    _frame_layer_against_checker(frame, None, m, subs[m], cam, part.box_low[m], part.box_up[m], None)
    del frame
    torch.cuda.empty_cache()
    with torch.no_grad():
        out = pipeline.render_frame(cam_d, subs, rel, torch.tensor([0.3, 0.2, 0.1], device=DEV))
    _check_compositing_identity(out, rel, torch.tensor([0.3, 0.2, 0.1], device=DEV))
    assert float(out["alpha"].mean()) > 0.01


def test_partition_on_device_matches_the_host_partition():
    """The tensor-operation partition used for the large scenes against the numpy one, on the GPU."""
    from retinags_amd.harness import partition
    for name, shrink in (("C1", 20.0), ("C3", 100.0), ("C4", 200.0)):
        scene, cam, cfg = scenes.make_config(name, "cpu", shrink, geometry_only=True)
        host = partition.partition_scene(scene["xyz"], scene["scales"], cfg["bvh_depth"])
        dev = partition.partition_scene_on_device(scene["xyz"].to(DEV), scene["scales"].to(DEV), cfg["bvh_depth"],
                                                  rows_per_pass=100_000)
        assert np.array_equal(host.grid.load, dev.grid.load)
        assert np.array_equal(host.box_low, dev.box_low) and np.array_equal(host.box_up, dev.box_up)
        assert np.array_equal(host.owner, dev.owner.cpu().numpy())
        assert all(np.array_equal(a, b.cpu().numpy()) for a, b in zip(host.members, dev.members))


@pytest.mark.parametrize("name", ["C1", "C3", "C4"])
def test_which_submodels_a_camera_sees_at_full_size(name):
    """The order vector and the box-against-frustum test of the harness (what decides how many submodels a
    frame of C3 / C4 renders) against the checker's restatement of the reference's hull test, on the
    partitions of the full-size scenes, for the benchmark camera and a ring of cameras around the scene."""
    from oracle import sharing_oracle as so
    from retinags_amd.harness import partition
    scene, cam0, cfg = scenes.make_config(name, DEV, geometry_only=True)
    part = partition.partition_scene_on_device(scene["xyz"], scene["scales"], cfg["bvh_depth"])
    del scene
    torch.cuda.empty_cache()
    K = 2 ** cfg["bvh_depth"]
    assert len(part.leaves) == K
    paths = [leaf.path for leaf in part.leaves]
    splits = {}
    for path, node in part.nodes.items():
        if not node.is_leaf and node.split_position is not None:
            d = node.split_dim
            splits[path] = (d, node.split_position * part.grid.voxel[d] + part.grid.low[d])
    centre = 0.5 * (part.grid.low + part.grid.up).astype(np.float64)
    radius = 0.35 * float(np.linalg.norm((part.grid.up - part.grid.low)[:2]))
    cams = [cam0]
    for k in range(12):
        phi = 2 * np.pi * k / 12
        eye = centre + np.array([radius * np.cos(phi), radius * np.sin(phi), 0.3 * radius * (1 + k % 3)])
        cams.append(scenes.look_at_camera(eye, centre, (0, 0, 1), cam0.image_width, cam0.image_height, 40.0 + 5 * k))
    unseen = 0
    for cam in cams:
        wvt = cam.world_view_transform.numpy()
        overlaps = [so.is_overlapping_spacebox_view(part.box_low[m], part.box_up[m], wvt, cam.FoVx, cam.FoVy, 0.01, 1000.0)
                    for m in range(K)]
        want = so.relation_vector(cam.camera_center.numpy(), paths, splits, overlaps)
        got = partition.relation_vector(part, cam, 0.01, 1000.0)
        assert np.array_equal(want, got), (name, cam.camera_center)
        assert np.array_equal(partition.boxes_overlap_view(part.box_low, part.box_up, cam, 0.01, 1000.0), np.array(overlaps))
        unseen += int((want < 0).sum())
    if K > 4:
        assert unseen > 0
