"""The public API of the HIP rasterizer on the GPU: golden vectors, input modes of the
reference interface (precomputed colours / covariance, empty input, markVisible, debug),
and a whole partitioned frame (4 submodels rendered in turn, composited, differentiated)
against the CPU checker."""
import os

import numpy as np
import pytest
import torch

from helpers import (DECISION_MARGIN, GRAD_TOL, IMAGE_TOL, ROOT, np32, oracle_settings, orc, rel_l2, scenes)
from test_golden_cpu import load_cases, settings_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _settings(c_or_s, debug=False):
    from retinags_amd import GaussianRasterizationSettings
    s = c_or_s
    t = lambda a: torch.from_numpy(np.asarray(a, np.float32)).to(DEV)
    return GaussianRasterizationSettings(
        image_height=s.image_height, image_width=s.image_width, tanfovx=s.tanfovx, tanfovy=s.tanfovy, bg=t(s.bg),
        scale_modifier=s.scale_modifier, viewmatrix=t(s.viewmatrix).view(4, 4), projmatrix=t(s.projmatrix).view(4, 4),
        projmatrix_inv=t(s.projmatrix_inv).view(4, 4), range_low=t(s.range_low), range_up=t(s.range_up),
        sh_degree=s.sh_degree, campos=t(s.campos), prefiltered=False, debug=debug)


def test_golden_vectors_forward_and_backward():
    from retinags_amd import GaussianRasterizer
    for name, c in load_cases().items():
        s = settings_of(c)
        t = lambda k: torch.from_numpy(c[k]).to(DEV).requires_grad_(True)
        xyz, opa, sc, rot, shs = t("xyz"), t("opacity"), t("scales"), t("rotations"), t("shs")
        m2d = torch.zeros_like(xyz, requires_grad=True)
        color, radii, depth, alpha = GaussianRasterizer(_settings(s))(
            means3D=xyz, means2D=m2d, opacities=opa, shs=shs, scales=sc, rotations=rot)
        assert np.array_equal(radii.cpu().numpy(), c["radii"]), name
        H, W = s.image_height, s.image_width
        safe = (c["margin"] > DECISION_MARGIN).reshape(H, W)
        for got, key in ((color, "color"), (depth, "depth"), (alpha, "alpha")):
            assert np.abs(got.detach().cpu().numpy() - c[key])[:, safe].max() <= IMAGE_TOL, (name, key)
        d = lambda k: torch.from_numpy(c[k]).to(DEV)
        torch.autograd.backward([color, depth, alpha], [d("g_color"), d("g_depth"), d("g_alpha")])
        for got, key in ((xyz.grad, "means3D"), (m2d.grad, "means2D"), (opa.grad, "opacity"), (sc.grad, "scales"),
                         (rot.grad, "rotations"), (shs.grad, "sh")):
            assert rel_l2(got.cpu().numpy(), c["grad_" + key]) <= GRAD_TOL, (name, key)


def _small_inputs(n=3000, seed=3):
    scene, cam, _ = scenes.make_config("C0", shrink=100_000 / n, resolution_scale=0.25)
    pad = 3.0 * float(scene["scales"].max()) + 1.0
    low, up = scene["xyz"].min(0).values - pad, scene["xyz"].max(0).values + pad
    return scene, cam, low, up


def test_precomputed_colours_and_covariance_modes():
    """colors_precomp / cov3D_precomp inputs (K/.../__init__.py:209-218) give the same image as
    SHs / scale+rotation when fed the values the preprocess would compute, and their
    gradients match the checker's."""
    from retinags_amd import GaussianRasterizer
    scene, cam, low, up = _small_inputs()
    bg = torch.tensor([0.2, 0.1, 0.4])
    s = oracle_settings(cam, low, up, bg)
    st = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]),
                     scales=np32(scene["scales"]), rotations=np32(scene["rotations"]))
    rgb, cov = st.rgb.copy(), st.cov3D.copy()
    st2 = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), colors_precomp=rgb, cov3D_precomp=cov, want_margin=True)
    assert np.array_equal(st2.color, st.color)
    H, W = cam.image_height, cam.image_width
    g_color = np32(torch.randn(3, H, W, generator=torch.Generator().manual_seed(1)) * 1e-2)
    want = orc.backward(s, st2, g_color)
    xyz = scene["xyz"].to(DEV).requires_grad_(True)
    opa = scene["opacity"].to(DEV).requires_grad_(True)
    col = torch.from_numpy(rgb).to(DEV).requires_grad_(True)
    c3d = torch.from_numpy(cov).to(DEV).requires_grad_(True)
    color, radii, depth, alpha = GaussianRasterizer(_settings(s))(
        means3D=xyz, means2D=torch.zeros_like(xyz), opacities=opa, colors_precomp=col, cov3D_precomp=c3d)
    assert np.array_equal(radii.cpu().numpy(), st.radii)
    # the parity rule of the other image tests: 1e-4 away from the blend's decision thresholds, and few pixels near them
    safe = (st2.margin > DECISION_MARGIN).reshape(H, W)
    assert (~safe).mean() <= 1e-3
    for got_plane, want_plane in ((color, st.color), (depth, st.depth), (alpha, st.alpha)):
        diff = np.abs(got_plane.detach().cpu().numpy() - want_plane)
        assert diff[:, safe].max() <= IMAGE_TOL and diff.max() <= 2e-2
    torch.autograd.backward([color], [torch.from_numpy(g_color).to(DEV)])
    assert rel_l2(col.grad.cpu().numpy(), want["colors"]) <= GRAD_TOL
    assert rel_l2(c3d.grad.cpu().numpy(), want["cov3D"]) <= GRAD_TOL
    assert rel_l2(xyz.grad.cpu().numpy(), want["means3D"]) <= GRAD_TOL
    assert rel_l2(opa.grad.cpu().numpy(), want["opacity"]) <= GRAD_TOL


def test_renderer_switches_for_tensor_expression_colours_and_covariances():
    """render4BoundedGaussianModel's branches (gaussian_renderer/render_half_gs.py:55-79) as pipeline.render_bounded_model
    restates them: SH colours and 3D covariances computed by tensor operations (convert_SHs_python,
    compute_cov3D_python) and override_color.  Every combination gives the checker's image by the rule of the other
    image tests (1e-4 away from decision thresholds), the same radii, and gradients that reach the SH coefficients,
    scales and rotations through autograd and equal the checker's in-kernel ones to GRAD_TOL."""
    from retinags_amd.harness import pipeline
    scene, cam, low, up = _small_inputs()
    bg = torch.tensor([0.2, 0.1, 0.4])
    s = oracle_settings(cam, low, up, bg)
    st = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]), scales=np32(scene["scales"]),
                     rotations=np32(scene["rotations"]), want_margin=True)
    H, W = cam.image_height, cam.image_width
    g_color = torch.randn(3, H, W, generator=torch.Generator().manual_seed(2)) * 1e-2
    want = orc.backward(s, st, np32(g_color))
    safe = (st.margin > DECISION_MARGIN).reshape(H, W)
    cam_d = cam.to(DEV)

    def submodel():
        t = lambda k: scene[k].to(DEV).clone().requires_grad_(True)
        return pipeline.Submodel(t("xyz"), t("opacity"), t("scales"), t("rotations"), t("shs"), low.to(DEV), up.to(DEV))

    for sh_python in (False, True):
        for cov_python in (False, True):
            sub = submodel()
            out = pipeline.render_bounded_model(cam_d, sub, pipeline.PipelineSwitches(sh_python, cov_python), bg.to(DEV))
            assert set(out) >= {"render", "viewspace_points", "radii", "depth", "alpha", "num_rendered"} and out["num_rendered"] == -1
            assert np.array_equal(out["radii"].cpu().numpy(), st.radii)
            assert torch.equal(out["visibility_filter"], out["radii"] > 0)
            for key, plane in (("render", st.color), ("depth", st.depth), ("alpha", st.alpha)):
                assert np.abs(out[key].detach().cpu().numpy() - plane)[:, safe].max() <= IMAGE_TOL, (sh_python, cov_python, key)
            torch.autograd.backward([out["render"]], [g_color.to(DEV)])
            for key, t in (("means3D", sub.means3D), ("opacity", sub.opacity), ("sh", sub.shs), ("scales", sub.scales),
                           ("rotations", sub.rotations)):
                expect = want[key]
                if cov_python and key == "rotations":
                    # the tensor expression normalises the quaternion first (utils/general_utils.py:79-82), the kernel uses
                    # it as given (K/cuda_rasterizer_hgs/backward.cu:340): for the unit quaternions of this scene the
                    # former's gradient is the latter's without its component along the quaternion
                    q = np32(scene["rotations"]).astype(np.float64)
                    expect = expect - q * (q * expect).sum(axis=1, keepdims=True)
                assert rel_l2(t.grad.cpu().numpy(), expect) <= GRAD_TOL, (sh_python, cov_python, key)
    # override_color: the rasterizer gets the caller's colours, the SH coefficients take no part
    sub = submodel()
    colours = torch.from_numpy(st.rgb.copy()).to(DEV).requires_grad_(True)
    out = pipeline.render_bounded_model(cam_d, sub, pipeline.PipelineSwitches(), bg.to(DEV), override_color=colours)
    assert np.abs(out["render"].detach().cpu().numpy() - st.color)[:, safe].max() <= IMAGE_TOL
    torch.autograd.backward([out["render"]], [g_color.to(DEV)])
    assert sub.shs.grad is None
    st_c = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), colors_precomp=st.rgb.copy(), scales=np32(scene["scales"]),
                       rotations=np32(scene["rotations"]))
    assert rel_l2(colours.grad.cpu().numpy(), orc.backward(s, st_c, np32(g_color))["colors"]) <= GRAD_TOL


def test_gaussians_stored_in_morton_order_render_the_same_frame():
    """pipeline.submodels_from_partition(order="morton") only changes the order of a submodel's rows: the per-tile
    lists hold the same Gaussians in the same depth order, so every image of the frame is the same bit for bit (the
    scene has no two Gaussians at the same depth), the radii are those of the given order, permuted, and the gradients
    agree up to the order of the atomic additions."""
    from retinags_amd.harness import partition, pipeline
    scene, cam, cfg = scenes.make_config("C1", "cpu", 300.0, 0.25)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    rel = partition.relation_vector(part, cam)
    cam_d = cam.to(DEV)
    bg = torch.tensor([0.2, 0.3, 0.1], device=DEV)
    g = (torch.randn(3, cam.image_height, cam.image_width, generator=torch.Generator().manual_seed(8)) * 1e-2).to(DEV)
    frames, grads, subs_of = {}, {}, {}
    for order in ("given", "morton"):
        subs = [s_.requires_grad_(True) for s_ in pipeline.submodels_from_partition(scene, part, DEV, order=order)]
        out = pipeline.render_frame(cam_d, subs, rel, bg, together=True)
        torch.autograd.backward([out["render"]], [g])
        frames[order], subs_of[order] = out, subs
    for key in ("render", "depth", "alpha"):
        assert torch.equal(frames["given"][key], frames["morton"][key]), key
    for m in range(len(part.members)):
        ids = torch.from_numpy(np.asarray(part.members[m]))
        perm = partition.morton_order(scene["xyz"][ids])
        a, b = subs_of["given"][m], subs_of["morton"][m]
        assert torch.equal(a.means3D.detach()[perm.to(DEV)], b.means3D.detach())
        if rel[m] >= 0:
            assert torch.equal(frames["given"]["partial"][m]["radii"][perm.to(DEV)], frames["morton"]["partial"][m]["radii"])
            for f in ("means3D", "opacity", "scales", "rotations", "shs"):
                want, got = getattr(a, f).grad[perm.to(DEV)], getattr(b, f).grad
                assert rel_l2(got.cpu().numpy(), want.cpu().numpy()) <= 1e-4, (m, f)


def test_frame_layers_with_different_input_modes():
    """rasterize_frame with one layer given SHs and scale/rotation and one given precomputed colours and 3D
    covariances: each layer's images and gradients are those of a call of its own."""
    from retinags_amd import GaussianRasterizer
    from retinags_amd.rasterizer import rasterize_frame
    scene, cam, low, up = _small_inputs()
    s = oracle_settings(cam, low, up, torch.tensor([0.2, 0.1, 0.4]))
    st = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]),
                     scales=np32(scene["scales"]), rotations=np32(scene["rotations"]))
    rz = GaussianRasterizer(_settings(s))
    H, W = cam.image_height, cam.image_width
    g = (torch.randn(2, 3, H, W, generator=torch.Generator().manual_seed(4)) * 1e-2).to(DEV)

    def inputs():
        leaf = lambda t: t.to(DEV).clone().requires_grad_(True)
        a = dict(means3D=leaf(scene["xyz"]), means2D=torch.zeros(scene["xyz"].shape[0], 3, device=DEV),
                 opacities=leaf(scene["opacity"]), shs=leaf(scene["shs"]), scales=leaf(scene["scales"]),
                 rotations=leaf(scene["rotations"]))
        b = dict(means3D=leaf(scene["xyz"]), means2D=torch.zeros(scene["xyz"].shape[0], 3, device=DEV),
                 opacities=leaf(scene["opacity"]), colors_precomp=leaf(torch.from_numpy(st.rgb.copy())),
                 cov3D_precomp=leaf(torch.from_numpy(st.cov3D.copy())))
        return a, b

    a, b = inputs()
    outs = rasterize_frame([rz, rz], [a, b])
    torch.autograd.backward([outs[0][0], outs[1][0]], [g[0], g[1]])
    a1, b1 = inputs()
    alone = [rz(**a1), rz(**b1)]
    torch.autograd.backward([alone[0][0], alone[1][0]], [g[0], g[1]])
    for got, want in zip(outs, alone):
        for x, y in zip(got, want):
            assert torch.equal(x, y)
    for together, apart in ((a, a1), (b, b1)):
        for name in together:
            if together[name].requires_grad:
                assert rel_l2(together[name].grad.cpu().numpy(), apart[name].grad.cpu().numpy()) <= 1e-5, name


def test_empty_input_and_nothing_visible():
    from retinags_amd import GaussianRasterizer
    scene, cam, low, up = _small_inputs(64)
    s = oracle_settings(cam, low, up, torch.tensor([0.3, 0.6, 0.9]))
    r = GaussianRasterizer(_settings(s))
    z = lambda *shape: torch.zeros(*shape, device=DEV)
    color, radii, depth, alpha = r(means3D=z(0, 3), means2D=z(0, 3), opacities=z(0, 1), shs=z(0, 16, 3),
                                   scales=z(0, 3), rotations=z(0, 4))
    assert radii.numel() == 0 and float(color.abs().sum()) == 0.0 and float(alpha.abs().sum()) == 0.0
    # every Gaussian behind the camera: no instance is generated, the image is the background
    xyz = scene["xyz"].clone()
    xyz[:, 2] = -xyz[:, 2]
    xyz = xyz.to(DEV).requires_grad_(True)
    color, radii, depth, alpha = r(means3D=xyz, means2D=torch.zeros_like(xyz), opacities=scene["opacity"].to(DEV),
                                   shs=scene["shs"].to(DEV), scales=scene["scales"].to(DEV),
                                   rotations=scene["rotations"].to(DEV))
    assert int(radii.abs().sum()) == 0 and float(alpha.detach().abs().sum()) == 0.0
    assert torch.allclose(color.detach(), torch.tensor([0.3, 0.6, 0.9], device=DEV).view(3, 1, 1).expand_as(color))
    color.sum().backward()
    assert float(xyz.grad.abs().sum()) == 0.0


def test_mark_visible_and_debug_mode():
    from retinags_amd import GaussianRasterizer
    scene, cam, low, up = _small_inputs(5000)
    scene["xyz"][::3, 2] -= 6.0
    s = oracle_settings(cam, low, up, torch.zeros(3))
    r = GaussianRasterizer(_settings(s, debug=True))
    vis = r.markVisible(scene["xyz"].to(DEV))
    assert vis.dtype == torch.bool
    assert np.array_equal(vis.cpu().numpy(), orc.mark_visible(s, np32(scene["xyz"])))
    st = orc.forward(s, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]),
                     scales=np32(scene["scales"]), rotations=np32(scene["rotations"]))
    xyz = scene["xyz"].to(DEV).requires_grad_(True)
    color, radii, _, _ = r(means3D=xyz, means2D=torch.zeros_like(xyz), opacities=scene["opacity"].to(DEV),
                           shs=scene["shs"].to(DEV), scales=scene["scales"].to(DEV), rotations=scene["rotations"].to(DEV))
    assert np.array_equal(radii.cpu().numpy(), st.radii)
    color.sum().backward()  # every stage synchronised and checked in debug mode
    assert torch.isfinite(xyz.grad).all()


def test_partitioned_frame_against_checker():
    """4 submodels with shared boundary Gaussians, rendered one after another, composited in
    BVH order, differentiated: images and every submodel's gradients vs the CPU checker."""
    from retinags_amd.harness import partition, pipeline
    scene, cam, _ = scenes.make_config("C1", shrink=150, resolution_scale=0.25)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    rel = partition.relation_vector(part, cam)
    subs = [s.requires_grad_(True) for s in pipeline.submodels_from_partition(scene, part, DEV)]
    H, W = cam.image_height, cam.image_width
    up = torch.randn(3, H, W, generator=torch.Generator().manual_seed(2)) * 1e-2
    bg = torch.tensor([0.5, 0.5, 0.5])
    out = pipeline.render_frame(cam.to(DEV), subs, rel, bg.to(DEV))
    torch.autograd.backward([out["render"]], [up.to(DEV)])
    torch.cuda.synchronize()

    order = sorted((m for m in range(4) if rel[m] >= 0), key=lambda m: rel[m])
    assert len(order) >= 2
    states, sets = [], []
    margin = np.full(H * W, np.inf, np.float32)
    for m in order:
        ids = part.members[m]
        s = oracle_settings(cam, torch.from_numpy(part.box_low[m]), torch.from_numpy(part.box_up[m]), torch.zeros(3))
        st = orc.forward(s, np32(scene["xyz"])[ids], np32(scene["opacity"])[ids], shs=np32(scene["shs"])[ids],
                         scales=np32(scene["scales"])[ids], rotations=np32(scene["rotations"])[ids], want_margin=True)
        margin = np.minimum(margin, st.margin)
        states.append(st)
        sets.append(s)
        got = out["partial"][m]
        assert np.array_equal(got["radii"].cpu().numpy(), st.radii)
    safe = (margin > DECISION_MARGIN).reshape(H, W)
    imgs, deps, alps = [st.color for st in states], [st.depth for st in states], [st.alpha for st in states]
    w_img, w_dep, w_alp = orc.composite_forward(imgs, deps, alps, np32(bg))
    assert np.abs(out["render"].detach().cpu().numpy() - w_img)[:, safe].max() <= IMAGE_TOL
    assert np.abs(out["alpha"].detach().cpu().numpy() - w_alp)[:, safe].max() <= IMAGE_TOL
    assert np.abs(out["depth"].detach().cpu().numpy() - w_dep)[:, safe].max() <= IMAGE_TOL * 10  # depths are O(10)
    d_img, d_dep, d_alp = orc.composite_backward(imgs, deps, alps, np32(bg), np32(up))
    for k, m in enumerate(order):
        g = orc.backward(sets[k], states[k], d_img[k], d_dep[k], d_alp[k])
        for key, t in (("means3D", subs[m].means3D), ("sh", subs[m].shs), ("opacity", subs[m].opacity),
                       ("scales", subs[m].scales), ("rotations", subs[m].rotations)):
            assert rel_l2(t.grad.cpu().numpy(), g[key]) <= GRAD_TOL, (m, key)
    # the partition is exact where it matters: compositing the clipped partial renders agrees
    # with one unclipped render of the whole scene up to the early-termination thresholds
    pad = 3.0 * float(scene["scales"].max()) + 1.0
    s_all = oracle_settings(cam, scene["xyz"].min(0).values - pad, scene["xyz"].max(0).values + pad, bg)
    whole = orc.forward(s_all, np32(scene["xyz"]), np32(scene["opacity"]), shs=np32(scene["shs"]),
                        scales=np32(scene["scales"]), rotations=np32(scene["rotations"]))
    assert np.abs(w_img - whole.color).mean() < 2e-3


def test_frame_on_several_streams_matches_one_stream():
    """Submodels rendered on separate HIP streams (forward and, through autograd, backward)
    give the images of the one-stream frame bit for bit and the same gradients up to the
    order of the atomic adds; repeated, to catch a missing dependency between streams."""
    from retinags_amd.harness import partition, pipeline
    scene, cam, _ = scenes.make_config("C1", shrink=40, resolution_scale=0.5)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    rel = partition.relation_vector(part, cam)
    subs = [s.requires_grad_(True) for s in pipeline.submodels_from_partition(scene, part, DEV)]
    H, W = cam.image_height, cam.image_width
    up = (torch.randn(3, H, W, generator=torch.Generator().manual_seed(5)) * 1e-2).to(DEV)
    bg = torch.tensor([0.2, 0.3, 0.4], device=DEV)
    cam_d = cam.to(DEV)

    def frame(streams):
        for s in subs:
            for p in s.parameters():
                p.grad = None
        out = pipeline.render_frame(cam_d, subs, rel, bg, streams=streams)
        torch.autograd.backward([out["render"]], [up])
        torch.cuda.synchronize()
        grads = [[p.grad.clone() for p in s.parameters()] for s in subs]
        return out["render"].detach().clone(), out["depth"].detach().clone(), out["alpha"].detach().clone(), grads

    ref = frame(None)
    for n_streams in (2, 4, 4):
        streams = [torch.cuda.Stream(device=DEV) for _ in range(n_streams)]
        if n_streams == 2:
            streams[0] = torch.cuda.current_stream(DEV)  # the caller's own stream may be one of them
        got = frame(streams)
        for a, b in zip(ref[:3], got[:3]):
            assert torch.equal(a, b)
        for ga, gb in zip(ref[3], got[3]):
            for a, b in zip(ga, gb):
                # float atomics commute only up to rounding; two one-stream runs differ as much
                assert rel_l2(b.cpu().numpy(), a.cpu().numpy()) <= 1e-4


def test_enqueued_geometry_stage_gives_the_same_forward_and_is_checked():
    """forward(..., geometry=stage) continues a stage started by enqueue_geometry: same outputs
    as the one-call forward, bit for bit; a stage cannot be used twice or for other inputs."""
    from retinags_amd import GaussianRasterizer
    scene, cam, low, up = _small_inputs(n=4000, seed=11)
    r = GaussianRasterizer(_settings(oracle_settings(cam, low, up, torch.tensor([0.1, 0.2, 0.3]))))
    kw = dict(means3D=scene["xyz"].to(DEV), opacities=scene["opacity"].to(DEV), shs=scene["shs"].to(DEV),
              scales=scene["scales"].to(DEV), rotations=scene["rotations"].to(DEV))
    m2d = torch.zeros_like(kw["means3D"])
    ref = r(means2D=m2d, **kw)
    stage = r.enqueue_geometry(**kw)
    got = r(means2D=m2d, geometry=stage, **kw)
    for a, b in zip(ref, got):
        assert torch.equal(a, b)
    with pytest.raises(RuntimeError):
        r(means2D=m2d, geometry=stage, **kw)  # already consumed
    stage2 = r.enqueue_geometry(**kw)
    other = dict(kw, means3D=kw["means3D"].clone())
    with pytest.raises(RuntimeError):
        r(means2D=m2d, geometry=stage2, **other)  # enqueued for another tensor
    got2 = r(means2D=m2d, geometry=stage2, **kw)  # the refused call did not consume it
    assert torch.equal(ref[0], got2[0])
    torch.cuda.synchronize()


def test_a_workspace_off_a_16_byte_boundary_is_refused():
    """The binning kernels move keys 16 bytes at a time: rgs_forward_raster refuses a workspace that does not
    start at a multiple of 16 bytes, before anything is launched, and accepts the same one when aligned."""
    import ctypes as C
    from retinags_amd import GaussianRasterizer, _capi
    from retinags_amd.rasterizer import ptr
    lib = _capi.lib
    scene, cam, low, up = _small_inputs(n=3000, seed=5)
    r = GaussianRasterizer(_settings(oracle_settings(cam, low, up, torch.zeros(3))))
    stage = r.enqueue_geometry(means3D=scene["xyz"].to(DEV), opacities=scene["opacity"].to(DEV), shs=scene["shs"].to(DEV),
                               scales=scene["scales"].to(DEV), rotations=scene["rotations"].to(DEV))
    R, t = stage.instances(), stage.tensors
    assert R > 0
    H, W = stage.H, stage.W
    byte = dict(dtype=torch.uint8, device=DEV)
    binning = torch.empty(lib.rgs_binning_bytes(R) + 16, **byte)
    image = torch.empty(lib.rgs_image_bytes(W, H), **byte)
    color, depth, alpha = (torch.empty(c, H, W, device=DEV) for c in (3, 1, 1))

    def raster(binning_at):
        return lib.rgs_forward_raster(
            stage.P, R, W, H, ptr(t["bg"]), t["tanfovx"], t["tanfovy"], ptr(t["projmatrix_inv"]), ptr(t["range_low"]),
            ptr(t["range_up"]), ptr(t["colors_precomp"]), ptr(stage.radii), ptr(stage.geomBuffer), stage.geom_bytes,
            C.c_void_p(binning.data_ptr() + binning_at), lib.rgs_binning_bytes(R), ptr(image), image.numel(), ptr(color),
            ptr(depth), ptr(alpha), C.c_void_p(stage.stream), 0)

    assert raster(4) != 0
    assert "16-byte aligned" in lib.rgs_last_error().decode()
    assert raster(0) == 0
    torch.cuda.synchronize()
    assert float(alpha.max()) > 0.0
    # the second half of the forward may run again on the same geometry state (its counters are left as it found them)
    first = (color.clone(), depth.clone(), alpha.clone())
    for out in (color, depth, alpha):
        out.fill_(-1.0)
    assert raster(0) == 0
    torch.cuda.synchronize()
    for a, b in zip(first, (color, depth, alpha)):
        assert torch.equal(a, b)


def test_forward_with_an_instance_bound_needs_no_count_and_reports_overflow():
    """enqueue_geometry(instance_bound=N) + forward: no wait for the instance count.  With room
    enough the outputs and gradients are those of the ordinary call, bit for bit (gradients up to
    the order of the atomic adds); with too little room the stage says so, nothing faults, and a
    repeat with the count it reports is right again."""
    from retinags_amd import GaussianRasterizer
    scene, cam, low, up = _small_inputs(n=6000, seed=21)
    r = GaussianRasterizer(_settings(oracle_settings(cam, low, up, torch.tensor([0.3, 0.2, 0.1]))))
    leaves = {k: scene[n].to(DEV).requires_grad_(True) for k, n in
              (("means3D", "xyz"), ("opacities", "opacity"), ("shs", "shs"), ("scales", "scales"), ("rotations", "rotations"))}
    weight = torch.randn(3, cam.image_height, cam.image_width, generator=torch.Generator().manual_seed(4)).to(DEV)

    def run(bound):
        for t in leaves.values():
            t.grad = None
        stage = r.enqueue_geometry(instance_bound=bound, **leaves) if bound != "wait" else r.enqueue_geometry(**leaves)
        out = r(means2D=torch.zeros_like(leaves["means3D"]), geometry=stage, **leaves)
        (out[0] * weight).sum().backward()
        torch.cuda.synchronize()
        return stage, [o.detach().clone() for o in out], [t.grad.clone() for t in leaves.values()]

    stage, ref_out, ref_grads = run("wait")
    R = stage.instances()
    assert R > 1000 and stage.within_bound()
    for bound in (R, R + 1, 3 * R + 12345):
        st, out, grads = run(bound)
        assert st.within_bound() and st.instances() == R
        assert all(torch.equal(a, b) for a, b in zip(ref_out, out))
        assert all(rel_l2(b.cpu().numpy(), a.cpu().numpy()) <= 1e-5 for a, b in zip(ref_grads, grads))
    for bound in (R - 1, R // 2, 1, 0):
        st, out, grads = run(bound)
        assert not st.within_bound() and st.instances() == R
        assert all(torch.isfinite(o.float()).all() for o in out) and all(torch.isfinite(g).all() for g in grads)
    st, out, grads = run(stage.instances())
    assert all(torch.equal(a, b) for a, b in zip(ref_out, out))


def test_frame_with_instance_bounds_matches_the_waiting_frame():
    from retinags_amd.harness import partition, pipeline
    scene, cam, _ = scenes.make_config("C1", shrink=40, resolution_scale=0.5)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 2)
    rel = partition.relation_vector(part, cam)
    subs = [s.requires_grad_(True) for s in pipeline.submodels_from_partition(scene, part, DEV)]
    up = (torch.randn(3, cam.image_height, cam.image_width, generator=torch.Generator().manual_seed(5)) * 1e-2).to(DEV)
    bg = torch.tensor([0.2, 0.3, 0.4], device=DEV)
    cam_d = cam.to(DEV)
    streams = [torch.cuda.current_stream(DEV)] + [torch.cuda.Stream(device=DEV) for _ in range(3)]

    def frame(bounds, lanes):
        for s in subs:
            for p in s.parameters():
                p.grad = None
        out = pipeline.render_frame(cam_d, subs, rel, bg, streams=lanes, instance_bounds=bounds)
        torch.autograd.backward([out["render"]], [up])
        counts = pipeline.check_instance_bounds(out)
        torch.cuda.synchronize()
        return out["render"].detach().clone(), counts, [[p.grad.clone() for p in s.parameters()] for s in subs]

    ref_img, counts, ref_grads = frame(None, streams)
    assert len(counts) >= 2 and min(counts.values()) > 0
    for lanes in (streams, None):
        img, again, grads = frame({m: c + 100 for m, c in counts.items()}, lanes)
        assert again == counts and torch.equal(img, ref_img)
        for ga, gb in zip(ref_grads, grads):
            assert all(rel_l2(b.cpu().numpy(), a.cpu().numpy()) <= 1e-4 for a, b in zip(ga, gb))
    tight = dict(counts)
    worst = max(counts, key=counts.get)
    tight[worst] = counts[worst] // 3
    with pytest.raises(pipeline.InstanceBoundExceeded) as info:
        frame(tight, streams)
    assert info.value.needed == {worst: counts[worst]}
    torch.cuda.synchronize()


@pytest.mark.parametrize("through_frame", [False, True])
def test_backward_writes_every_gradient_row_whatever_the_arrays_held(monkeypatch, through_frame):
    """The reference's shim hands its backward zero-filled gradient tensors
    (K/rasterize_points.cu:165-174) and the kernel writes the rendered Gaussians' rows; here the
    tensors arrive uninitialised and the library writes every row, zeros for the Gaussians that
    were not rendered.  With every output (and the scratch of the sums) poisoned beforehand the
    gradients are those of an unpoisoned run (up to the order of the float atomics), free of
    NaN, and exactly zero where nothing was rendered."""
    from retinags_amd import GaussianRasterizer, rasterizer
    scene, cam, low, up = _small_inputs(n=5000, seed=4)
    scene = dict(scene)
    scene["xyz"] = scene["xyz"].clone()
    scene["xyz"][::3] = 2.0 * cam.camera_center - scene["xyz"][::3]  # every third one behind the camera
    r = GaussianRasterizer(_settings(oracle_settings(cam, low, up, torch.tensor([0.3, 0.2, 0.1]))))

    def run():
        leaves = {k: scene[k].to(DEV).requires_grad_(True) for k in ("xyz", "opacity", "shs", "scales", "rotations")}
        m2d = torch.zeros_like(leaves["xyz"], requires_grad=True)
        kw = dict(means3D=leaves["xyz"], means2D=m2d, opacities=leaves["opacity"], shs=leaves["shs"],
                  scales=leaves["scales"], rotations=leaves["rotations"])
        color, radii, depth, alpha = rasterizer.rasterize_frame([r], [kw])[0] if through_frame else r(**kw)
        g = torch.randn(color.shape, generator=torch.Generator().manual_seed(9)).to(DEV) * 1e-2
        return radii, torch.autograd.grad([color], [m2d] + list(leaves.values()), [g])

    radii, clean = run()
    make = rasterizer._gradient_outputs
    poisoned = []

    def poisoning(*args, **kwargs):
        out = make(*args, **kwargs)
        for name, t in out.items():
            if t is not None and (name != "sums" or kwargs.get("sums") is None):
                t.fill_(float("nan"))
        poisoned.append(out)
        return out

    monkeypatch.setattr(rasterizer, "_gradient_outputs", poisoning)
    radii2, dirty = run()
    assert poisoned and torch.equal(radii, radii2)
    seen = radii > 0
    assert seen.any() and not seen.all()
    for a, b in zip(clean, dirty):
        assert not torch.isnan(b).any()
        assert rel_l2(b.cpu().numpy(), a.cpu().numpy()) <= 1e-4
        assert (b[~seen] == 0).all() and (a[~seen] == 0).all()


def test_partial_images_and_their_gradients_come_packed_for_transport():
    """Colour, depth and alpha of a submodel's render, and their gradients from the compositor, each sit in
    one (5,H,W) block in the reference's wire order (task_utils.py:156-163, 187-195): packing is free."""
    from retinags_amd import GaussianRasterizer
    from retinags_amd.compositor import composite_partial_images, partial_image_package, unpack_partial_image
    scene, cam, low, up = _small_inputs(n=3000, seed=5)
    r = GaussianRasterizer(_settings(oracle_settings(cam, low, up, torch.zeros(3))))
    xyz = scene["xyz"].to(DEV).requires_grad_(True)
    color, radii, depth, alpha = r(means3D=xyz, means2D=torch.zeros_like(xyz), opacities=scene["opacity"].to(DEV),
                                   shs=scene["shs"].to(DEV), scales=scene["scales"].to(DEV), rotations=scene["rotations"].to(DEV))
    package = partial_image_package(color, depth, alpha)
    assert package.shape == (5, cam.image_height, cam.image_width) and package.data_ptr() == color.data_ptr()
    assert torch.equal(package, torch.cat([color, depth, alpha]).detach())
    c, d, a = unpack_partial_image(package)
    assert torch.equal(c, color.detach()) and torch.equal(d, depth.detach()) and torch.equal(a, alpha.detach())
    # tensors that are not one block are concatenated
    other = partial_image_package(color.detach().clone(), depth.detach().clone(), alpha.detach().clone())
    assert torch.equal(other, package) and other.data_ptr() != package.data_ptr()
    # gradients of a layer out of the compositor
    # (as they leave the compositor's backward; a leaf's .grad is a copy that autograd makes of a view)
    layers = [t.detach().clone().requires_grad_(True) for t in (color, depth, alpha)]
    arrived = {}
    for name, t in zip(("render", "depth", "alpha"), layers):
        t.register_hook(lambda g, name=name: arrived.__setitem__(name, g))
    image, dep, alp = composite_partial_images([layers[0]], [layers[1]], [layers[2]], torch.tensor([0.1, 0.2, 0.3], device=DEV))
    (image.sum() + 2 * dep.sum() + 3 * alp.sum()).backward()
    g = partial_image_package(arrived["render"], arrived["depth"], arrived["alpha"])
    assert g.data_ptr() == arrived["render"].data_ptr() and g.shape[0] == 5
    assert torch.equal(g[3:4], layers[1].grad) and torch.equal(g[0:3], layers[0].grad)
    # the rasterizer's backward takes the views as they are
    (color.sum() + depth.sum() + alpha.sum()).backward()
    assert torch.isfinite(xyz.grad).all() and float(xyz.grad.abs().sum()) > 0


def test_a_sort_that_gives_up_is_reported_by_the_next_call():
    """The radix sorts wait for neighbouring workgroups with a bounded number of polls.  With the limit
    set below zero from the host every such wait gives up at once (every kernel still runs to its end):
    the forward must then leave a background-only image, stay inside its buffers, and the next call
    into the library on this device must fail with a message that says so; after that, and with the
    limit restored, the same forward is correct again."""
    import ctypes as C
    from retinags_amd import _capi, GaussianRasterizer
    scene, cam, low, up = _small_inputs(n=30000)
    cam_d = cam.to(DEV)
    s = oracle_settings(cam, low, up, torch.tensor([0.2, 0.4, 0.6]))
    settings = _settings(s)
    args = dict(means3D=scene["xyz"].to(DEV), means2D=torch.zeros(scene["xyz"].shape[0], 3, device=DEV),
                opacities=scene["opacity"].to(DEV), shs=scene["shs"].to(DEV), scales=scene["scales"].to(DEV),
                rotations=scene["rotations"].to(DEV))
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    good, radii, _, _ = GaussianRasterizer(settings)(**args)
    torch.cuda.synchronize()
    assert _capi.lib.rgs_sort_fault(stream) == 0
    assert int((radii > 0).sum()) > 8192      # more than one block of the depth sort, so a look-back happens
    try:
        _capi.check(_capi.lib.rgs_set_lookback_spin_limit(-1))
        color, radii2, depth, alpha = GaussianRasterizer(settings)(**args)
        torch.cuda.synchronize()
    finally:
        _capi.check(_capi.lib.rgs_set_lookback_spin_limit(0))
    assert torch.equal(radii, radii2)                        # the geometry stage does not depend on the sorts
    assert float(alpha.abs().max()) == 0.0                   # empty tile lists: nothing was blended
    assert torch.allclose(color, torch.tensor([0.2, 0.4, 0.6], device=DEV).view(3, 1, 1).expand_as(color))
    with pytest.raises(_capi.RgsError, match="gave up"):
        GaussianRasterizer(settings)(**args)                 # the report surfaces here, and is cleared
    assert _capi.lib.rgs_sort_fault(stream) == 0
    again, _, _, _ = GaussianRasterizer(settings)(**args)
    torch.cuda.synchronize()
    assert torch.equal(again, good)
    assert _capi.lib.rgs_sort_fault(stream) == 0


@pytest.mark.parametrize("with_streams,bvh_depth", [(False, 2), (True, 2), (False, 5), (True, 5)])
def test_frame_rendered_together_matches_one_call_per_submodel(with_streams, bvh_depth):
    """render_frame(together=True) sends the related submodels through rgs_frame_forward_raster /
    rgs_frame_backward (one blend launch per direction for all of them): images bit for bit those of one
    call per submodel, gradients equal up to the order of the atomic sums.  With 32 submodels a frame has more
    layers than one launch takes (16), so every stage goes in two launches."""
    from retinags_amd.harness import partition, pipeline
    scene, cam, _ = scenes.make_config("C1", shrink=300, resolution_scale=0.25)
    part = partition.partition_scene(scene["xyz"], scene["scales"], bvh_depth)
    rel = partition.relation_vector(part, cam)
    assert bvh_depth < 5 or int((rel >= 0).sum()) > 16
    H, W = cam.image_height, cam.image_width
    g = (torch.randn(3, H, W, generator=torch.Generator().manual_seed(2)) * 1e-2).to(DEV)
    bg = torch.tensor([0.3, 0.1, 0.2], device=DEV)
    results = []
    for together in (False, True):
        subs = [s.requires_grad_(True) for s in pipeline.submodels_from_partition(scene, part, DEV)]
        for s in subs:
            s.means2D = torch.zeros_like(s.means3D, requires_grad=True)
        streams = ([torch.cuda.current_stream()] + [torch.cuda.Stream() for _ in range(2)]) if with_streams else None
        out = pipeline.render_frame(cam.to(DEV), subs, rel, bg, streams=streams, together=together)
        torch.autograd.backward([out["render"]], [g])
        torch.cuda.synchronize()
        results.append((out, subs))
    (a, subs_a), (b, subs_b) = results
    for key in ("render", "depth", "alpha"):
        assert torch.equal(a[key], b[key]), key
    for m in a["partial"]:
        for key in ("render", "depth", "alpha", "radii"):
            assert torch.equal(a["partial"][m][key], b["partial"][m][key]), (m, key)
    for sa, sb in zip(subs_a, subs_b):
        for ta, tb in zip(sa.parameters() + [sa.means2D], sb.parameters() + [sb.means2D]):
            assert (ta.grad is None) == (tb.grad is None)
            if ta.grad is not None:
                assert rel_l2(ta.grad.cpu().numpy(), tb.grad.cpu().numpy()) <= 1e-5


def test_rasterize_frame_with_an_empty_layer_and_without_stages():
    """rasterize_frame called directly, one layer of which has no Gaussians."""
    from retinags_amd import GaussianRasterizer
    from retinags_amd.rasterizer import rasterize_frame
    scene, cam, low, up = _small_inputs(n=2000)
    s = oracle_settings(cam, low, up, torch.tensor([0.2, 0.4, 0.6]))
    settings = _settings(s)
    full = dict(means3D=scene["xyz"].to(DEV).requires_grad_(True), means2D=torch.zeros(scene["xyz"].shape[0], 3, device=DEV),
                opacities=scene["opacity"].to(DEV), shs=scene["shs"].to(DEV), scales=scene["scales"].to(DEV),
                rotations=scene["rotations"].to(DEV))
    empty = dict(means3D=torch.zeros(0, 3, device=DEV, requires_grad=True), means2D=torch.zeros(0, 3, device=DEV),
                 opacities=torch.zeros(0, 1, device=DEV), shs=torch.zeros(0, 16, 3, device=DEV),
                 scales=torch.zeros(0, 3, device=DEV), rotations=torch.zeros(0, 4, device=DEV))
    rz = GaussianRasterizer(settings)
    (c0, r0, d0, a0), (c1, r1, d1, a1) = rasterize_frame([rz, rz], [full, empty])
    want = rz(**{k: (v.detach() if k == "means3D" else v) for k, v in full.items()})
    assert torch.equal(c0, want[0]) and torch.equal(r0, want[1]) and torch.equal(d0, want[2]) and torch.equal(a0, want[3])
    assert r1.numel() == 0 and float(c1.detach().abs().max()) == 0.0 and float(a1.detach().abs().max()) == 0.0
    (c0.sum() + c1.sum()).backward(retain_graph=True)
    assert full["means3D"].grad is not None and float(full["means3D"].grad.abs().sum()) > 0
    assert empty["means3D"].grad is not None and empty["means3D"].grad.shape == (0, 3)
    # a second backward of the same graph adds the same gradient again
    once = full["means3D"].grad.clone()
    (c0.sum() + c1.sum()).backward()
    assert rel_l2(full["means3D"].grad.cpu().numpy(), 2.0 * once.cpu().numpy()) <= 1e-5
