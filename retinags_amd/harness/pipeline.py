"""One-GPU render -> composite -> backward loop over the submodels of a partitioned scene:
what the reference does per camera in gather_RenderResult_pool
(parallel_utils/basic_parallel_trainer/result_aggregator.py:22-38), forward_blender_local
(parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:417-434) and the backward
through both, with every submodel resident on the same GPU and rendered one after another.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np
import torch

from ..rasterizer import GaussianRasterizationSettings, GaussianRasterizer, rasterize_frame
from ..compositor import blender_render_result
from .partition import Partition, partition_scene, relation_vector
from .scenes import Camera


@dataclass
class Submodel:
    """The tensors render4renderinfo takes from a BoundedGaussianModel and its shared
    Gaussians (gaussian_renderer/render_half_gs.py:103-110): activated values, box."""
    means3D: torch.Tensor
    opacity: torch.Tensor
    scales: torch.Tensor
    rotations: torch.Tensor
    shs: torch.Tensor
    range_low: torch.Tensor
    range_up: torch.Tensor
    active_sh_degree: int = 3
    means2D: Optional[torch.Tensor] = None   # screen-space placeholder whose gradient densification reads

    def parameters(self) -> List[torch.Tensor]:
        return [self.means3D, self.opacity, self.scales, self.rotations, self.shs]

    def requires_grad_(self, flag: bool = True) -> "Submodel":
        for t in self.parameters():
            t.requires_grad_(flag)
        return self


def submodels_from_partition(scene: Dict[str, torch.Tensor], part: Partition, device, order: str = "given") -> List[Submodel]:
    """A submodel's Gaussians (its own and the straddlers lent to it) as renderer inputs.  order: "given" keeps the
    order of part.members (the reference's: own Gaussians in file order, then the lent ones by lender); "morton"
    stores them along a Z-order curve (partition.morton_order), which changes nothing but the order of the rows."""
    from .partition import morton_order
    if order not in ("given", "morton"):
        raise ValueError("order must be 'given' or 'morton'")
    subs = []
    for k, ids in enumerate(part.members):
        idx = ids if torch.is_tensor(ids) else torch.from_numpy(ids)
        if order == "morton":
            idx = idx[morton_order(scene["xyz"][idx.to(scene["xyz"].device)]).to(idx.device)]
        pick = lambda t: t[idx.to(t.device)].to(device).contiguous()
        subs.append(Submodel(pick(scene["xyz"]), pick(scene["opacity"]), pick(scene["scales"]),
                             pick(scene["rotations"]), pick(scene["shs"]),
                             torch.from_numpy(part.box_low[k]).to(device), torch.from_numpy(part.box_up[k]).to(device)))
    return subs


def reorder_submodel(sub: Submodel, permutation: torch.Tensor) -> Submodel:
    """The same submodel with its Gaussians stored in another order (row k of every tensor becomes row
    permutation[k] of the old one); a screen-space placeholder, if any, is dropped."""
    flag = sub.means3D.requires_grad
    take = lambda t: t.detach()[permutation.to(t.device)].contiguous().requires_grad_(flag)
    return Submodel(take(sub.means3D), take(sub.opacity), take(sub.scales), take(sub.rotations), take(sub.shs), sub.range_low,
                    sub.range_up, sub.active_sh_degree)


def owned_models_from_partition(scene: Dict[str, torch.Tensor], part: Partition, device,
                                spare_fraction: float = 0.0) -> List["SharedGSInfo"]:
    """Every submodel's OWN Gaussians (no lent rows) as the six tensors it shows its neighbours.
    With spare_fraction every tensor has room for that share of its rows (+4096) behind them,
    which is what sharing.merge_shared(append=True) writes the lent rows into."""
    from ..sharing import SharedGSInfo, with_spare_rows
    out = []
    for k in range(len(part.leaves)):
        idx = torch.from_numpy(np.nonzero(part.owner == k)[0])
        spare = int(len(idx) * spare_fraction) + 4096 if spare_fraction > 0 else 0
        pick = lambda t: with_spare_rows(t[idx].to(device).contiguous(), spare)
        xyz = pick(scene["xyz"])
        out.append(SharedGSInfo(xyz, with_spare_rows(torch.zeros_like(xyz), spare), pick(scene["opacity"]), pick(scene["scales"]),
                                pick(scene["rotations"]), pick(scene["shs"])))
    return out


def submodels_from_shared(merged: List["SharedGSInfo"], part: Partition, device) -> List[Submodel]:
    """Renderer inputs from merged (own + lent) tensors, e.g. those of sharing.merge_shared."""
    return [Submodel(m.means3D, m.opacity, m.scales, m.rotations, m.shs, torch.from_numpy(part.box_low[k]).to(device),
                     torch.from_numpy(part.box_up[k]).to(device), means2D=m.means2D) for k, m in enumerate(merged)]


def whole_scene_submodel(scene: Dict[str, torch.Tensor], device, margin: float = 1.0) -> Submodel:
    """A single submodel whose box encloses every Gaussian (bvh_depth = 0)."""
    xyz = scene["xyz"]
    pad = 3.0 * float(scene["scales"].max()) + margin
    low = (xyz.min(dim=0).values - pad).to(device)
    up = (xyz.max(dim=0).values + pad).to(device)
    mv = lambda t: t.to(device).contiguous()
    return Submodel(mv(xyz), mv(scene["opacity"]), mv(scene["scales"]), mv(scene["rotations"]), mv(scene["shs"]), low, up)


class GradNormHelper(torch.autograd.Function):
    """The placeholder through which the reference collects the screen-space gradient norm that
    densification reads (gaussian_renderer/render_half_gs.py:7-19): forward turns an (N,1) meta
    tensor into the (N,3) zeros passed as means2D; backward hands the meta tensor the length of
    each row's (x, y) gradient."""

    @staticmethod
    def forward(ctx, meta: torch.Tensor) -> torch.Tensor:
        if meta.dim() != 2 or meta.shape[1] != 1:
            raise RuntimeError("meta must have shape (N, 1)")
        return torch.zeros((meta.shape[0], 3), dtype=meta.dtype, device=meta.device)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> torch.Tensor:
        return torch.norm(grad_output[:, :2], dim=-1, keepdim=True)


gradNormHelpFunction = GradNormHelper.apply


def raster_settings(cam: Camera, sub: Submodel, bg: torch.Tensor, scaling_modifier: float = 1.0,
                    debug: bool = False) -> GaussianRasterizationSettings:
    return GaussianRasterizationSettings(
        image_height=int(cam.image_height), image_width=int(cam.image_width),
        tanfovx=math.tan(cam.FoVx * 0.5), tanfovy=math.tan(cam.FoVy * 0.5),
        bg=bg, scale_modifier=scaling_modifier, viewmatrix=cam.world_view_transform,
        projmatrix=cam.full_proj_transform, projmatrix_inv=cam.projection_matrix_inv,
        range_low=sub.range_low, range_up=sub.range_up, sh_degree=sub.active_sh_degree,
        campos=cam.camera_center, prefiltered=False, debug=debug)


def _screenspace_placeholder(sub: Submodel) -> torch.Tensor:
    """The zero tensor whose gradient carries the screen-space gradient of the means
    (gaussian_renderer/render.py:16 makes one with zeros_like per render).  Nothing
    ever writes its values, so one block of zeros per submodel serves every frame: a frame that
    takes gradients gets a fresh leaf over that block (its own .grad, no fill), one that does
    not gets the block itself."""
    zeros = getattr(sub, "_still_means2D", None)
    if zeros is None or zeros.shape != sub.means3D.shape or zeros.device != sub.means3D.device \
            or zeros.dtype != sub.means3D.dtype:
        zeros = torch.zeros_like(sub.means3D, requires_grad=False)
        sub._still_means2D = zeros
    return zeros.detach().requires_grad_(True) if sub.means3D.requires_grad else zeros


def render_submodel(cam: Camera, sub: Submodel, bg: torch.Tensor, scaling_modifier: float = 1.0,
                    debug: bool = False, started=None) -> dict:
    """Same call sequence and return dict as render4renderinfo
    (gaussian_renderer/render_half_gs.py:112-182).  `started` is what start_submodel returned
    for the same submodel, if its geometry stage is already in flight."""
    if started is None:
        rasterizer, geometry = GaussianRasterizer(raster_settings=raster_settings(cam, sub, bg, scaling_modifier, debug)), None
    else:
        rasterizer, geometry = started
    means2D = sub.means2D
    if means2D is None:
        means2D = _screenspace_placeholder(sub)
    color, radii, depth, alpha = rasterizer(
        means3D=sub.means3D, means2D=means2D, shs=sub.shs, colors_precomp=None, opacities=sub.opacity,
        scales=sub.scales, rotations=sub.rotations, cov3D_precomp=None, geometry=geometry)
    return RenderResult({"render": color, "viewspace_points": means2D, "radii": radii,
                         "depth": depth, "alpha": alpha, "num_rendered": -1})


@dataclass
class PipelineSwitches:
    """The fields of the reference's PipelineParams that the renderer reads (arguments/__init__.py:71-79)."""
    convert_SHs_python: bool = False
    compute_cov3D_python: bool = False
    debug: bool = False


_SH_C0 = 0.5 * math.sqrt(1.0 / math.pi)
_SH_C1 = math.sqrt(3.0 / (4.0 * math.pi))
_SH_C2 = (0.5 * math.sqrt(15.0 / math.pi), 0.25 * math.sqrt(5.0 / math.pi), 0.25 * math.sqrt(15.0 / math.pi))
_SH_C3 = (0.25 * math.sqrt(35.0 / (2.0 * math.pi)), 0.5 * math.sqrt(105.0 / math.pi), 0.25 * math.sqrt(21.0 / (2.0 * math.pi)),
          0.25 * math.sqrt(7.0 / math.pi), 0.25 * math.sqrt(105.0 / math.pi))


def sh_basis(degree: int, directions: torch.Tensor) -> torch.Tensor:
    """(N, (degree+1)^2) values of the real spherical harmonics in the sign convention of the reference's eval_sh
    (utils/sh_utils.py:57-115) at unit directions (N,3): column k multiplies SH coefficient k."""
    if not 0 <= degree <= 3:
        raise ValueError("SH degree must be 0..3")
    x, y, z = directions.unbind(-1)
    cols = [torch.full_like(x, _SH_C0)]
    if degree > 0:
        cols += [-_SH_C1 * y, _SH_C1 * z, -_SH_C1 * x]
    if degree > 1:
        xx, yy, zz = x * x, y * y, z * z
        cols += [_SH_C2[0] * x * y, -_SH_C2[0] * y * z, _SH_C2[1] * (2 * zz - xx - yy), -_SH_C2[0] * x * z,
                 _SH_C2[2] * (xx - yy)]
    if degree > 2:
        cols += [-_SH_C3[0] * y * (3 * xx - yy), _SH_C3[1] * x * y * z, -_SH_C3[2] * y * (4 * zz - xx - yy),
                 _SH_C3[3] * z * (2 * zz - 3 * xx - 3 * yy), -_SH_C3[2] * x * (4 * zz - xx - yy), _SH_C3[4] * z * (xx - yy),
                 -_SH_C3[0] * x * (xx - 3 * yy)]
    return torch.stack(cols, dim=-1)


def colours_from_sh(shs: torch.Tensor, degree: int, means3D: torch.Tensor, camera_center: torch.Tensor) -> torch.Tensor:
    """The convert_SHs_python branch of render4BoundedGaussianModel (gaussian_renderer/render_half_gs.py:69-74): the
    view-dependent colour of every Gaussian from its SH coefficients (N,16,3) as tensor operations,
    clamp_min(SH(direction) + 0.5, 0), differentiable by autograd."""
    direction = means3D - camera_center.view(1, 3)
    direction = direction / direction.norm(dim=1, keepdim=True)
    basis = sh_basis(degree, direction)                                   # (N, n)
    rgb = torch.einsum("nk,nkc->nc", basis, shs[:, :basis.shape[1], :])
    return torch.clamp_min(rgb + 0.5, 0.0)


def covariance_from_scaling_rotation(scales: torch.Tensor, scaling_modifier: float, rotations: torch.Tensor) -> torch.Tensor:
    """The compute_cov3D_python branch (render_half_gs.py:57-58 -> scene/gaussian_nn_module.py:298-302,
    utils/general_utils.py:79-111): L = R(q / |q|) diag(modifier * s), Sigma = L L^T, returned as its six upper
    entries (xx, xy, xz, yy, yz, zz)."""
    q = rotations / rotations.norm(dim=1, keepdim=True)
    r, x, y, z = q.unbind(-1)
    R = torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y),
                     2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x),
                     2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], dim=-1).view(-1, 3, 3)
    L = R * (scaling_modifier * scales).unsqueeze(1)                      # scales the columns: R @ diag(s)
    sigma = L @ L.transpose(1, 2)
    return torch.stack([sigma[:, 0, 0], sigma[:, 0, 1], sigma[:, 0, 2], sigma[:, 1, 1], sigma[:, 1, 2], sigma[:, 2, 2]], dim=-1)


def render_bounded_model(cam: Camera, sub: Submodel, pipe: PipelineSwitches, bg: torch.Tensor, scaling_modifier: float = 1.0,
                         override_color: Optional[torch.Tensor] = None) -> dict:
    """render4BoundedGaussianModel (gaussian_renderer/render_half_gs.py:21-101) for a Submodel: the same switches decide
    whether the rasterizer gets scales and rotations or a 3D covariance computed by tensor operations, and SH
    coefficients, colours computed from them by tensor operations, or the caller's override_color; same return dict."""
    rasterizer = GaussianRasterizer(raster_settings=raster_settings(cam, sub, bg, scaling_modifier, pipe.debug))
    means2D = sub.means2D
    if means2D is None:
        means2D = _screenspace_placeholder(sub)
    scales = rotations = cov3D_precomp = None
    if pipe.compute_cov3D_python:
        cov3D_precomp = covariance_from_scaling_rotation(sub.scales, scaling_modifier, sub.rotations)
    else:
        scales, rotations = sub.scales, sub.rotations
    shs = colors_precomp = None
    if override_color is None:
        if pipe.convert_SHs_python:
            colors_precomp = colours_from_sh(sub.shs, sub.active_sh_degree, sub.means3D, cam.camera_center)
        else:
            shs = sub.shs
    else:
        colors_precomp = override_color
    color, radii, depth, alpha = rasterizer(means3D=sub.means3D, means2D=means2D, shs=shs, colors_precomp=colors_precomp,
                                            opacities=sub.opacity, scales=scales, rotations=rotations, cov3D_precomp=cov3D_precomp)
    return RenderResult({"render": color, "viewspace_points": means2D, "radii": radii, "depth": depth, "alpha": alpha,
                         "num_rendered": -1})


class RenderResult(dict):
    """What the reference's render() returns for a submodel (gaussian_renderer/__init__.py: "render",
    "viewspace_points", "visibility_filter", "radii", "depth", "alpha", "num_rendered").  The visibility filter
    (radii > 0) is formed when somebody asks for it: a training iteration that does not densify never does."""

    def __missing__(self, key):
        if key == "visibility_filter":
            value = self["radii"] > 0
            self[key] = value
            return value
        raise KeyError(key)


def start_submodel(cam: Camera, sub: Submodel, bg: torch.Tensor, scaling_modifier: float = 1.0, debug: bool = False,
                   instance_bound: Optional[int] = None):
    """Enqueues the geometry stage of a submodel's forward on the current stream without waiting
    for its instance count; hand the result to render_submodel(..., started=...)."""
    rasterizer = GaussianRasterizer(raster_settings=raster_settings(cam, sub, bg, scaling_modifier, debug))
    geometry = rasterizer.enqueue_geometry(means3D=sub.means3D, opacities=sub.opacity, shs=sub.shs,
                                           scales=sub.scales, rotations=sub.rotations, instance_bound=instance_bound)
    return rasterizer, geometry


class InstanceBoundExceeded(RuntimeError):
    """A submodel had more (Gaussian, tile) instances than the room its forward was given;
    `needed` maps submodel id to the count."""

    def __init__(self, needed: Dict[int, int]):
        super().__init__(f"instance bounds exceeded: {needed}")
        self.needed = needed


def check_instance_bounds(frame: dict) -> Dict[int, int]:
    """For a frame rendered with instance_bounds: the instance count of every submodel; raises
    InstanceBoundExceeded if any forward ran out of room (its images are then wrong and the
    frame must be rendered again with larger bounds)."""
    counts = {m: st.instances() if st.P else 0 for m, st in frame.get("stages", {}).items()}
    over = {m: c for m, c in counts.items() if not frame["stages"][m].within_bound()}
    if over:
        raise InstanceBoundExceeded(over)
    return counts


_pools = {}


def _host_pool(n: int):
    from concurrent.futures import ThreadPoolExecutor
    if n not in _pools:
        _pools[n] = ThreadPoolExecutor(max_workers=n, thread_name_prefix="rgs-stream")
    return _pools[n]


def render_frame(cam: Camera, subs: List[Submodel], relation: np.ndarray, background: torch.Tensor,
                 submodel_bg: Optional[torch.Tensor] = None,
                 streams: Optional[List["torch.cuda.Stream"]] = None, host_threads: bool = False,
                 instance_bounds: Optional[Dict[int, int]] = None, together: bool = False,
                 keep_workspaces: bool = False) -> dict:
    """Render every related submodel (black background, as the trainer does:
    trainer4tree_partition.py:397) and composite the partial images in BVH order.

    The reference renders the submodels on different GPUs at the same time.  On one GPU the
    same independence is offered to the hardware through `streams`: submodel k is rendered on
    streams[k % len(streams)] (default priority), so one submodel's short kernels and the tail
    of its blend run beside another's; autograd replays each submodel's backward on the stream
    its forward used.  The compositor runs on the caller's stream after all of them.  The
    The forward is issued in two rounds (all geometry stages, then all sort-and-blend stages): the
    host has to read each submodel's instance count in between, and this way it waits once.
    With host_threads each stream's forward calls are instead issued by a host thread of their
    own (ctypes releases the interpreter lock inside the library); measured no faster, and less
    steady, than the two rounds: the threads contend for the interpreter between the calls.

    together: the related submodels go through rasterize_frame: three library calls per frame, every stage one
    launch for all submodels.  Every forward stage runs on the current stream; `streams`, if given, only offers the
    backward a second stream (the first that is not the current one) for its per-Gaussian half; same results.
    keep_workspaces (with together): the frame also carries, under "workspaces", per submodel id what a single
    forward call returns beside its images: (num_rendered, geomBuffer, binningBuffer, imgBuffer).

    instance_bounds (submodel id -> room for that many instances; with or without `streams`): the
    forward of each submodel is issued in one go, without waiting for its instance count.  The
    stages come back under "stages"; call check_instance_bounds(frame) before using the frame's
    results (after the backward has been issued is early enough).
    """
    device = subs[0].means3D.device
    if submodel_bg is None:
        submodel_bg = torch.zeros(3, device=device)
    related = [m for m in range(len(subs)) if relation[m] >= 0]
    stages = {}
    if together:
        if instance_bounds is not None or host_threads:
            raise ValueError("together=True takes neither instance_bounds nor host_threads")
        main = torch.cuda.current_stream(device)
        lanes = streams if streams else [main]
        rasterizers, inputs = [], []
        for m in related:
            sub = subs[m]
            means2D = sub.means2D
            if means2D is None:
                means2D = _screenspace_placeholder(sub)
            rasterizers.append(GaussianRasterizer(raster_settings=raster_settings(cam, sub, submodel_bg)))
            inputs.append(dict(means3D=sub.means3D, means2D=means2D, shs=sub.shs, opacities=sub.opacity, scales=sub.scales,
                               rotations=sub.rotations))
        taps = [] if keep_workspaces else None
        outs = rasterize_frame(rasterizers, inputs,
                               streams=[lanes[k % len(lanes)].cuda_stream for k in range(len(related))] if streams else None,
                               workspaces=taps)
        partial = {}
        for k, m in enumerate(related):
            color, radii, depth, alpha = outs[k]
            partial[m] = RenderResult({"render": color, "viewspace_points": inputs[k]["means2D"], "radii": radii,
                                       "depth": depth, "alpha": alpha, "num_rendered": -1})
    elif instance_bounds is not None:
        main = torch.cuda.current_stream(device)
        lanes = streams if streams else [main]
        for side in lanes[:len(related)]:
            if side is not main:
                side.wait_stream(main)
        partial = {}

        def forward_in_one_go(k, m):
            with torch.cuda.device(device), torch.cuda.stream(lanes[k % len(lanes)]):
                started = start_submodel(cam, subs[m], submodel_bg, instance_bound=instance_bounds.get(m))
                return m, started[1], render_submodel(cam, subs[m], submodel_bg, started=started)

        if host_threads and len(lanes) > 1:
            # nothing waits for the device here, so a host thread per stream spends its time inside
            # the library's launches, where it does not hold the interpreter lock
            def lane_work(j):
                return [forward_in_one_go(k, m) for k, m in enumerate(related) if k % len(lanes) == j]
            done = [r for rs in _host_pool(len(lanes)).map(lane_work, range(min(len(lanes), len(related)))) for r in rs]
        else:
            done = [forward_in_one_go(k, m) for k, m in enumerate(related)]
        for m, stage, res in sorted(done, key=lambda d: related.index(d[0])):
            stages[m] = stage
            partial[m] = res
        for side in lanes[:len(related)]:
            if side is not main:
                main.wait_stream(side)
        for res in partial.values():
            for t in res.values():
                if torch.is_tensor(t) and t.is_cuda:
                    t.record_stream(main)
    elif not streams:
        partial = {}
        for m in related:
            started = start_submodel(cam, subs[m], submodel_bg)
            stages[m] = started[1]
            partial[m] = render_submodel(cam, subs[m], submodel_bg, started=started)
    else:
        main = torch.cuda.current_stream(device)
        for side in streams[:len(related)]:
            side.wait_stream(main)
        partial = {}
        if host_threads:
            # one host thread per stream: a forward call is some thirty kernel launches, and issued
            # from one thread the four submodels' launches would queue up behind each other
            def forward_on(j):
                with torch.cuda.device(device), torch.cuda.stream(streams[j]):
                    return [(m, render_submodel(cam, subs[m], submodel_bg,
                                                started=start_submodel(cam, subs[m], submodel_bg)))
                            for k, m in enumerate(related) if k % len(streams) == j]
            for done in _host_pool(len(streams)).map(forward_on, range(min(len(streams), len(related)))):
                partial.update(done)
            partial = {m: partial[m] for m in related}
        else:
            # every geometry stage is enqueued before the host waits for the first instance count
            started = {}
            for k, m in enumerate(related):
                with torch.cuda.stream(streams[k % len(streams)]):
                    started[m] = start_submodel(cam, subs[m], submodel_bg)
            for k, m in enumerate(related):
                with torch.cuda.stream(streams[k % len(streams)]):
                    partial[m] = render_submodel(cam, subs[m], submodel_bg, started=started[m])
                    stages[m] = started[m][1]
        for side in streams[:len(related)]:
            main.wait_stream(side)
        for res in partial.values():
            for t in res.values():
                if torch.is_tensor(t) and t.is_cuda:
                    t.record_stream(main)
    out = blender_render_result(partial, relation, background)
    out["partial"] = partial
    out["stages"] = stages
    if together and keep_workspaces:
        out["workspaces"] = {m: taps[k] for k, m in enumerate(related)}
    return out


REFERENCE_LEARNING_RATES = {"means3D": 0.00016, "means2D": 0.0, "opacity": 0.05, "scales": 0.005, "rotations": 0.001,
                            "shs": 0.0025}   # arguments/__init__.py:84-95 (one rate for all SH coefficients here)


def make_optimisers(models: List["SharedGSInfo"], rates: Optional[Dict[str, float]] = None):
    """One Adam per submodel with a parameter group per field, eps 1e-15, as the reference sets up
    (scene/gaussian_nn_module.py:433-443).  The harness trains the activated values directly."""
    from ..optimizer import Adam
    from ..sharing import FIELDS
    rates = REFERENCE_LEARNING_RATES if rates is None else rates
    return [Adam([{"params": [getattr(m, n)], "lr": rates[n], "name": n} for n in FIELDS], lr=0.0, eps=1e-15)
            for m in models]


def training_iteration(models: List["SharedGSInfo"], optimisers, part: Partition, cam: Camera, relation: np.ndarray,
                       gt_image: torch.Tensor, background: torch.Tensor, lambda_dssim: float = 0.2,
                       streams: Optional[List["torch.cuda.Stream"]] = None, append: bool = False) -> dict:
    """One iteration of the reference's training loop for one camera with every submodel on one GPU
    (parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:596-666, without densification
    and logging): share the boundary Gaussians, render every related submodel, composite, take the
    L1 + SSIM loss against gt_image, differentiate back to every submodel's own Gaussians, step the
    optimisers.  Returns the loss terms (device scalars) and the frame."""
    from ..loss import l1_ssim_loss
    from ..sharing import merge_shared, select_straddlers
    device = models[0].means3D.device
    table = select_straddlers(models, part.box_low, part.box_up)
    merged = merge_shared(models, table, reuse_gradients=True, append=append)
    frame = render_frame(cam, submodels_from_shared(merged, part, device), relation, background, streams=streams, together=True)
    loss, l1 = l1_ssim_loss(frame["render"], gt_image, lambda_dssim)
    loss.backward()
    for opt in optimisers:
        opt.step()
        opt.zero_grad(set_to_none=True)
    return {"loss": loss.detach(), "l1": l1, "frame": frame, "lent_rows": int(table.counts.sum())}


@dataclass
class StoredModel:
    """A submodel's trainable tensors as the reference stores them (scene/gaussian_nn_module.py:420-426):
    positions, first and remaining SH coefficients, log scales, quaternions, opacity logits, and the
    (N,1) placeholder whose gradient densification reads."""
    xyz: torch.Tensor
    features_dc: torch.Tensor
    features_rest: torch.Tensor
    scaling: torch.Tensor
    rotation: torch.Tensor
    opacity: torch.Tensor
    means2D_meta: torch.Tensor
    spare_rows: int = 0

    def parameters(self) -> List[torch.Tensor]:
        return [self.xyz, self.features_dc, self.features_rest, self.opacity, self.means2D_meta, self.scaling, self.rotation]

    def activated(self) -> "SharedGSInfo":
        """get_xyz, get_opacity, get_scaling, get_rotation, get_features and the means2D placeholder
        (parallel_utils/basic_parallel_trainer/result_aggregator.py:40-52)."""
        from ..activation import activate_gaussians
        means2D = gradNormHelpFunction(self.means2D_meta)
        if self.spare_rows:
            means2D = _RoomBehind.apply(means2D, self.spare_rows)
        return activate_gaussians(self.xyz, self.features_dc, self.features_rest, self.scaling, self.rotation,
                                  self.opacity, means2D=means2D, spare_rows=self.spare_rows)


class _RoomBehind(torch.autograd.Function):
    """Identity that moves a tensor to the start of an allocation with spare rows behind it."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, spare: int) -> torch.Tensor:
        from ..sharing import with_spare_rows
        return with_spare_rows(t, spare).detach()

    @staticmethod
    def backward(ctx, g: torch.Tensor):
        return g, None


def stored_models_from_partition(scene: Dict[str, torch.Tensor], part: Partition, device,
                                 spare_fraction: float = 0.0) -> List[StoredModel]:
    """Every submodel's own Gaussians in stored form: log of the scene's scales, logit of its
    opacities, its SH coefficients split into the first and the rest."""
    from ..sharing import with_spare_rows
    out = []
    for k in range(len(part.leaves)):
        idx = torch.from_numpy(np.nonzero(part.owner == k)[0])
        spare = int(len(idx) * spare_fraction) + 4096 if spare_fraction > 0 else 0
        pick = lambda t: t[idx].to(device).contiguous()
        opacity = pick(scene["opacity"]).clamp(1e-6, 1 - 1e-6)
        shs = pick(scene["shs"])
        out.append(StoredModel(
            xyz=with_spare_rows(pick(scene["xyz"]), spare), features_dc=shs[:, :1].contiguous(),
            features_rest=shs[:, 1:].contiguous(), scaling=torch.log(pick(scene["scales"])), rotation=pick(scene["rotations"]),
            opacity=torch.log(opacity / (1 - opacity)), means2D_meta=torch.zeros(len(idx), 1, device=device),
            spare_rows=spare))
    return out


def make_stored_optimisers(models: List[StoredModel], scale: float = 1.0):
    """The reference's seven parameter groups per submodel (scene/gaussian_nn_module.py:433-443)."""
    from ..optimizer import Adam
    lr = REFERENCE_LEARNING_RATES
    out = []
    for m in models:
        groups = [(m.xyz, lr["means3D"], "xyz"), (m.features_dc, lr["shs"], "f_dc"), (m.features_rest, lr["shs"] / 20.0, "f_rest"),
                  (m.opacity, lr["opacity"], "opacity"), (m.means2D_meta, 0.0, "means2D_meta"), (m.scaling, lr["scales"], "scaling"),
                  (m.rotation, lr["rotations"], "rotation")]
        out.append(Adam([{"params": [p], "lr": r * scale, "name": n} for p, r, n in groups], lr=0.0, eps=1e-15))
    return out


def stored_training_iteration(models: List[StoredModel], optimisers, part: Partition, cam: Camera, relation: np.ndarray,
                              gt_image: torch.Tensor, background: torch.Tensor, lambda_dssim: float = 0.2,
                              streams: Optional[List["torch.cuda.Stream"]] = None) -> dict:
    """training_iteration from the stored parameters: activation first, and its backward last, so the
    optimisers step what the reference's step (log scales, opacity logits, raw quaternions, split
    SH coefficients).  Lent rows are appended when the models were made with spare rows."""
    from ..loss import l1_ssim_loss
    from ..sharing import merge_shared, select_straddlers
    device = models[0].xyz.device
    shown = [m.activated() for m in models]
    table = select_straddlers(shown, part.box_low, part.box_up)
    merged = merge_shared(shown, table, reuse_gradients=True, append=all(m.spare_rows > 0 for m in models))
    frame = render_frame(cam, submodels_from_shared(merged, part, device), relation, background, streams=streams, together=True)
    loss, l1 = l1_ssim_loss(frame["render"], gt_image, lambda_dssim)
    loss.backward()
    for opt in optimisers:
        opt.step()
        opt.zero_grad(set_to_none=True)
    return {"loss": loss.detach(), "l1": l1, "frame": frame, "lent_rows": int(table.counts.sum())}
