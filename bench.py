#!/usr/bin/env python3
"""Benchmark of the half-Gaussian rasterizer + compositor on one MI355X.

A step is one forward + backward pass of the whole hot path over one synthetic frame:
every related submodel is rendered in turn (preprocess, key duplication, sort, tile ranges,
blend), the partial images are composited front to back, a random upstream gradient is sent
back through the compositor and through every submodel's rasterizer backward.  Inputs
(Gaussian parameters, camera, upstream gradient) are resident in HBM before the timed region.

Prints one JSON line: metric/value per the driver contract, plus `roofline` for the
dominant kernel (HIP-event timing taken live on the stream the kernels run on), `stages`
(every stage's time and achieved rate) and `cpu_baseline` (the CPU checker timed on this
host's cores for the same workload).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
FP32_PEAK_TFLOPS = 157.3   # MI355X fp32 vector
SIMDS = 256 * 4            # compute units x SIMDs
CLOCK_HZ = 2.4e9           # peak engine clock
GRADIENT_AGREEMENT = 1e-4  # relative L2 allowed between the gradients of the timed path and of one call per submodel

def load_traffic_table():
    """HBM bytes per launch of each stage's kernels on the default workload (C1 at full size), measured with
    rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this script.  Counters cannot be read from inside the process, so
    the figures are kept in a small text file beside the profile summaries, which also names the commit they
    were taken at; without that file the line reports null."""
    path = os.path.join(ROOT, "profiles", "c1_hbm_traffic_per_launch.txt")
    table, commit = {}, None
    try:
        for raw in open(path):
            line = raw.strip()
            if line.startswith("# commit:"):
                commit = line.split(":", 1)[1].strip()
            if not line or line.startswith("#"):
                continue
            name, mb = line.split()[:2]
            table[name] = float(mb)
    except (OSError, ValueError):
        return {}, None
    return table, commit


def load_valu_table():
    """Wave-level vector-ALU instructions per launch of the kernels that are bound by instruction issue, on the
    default workload (C1 at full size), from a rocprofv3 SQ_INSTS_VALU run of this script; kept like the traffic
    figures in a small text file that names the commit it was taken at."""
    path = os.path.join(ROOT, "profiles", "c1_valu_instructions_per_launch.txt")
    table, commit = {}, None
    try:
        for raw in open(path):
            line = raw.strip()
            if line.startswith("# commit:"):
                commit = line.split(":", 1)[1].strip()
            if not line or line.startswith("#"):
                continue
            name, millions = line.split()[:2]
            table[name] = float(millions) * 1e6
    except (OSError, ValueError):
        return {}, None
    return table, commit


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="C1", choices=["C0", "C1", "C2", "C3", "C4"])
    ap.add_argument("--shrink", type=float, default=1.0, help="divide the Gaussian count (debugging only)")
    ap.add_argument("--resolution-scale", type=float, default=1.0, help="scale the image size (debugging only)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--forward-only", action="store_true",
                    help="render and composite only (the ms/frame figure; ms_per_step is then the render time)")
    ap.add_argument("--cpu-threads", type=int, default=0)
    ap.add_argument("--streams", type=int, default=0,
                    help="0: every kernel of a frame on the current stream (the default, and the fastest since the gradient "
                         "arrays need no clearing); N > 0: offer the library N HIP streams (it runs the per-Gaussian "
                         "backward beside the blend on the second); value_one_stream is then reported next to value")
    ap.add_argument("--instance-room", type=float, default=0.0,
                    help="if > 0: room for (Gaussian, tile) instances as a multiple of the first frame's count; the "
                         "forward then runs without a host round trip and the count is checked after each frame "
                         "(0: wait for every count before sorting, as the reference does; measured as fast)")
    ap.add_argument("--host-threads", action="store_true",
                    help="issue each stream's forward calls from a host thread of its own")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a 1 GiB device-to-device copy, the known-size reference for HBM traffic counters")
    ap.add_argument("--scene-on", default="auto", choices=["auto", "host", "device"],
                    help="where the synthetic scene is generated and partitioned (auto: C3 and C4 on the device, "
                         "where it takes seconds; the others on the host, so that the CPU baseline sees the same values)")
    ap.add_argument("--no-render-metric", action="store_true",
                    help="skip the second half of the metric (render-only ms/frame at C3 and C4) in the default run")
    ap.add_argument("--apart", action="store_true",
                    help="one rasterizer call per submodel, as the reference issues them (default: the submodels of a frame "
                         "go through one call that blends them in one launch per direction)")
    ap.add_argument("--no-asides", action="store_true", help="skip the stages beside the metric (sharing, loss, optimiser)")
    ap.add_argument("--gaussian-order", default="given", choices=["given", "morton"],
                    help="the order in which a submodel's Gaussians are stored: as the scene generator emitted them (the "
                         "default), or along a Z-order curve, as a loader that sorts them would store them")
    ap.add_argument("--whole-iteration", action="store_true",
                    help="also time one whole training iteration from the stored parameters (activation, sharing, render, loss, "
                         "backward, Adam); not part of the metric")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip fwd+bwd at C0, C2 and C3 and the one-call-per-submodel figure in the default run")
    ap.add_argument("--no-verify", action="store_true",
                    help="skip the check of the timed path (all submodels through one call) against one call per submodel")
    return ap.parse_args()


def ensure_built():
    lib = os.path.join(ROOT, "retinags_amd", "librgs_gfx950.so")
    if not os.path.exists(lib):
        from retinags_amd import build as b
        b.build(verbose=False)


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: all submodels of a frame are rendered on a single MI355X (on its HIP "
              f"streams) and composited there; --gpus {args.gpus} is not supported.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP library is the only implementation).", file=sys.stderr)
        sys.exit(2)
    ensure_built()
    default_run = (args.config == "C1" and not args.forward_only and args.shrink == 1.0 and args.resolution_scale == 1.0)
    line = measure(args, args.config, args.forward_only, asides=not args.no_asides, cpu=not args.no_cpu_baseline,
                   apart_too=default_run and not args.no_other_configs, morton_too=default_run and not args.no_other_configs)
    if default_run and not args.no_render_metric:
        # the second half of the metric: render only (every related submodel's forward and the compositing)
        for name in ("C3", "C4"):
            try:
                sub = measure(args, name, True, asides=False, cpu=not args.no_cpu_baseline, morton_too=not args.no_other_configs)
                line[f"render_ms_per_frame_{name.lower()}"] = {
                    "value": sub["ms_per_step"], "unit": "ms/frame", "ms_per_frame_one_stream": sub["ms_per_step_one_stream"],
                    "verified": sub["verified"], "verification": sub["verification"],
                    "workload": sub["config"]["workload"], "instances": sub["config"]["instances"],
                    "visible": sub["config"]["visible"], "setup_s": sub["config"]["setup_s"],
                    "peak_device_memory_GB": sub["config"]["peak_device_memory_GB"], "roofline": sub["roofline"],
                    "cpu_baseline": sub["cpu_baseline"], "morton_order": sub["morton_order"],
                    "blend_forward": sub["stages"].get("blend_forward"), "stages_ms": {k: v["ms_per_step"] for k, v in sub["stages"].items()},
                    "blend_work": sub["blend_work"]}
            except Exception as ex:   # the first half of the metric must not be lost with the second
                torch.cuda.synchronize()
                line[f"render_ms_per_frame_{name.lower()}"] = {"error": f"{type(ex).__name__}: {ex}"}
    if default_run and not args.no_other_configs:
        # forward + backward at the other configurations the reference's table lists (same step as `value`)
        for name in ("C0", "C2", "C3"):
            try:
                sub = measure(args, name, False, asides=False, cpu=False)
                line[f"fwd_bwd_{name.lower()}"] = {
                    "value": sub["value"], "unit": "it/s", "ms_per_step": sub["ms_per_step"], "steps": sub["steps"],
                    "verified": sub["verified"], "verification": sub["verification"],
                    "workload": sub["config"]["workload"], "instances": sub["config"]["instances"],
                    "visible": sub["config"]["visible"], "sort_passes": sub["config"]["sort_passes"],
                    "peak_device_memory_GB": sub["config"]["peak_device_memory_GB"], "roofline": sub["roofline"],
                    "stages_ms": {k: v["ms_per_step"] for k, v in sub["stages"].items()},
                    "gpu_kernel_ms_per_step": sub["gpu_kernel_ms_per_step"], "blend_work": sub["blend_work"]}
            except Exception as ex:
                torch.cuda.synchronize()
                line[f"fwd_bwd_{name.lower()}"] = {"error": f"{type(ex).__name__}: {ex}"}
    print(json.dumps(line))


def measure(args, config, forward_only, asides, cpu, apart_too=False, morton_too=False):
    """Times `config` and returns the JSON line's dictionary."""
    from retinags_amd import _capi, rasterizer as R
    from retinags_amd.harness import scenes, partition, pipeline

    dev = torch.device("cuda:0")
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats(dev)
    t0 = time.time()
    on_device = args.scene_on == "device" or (args.scene_on == "auto" and config in ("C3", "C4"))
    scene, cam, cfg = scenes.make_config(config, dev if on_device else "cpu", args.shrink, args.resolution_scale)
    depth = cfg["bvh_depth"]
    if depth > 0:
        split = partition.partition_scene_on_device if on_device else partition.partition_scene
        part = split(scene["xyz"], scene["scales"], depth)
        rel = partition.relation_vector(part, cam)
        subs = pipeline.submodels_from_partition(scene, part, dev, order=args.gaussian_order)
        members = part.members
    else:
        part = None
        rel = np.zeros(1, dtype=np.int64)
        subs = [pipeline.whole_scene_submodel(scene, dev)]
        members = [np.arange(scene["xyz"].shape[0])]
    if on_device:
        scene = None   # the submodels hold their own copies; the CPU baseline is not run on such scenes
        torch.cuda.empty_cache()
    cam_d = cam.to(dev)
    H, W = cam.image_height, cam.image_width
    do_backward = bool(cfg["backward"]) and not forward_only
    if do_backward:
        for s in subs:
            s.requires_grad_(True)
    bg = torch.zeros(3, device=dev)
    gen = torch.Generator().manual_seed(cfg["seed"] + 77)
    upstream = (torch.randn(3, H, W, generator=gen) * 1e-2).to(dev)
    related = [m for m in range(len(subs)) if rel[m] >= 0]
    torch.cuda.synchronize()
    setup_s = time.time() - t0

    # the current stream counts as one of them: a process has 4 hardware queues here, and a fifth
    # stream would share a queue with another, which serialises the two
    streams = ([torch.cuda.current_stream(dev)] + [torch.cuda.Stream(device=dev) for _ in range(args.streams - 1)]
               if args.streams > 0 else None)

    bounds = None   # room for each submodel's instances; None: wait for every count
    together = not args.apart and args.instance_room <= 0 and not args.host_threads

    def step(streams=streams, host_threads=args.host_threads, together=together):
        nonlocal bounds
        while True:
            for s in subs:
                for p in s.parameters():
                    p.grad = None
            if do_backward:
                out = pipeline.render_frame(cam_d, subs, rel, bg, streams=streams, host_threads=host_threads,
                                            instance_bounds=bounds, together=together)
                torch.autograd.backward([out["render"]], [upstream])
            else:
                with torch.no_grad():
                    out = pipeline.render_frame(cam_d, subs, rel, bg, streams=streams, host_threads=host_threads,
                                                instance_bounds=bounds, together=together)
            if bounds is None:
                return out
            try:   # the counts have long arrived by now; a frame that ran out of room is rendered again
                pipeline.check_instance_bounds(out)
                return out
            except pipeline.InstanceBoundExceeded as ex:
                bounds.update({m: int(c * args.instance_room) + 4096 for m, c in ex.needed.items()})

    if args.instance_room > 0:
        first = step(host_threads=False)   # waits for the counts, and so learns them
        bounds = {m: int(c * args.instance_room) + 4096 for m, c in pipeline.check_instance_bounds(first).items()}
        del first

    host_ms = {}

    def timed(**kw):
        for _ in range(args.warmup):
            step(**kw)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            step(**kw)
        t2 = time.perf_counter()   # everything is queued; what is left is the device catching up
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        host_ms["one_call_per_submodel" if kw.get("together", together) is False and together else
                "one_stream" if kw.get("streams", streams) is None else "streams"] = (t2 - t1) * 1e3 / args.steps
        return t3 - t1

    elapsed = timed()
    ms_per_step = elapsed * 1e3 / args.steps
    # the same steps with every submodel on the caller's stream, one after the other
    elapsed_one = timed(streams=None) if streams is not None else elapsed
    peak_gb = torch.cuda.max_memory_allocated(dev) / 1e9   # inputs, workspaces and gradients of the timed steps
    # the same steps with one rasterizer call per submodel, as the reference issues them (result_aggregator.py:22-38)
    elapsed_apart = timed(together=False) if (apart_too and together) else None

    # ---- the timed path against one call per submodel, on this very workload
    verification = (verify_timed_path(pipeline, R, _capi, cam_d, cam, subs, rel, bg, upstream, do_backward, streams)
                    if (together and not args.no_verify) else None)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- per-stage time: HIP events recorded by the library on the stream it launches on
    prof_steps = max(1, min(args.steps, 5))
    _capi.stage_timing(True)
    for _ in range(prof_steps):
        step(streams=None)  # one stream, so that consecutive events bracket one stage each
    stage_ms = _capi.stage_timing_read()
    _capi.stage_timing(False)

    # ---- work sizes for the algorithmic byte / flop counts
    P_tot = P_vis = R_tot = 0
    counters = np.zeros(_capi.WORK_COUNTERS, dtype=np.uint64)
    e = torch.Tensor([])
    with torch.no_grad():
        for m in related:
            s = subs[m]
            outs = R._rasterize_forward(bg, s.means3D.detach(), e, s.opacity.detach(), s.scales.detach(),
                                        s.rotations.detach(), 1.0, e, cam_d.world_view_transform,
                                        cam_d.full_proj_transform, cam_d.projection_matrix_inv, s.range_low,
                                        s.range_up, cam.tanfovx, cam.tanfovy, H, W, s.shs.detach(), 3,
                                        cam_d.camera_center, False, False)
            Rm, _, _, _, radii, geom, binning, img = outs
            Pm = int(s.means3D.shape[0])
            P_tot += Pm
            P_vis += int((radii > 0).sum())
            R_tot += Rm
            cnt = torch.zeros(_capi.WORK_COUNTERS, dtype=torch.int64, device=dev)
            _capi.check(_capi.lib.rgs_blend_work_counters(
                Pm, Rm, W, H, cam.tanfovx, cam.tanfovy, _capi.ptr(cam_d.projection_matrix_inv),
                _capi.ptr(s.range_low), _capi.ptr(s.range_up), C.c_void_p(0), _capi.ptr(geom), _capi.ptr(binning),
                _capi.ptr(img), _capi.ptr(cnt), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
            counters += cnt.cpu().numpy().astype(np.uint64)
            del outs, geom, binning, img
    nA, nB, nC, nD, nE, nBl, nCl, nAl = (float(v) for v in counters)
    K = len(related)
    T = ((W + 15) // 16) * ((H + 15) // 16)
    N = W * H
    tile_bits = int(_capi.lib.rgs_get_higher_msb(T))
    passes = min((tile_bits + 8) // 9, (tile_bits + 7) // 8)   # of the instance sort, on the tile key: digits of up to 9 bits
    # The backward revisits, per pixel, the entries up to the last blended one: nAl of the nA visits.
    flops_fwd = 12 * nA + 3 * nB + 27 * nC + 3 * nD + 14 * nE
    flops_bwd = 12 * nAl + 3 * nBl + 27 * nCl + 80 * nE
    # Algorithmic bytes per frame of every HBM-bound stage (one launch per submodel; the sort
    # kernels run `passes` times per submodel).
    alg_bytes = {
        # mean in, radius and tile count out for all; scale, rotation, opacity, SH row in and depth, clamp flags,
        # 64-byte record out for the rendered ones
        "preprocess_forward": 20.0 * P_tot + (224.0 + 69.0) * P_vis,
        # depths and tile counts of all in; for the visible ones the (depth key, index and tile count) pairs out, 3 passes
        # over them (the last writes index and tile count apart), the tile counts in depth order in twice (block totals,
        # scan) and their offsets out
        "depth_order": 8.0 * P_tot + (8.0 + 3 * 16.0 + 12.0) * P_vis,
        # per rendered Gaussian its place in the depth order, its offset and its 64-byte record in; key and index out per instance
        "duplicate_with_keys": 72.0 * P_vis + 8.0 * R_tot,
        "sort_setup": 4.0 * R_tot,
        "sort_onesweep": 16.0 * R_tot * passes,
        "tile_ranges": 4.0 * R_tot + 16.0 * T * K,
        # the sorted keys in, the filed positions out (at most four per instance; counted as one)
        "strip_filing": 8.0 * R_tot + 16.0 * T * K,
        # the rows of sums the backward blend adds into (the gradient tensors themselves need no clearing)
        "clear_gradients": 48.0 * P_tot,
        # the radius of every Gaussian in; sums, mean, SH, scale, rotation, clamp flags of the rendered ones in; for every
        # Gaussian the six gradient rows a frame hands out (mean2D, opacity, mean3D, SH, scale, rotation: zeros for the
        # ones that were not rendered)
        "preprocess_backward": 285.0 * P_vis + (4.0 + 248.0) * P_tot,
        "composite_forward": (20.0 * K + 20.0) * N,
        "composite_backward": (40.0 * K + 20.0) * N,
    }
    alg_flops = {"blend_forward": flops_fwd, "blend_backward": flops_bwd}
    # Where this design's bytes differ from those of the reference's design, both are carried.  The reference's backward
    # preprocess writes the rendered rows only, into arrays its caller has cleared (4 P + 559 P_vis, or with that clearing
    # 304 P more); here every row of the dense outputs is written once, zeros included.  The reference sorts 12-byte pairs
    # on (tile << 32 | depth) in ceil((32 + bits) / 8) passes after one read of the keys (R (8 + 24 p)); here the instances
    # are emitted in depth order and sorted on the tile alone, 8-byte pairs, ceil(bits / 8) passes.
    ref_passes = (32 + int(_capi.lib.rgs_get_higher_msb(T)) + 7) // 8
    reference_design_bytes = {
        "preprocess_backward": {"rendered_rows_only": 4.0 * P_tot + 559.0 * P_vis,
                                "with_the_clearing_of_the_outputs": (4.0 + 304.0) * P_tot + 559.0 * P_vis},
        "sort_onesweep": {f"one_sort_of_12_byte_pairs_in_{ref_passes}_passes": R_tot * (8.0 + 24.0 * ref_passes)},
    }

    stages = {}
    for name, (ms, launches) in stage_ms.items():
        per_step = ms / prof_steps
        entry = {"ms_per_step": round(per_step, 4), "launches_per_step": launches / prof_steps,
                 "avg_launch_ms": round(ms / max(launches, 1), 5)}
        if name in alg_bytes and per_step > 0:
            entry["bound"] = "hbm"
            entry["achieved_GBps"] = round(alg_bytes[name] / (per_step * 1e-3) / 1e9, 2)
            entry["frac"] = round(entry["achieved_GBps"] / HBM_PEAK_GBS, 4)
        if name in reference_design_bytes and per_step > 0:
            # the same stage time priced with the bytes of the reference's design (an equivalent rate, not traffic)
            entry["by_reference_design_bytes"] = {
                k: {"bytes": v, "equivalent_GBps": round(v / (per_step * 1e-3) / 1e9, 2),
                    "frac": round(v / (per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)} for k, v in reference_design_bytes[name].items()}
        if name in alg_flops and per_step > 0:
            entry["bound"] = "valu"
            entry["achieved_TFLOPs"] = round(alg_flops[name] / (per_step * 1e-3) / 1e12, 3)
            entry["frac"] = round(entry["achieved_TFLOPs"] / FP32_PEAK_TFLOPS, 4)
        stages[name] = entry
    dominant = max(stages, key=lambda n: stages[n]["ms_per_step"]) if stages else None
    roofline = None
    if dominant is not None:
        d = stages[dominant]
        if d.get("bound") == "hbm":
            roofline = {"kernel": dominant, "bound": "hbm", "achieved": d["achieved_GBps"], "peak": HBM_PEAK_GBS,
                        "unit": "GB/s", "frac": d["frac"], "traffic": None}
        elif d.get("bound") == "valu":
            roofline = {"kernel": dominant, "bound": "valu", "achieved": d["achieved_TFLOPs"],
                        "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": d["frac"], "traffic": None,
                        "bound_note": "fp32 vector-ALU issue (per-pixel compare / exp / blend arithmetic, no dense "
                                      "contraction, so no MFMA); peak is the published 157.3 TFLOP/s fp32 figure, which "
                                      "counts packed two-wide fp32 instructions; the library is built with those switched "
                                      "off, so full-rate issue of fused multiply-adds is 78.6 TFLOP/s",
                        "frac_of_unpacked_fp32_issue_peak": round(d["achieved_TFLOPs"] / (FP32_PEAK_TFLOPS / 2), 4)}
        if roofline is not None:
            full_c1 = config == "C1" and args.shrink == 1.0 and args.resolution_scale == 1.0
            traffic, commit = load_traffic_table()
            if full_c1 and dominant in traffic:
                roofline["traffic"] = traffic[dominant] * 1e6  # bytes per launch
                roofline["traffic_measured_at_commit"] = commit
            valu, valu_commit = load_valu_table()
            if full_c1 and dominant in valu and d.get("bound") == "valu":
                # a SIMD has 16 lanes: a wave-level instruction occupies it for 4 cycles
                issue_ms = valu[dominant] * 4 / (SIMDS * CLOCK_HZ) * 1e3
                roofline["valu_issue"] = {"wave_instructions": valu[dominant], "issue_ms": round(issue_ms, 4),
                                          "frac_of_launch": round(issue_ms / d["avg_launch_ms"], 4),
                                          "simds": SIMDS, "clock_GHz": CLOCK_HZ / 1e9, "measured_at_commit": valu_commit}
            roofline["timing"] = "HIP events on the launching stream, all submodels on one stream"
            roofline["avg_launch_ms"] = d["avg_launch_ms"]
            roofline["launches_per_step"] = d["launches_per_step"]

    gpu_stage_ms = sum(v["ms_per_step"] for v in stages.values())
    evals = {
        "visits_per_frame": nA, "exp_per_frame": nB, "blended_per_frame": nE, "backward_visits_per_frame": nAl,
        "fwd_visits_per_s": round(nA / (stages["blend_forward"]["ms_per_step"] * 1e-3), 1)
        if "blend_forward" in stages and stages["blend_forward"]["ms_per_step"] > 0 else None,
    }

    # ---- the step before the path: who lends which Gaussians to whom, and the merged inputs
    def aside(fn):
        """The sections beside the metric must not take the metric's line with them."""
        try:
            return fn()
        except Exception as ex:   # reported in the line instead
            torch.cuda.synchronize()
            return {"error": f"{type(ex).__name__}: {ex}"}

    asides = asides and scene is not None
    sharing = (aside(lambda: {"appending": sharing_stages(scene, part, dev, prof_steps, True),
                              "copying": sharing_stages(scene, part, dev, prof_steps, False)})
               if (part is not None and asides) else None)

    # ---- the steps after the path: image loss with its gradient, and the optimiser step
    after = aside(lambda: training_stages(subs, H, W, dev, prof_steps)) if (do_backward and asides) else None

    # ---- everything together: one training iteration for this camera
    whole = (aside(lambda: whole_iteration(scene, part, cam_d, rel, bg, streams, dev, args.steps))
             if (part is not None and do_backward and asides and args.whole_iteration) else None)

    # ---- the same frame with every submodel's Gaussians stored along a Z-order curve instead of in the order the scene
    # generator emitted them: what a loader that sorts its Gaussians hands the rasterizer (same Gaussians, same images)
    morton = None
    if morton_too and args.gaussian_order == "given" and depth > 0:
        for m in related:
            subs[m] = pipeline.reorder_submodel(subs[m], partition.morton_order(subs[m].means3D.detach()))
        torch.cuda.empty_cache()
        elapsed_m = timed()
        _capi.stage_timing(True)
        for _ in range(prof_steps):
            step(streams=None)
        stage_m = _capi.stage_timing_read()
        _capi.stage_timing(False)
        morton = {"value": round(args.steps / elapsed_m, 4), "unit": "it/s", "ms_per_step": round(elapsed_m * 1e3 / args.steps, 3),
                  "stages_ms": {k: round(v[0] / prof_steps, 4) for k, v in stage_m.items()},
                  "order": "each submodel's Gaussians sorted by the Morton code of their centres (10 bits per axis)"}

    # ---- host-CPU baseline: the CPU checker on the same frame, same seeded inputs
    cpu_line = None
    if cpu and scene is not None:
        cpu_line = cpu_baseline(scene, members, part, cam, rel, related, upstream.cpu().numpy(), do_backward, args)
    elif cpu and not do_backward:
        # a scene that lives on the device only (C3, C4): the render on the CPU checker, one submodel copied to the host at a time
        cpu_line = cpu_render_baseline(subs, cam, rel, related, args)

    return {
        "metric": "fwd+bwd iterations/s, 5.6M Gaussians, 1600x1036, 4 composited submodels"
        if (config == "C1" and do_backward) else f"fwd{'+bwd' if do_backward else ''} iterations/s, config {config}",
        "value": round(args.steps / elapsed, 4), "unit": "it/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        # every submodel on one stream, rendered strictly one after the other (`value` offers the independent
        # submodels to the GPU on several HIP streams; no work differs)
        "value_one_stream": round(args.steps / elapsed_one, 4), "ms_per_step_one_stream": round(elapsed_one * 1e3 / args.steps, 3),
        # one rasterizer call per submodel, as the reference issues them (the default batches the submodels of a frame)
        "value_apart": round(args.steps / elapsed_apart, 4) if elapsed_apart else None,
        "ms_per_step_apart": round(elapsed_apart * 1e3 / args.steps, 3) if elapsed_apart else None,
        # the timed calls (all submodels through one call per stage) checked against one call per submodel on this workload
        "verified": verification["verified"] if verification else None, "verification": verification,
        # not the metric's workload order: the same Gaussians stored along a Z-order curve (see measure())
        "morton_order": morton,
        # how long the host takes to queue a step (the forward's waits for the instance counts included)
        "host_ms_per_step": {k: round(v, 3) for k, v in host_ms.items()},
        "config": {"workload": f"{config}: {cfg['n']} Gaussians, {W}x{H}, bvh_depth={depth} "
                               f"({K} of {len(subs)} submodels related), SH degree 3, "
                               f"{'fwd+bwd' if do_backward else 'fwd only'}",
                   "gaussians_rendered_incl_shared": P_tot, "visible": P_vis, "instances": R_tot,
                   "tiles": T, "sort_passes": passes, "setup_s": round(setup_s, 1),
                   "scene_generated_on": "device" if on_device else "host",
                   "gaussian_order": "as generated (uniformly random in memory)" if args.gaussian_order == "given" else "Morton order per submodel",
                   "streams": args.streams,
                   "submodels_of_a_frame": "one call, blended in one launch per direction" if together else "one call each",
                   "peak_device_memory_GB": round(peak_gb, 2),
                   "instance_room": (f"{args.instance_room} x the first frame's count, checked after every frame"
                                     if bounds is not None else "sized from each call's count (host waits)")},
        "roofline": roofline, "cpu_baseline": cpu_line, "stages": stages, "gpu_kernel_ms_per_step": round(gpu_stage_ms, 3),
        "blend_work": evals, "sharing": sharing, "loss_and_optimiser": after, "training_iteration": whole,
    }


def sharing_stages(scene, part, dev, repeats, append):
    """Times the selection of boundary straddlers, the merge of every submodel's input and the
    backward of the merge (not part of a step: the step starts from merged inputs).  HIP events
    recorded by the library on the launching stream; algorithmic bytes: one read of means and
    scales per Gaussian and 4 per lent row for the selection, one read and one write of every
    merged row (59 floats) for the merge, one read of a lent row's gradient (62 floats) and a
    read-modify-write of the lender's row for the backward.  append: a submodel's own rows stay in
    place and only the lent rows move; otherwise the merge copies the own rows too, as the
    reference's torch.cat does."""
    from retinags_amd import _capi, sharing
    from retinags_amd.harness import pipeline
    models = pipeline.owned_models_from_partition(scene, part, dev, spare_fraction=0.1 if append else 0.0)
    for m in models:
        for t in m.fields():
            t.requires_grad_(True)
    K = len(models)

    def once():
        table = sharing.select_straddlers(models, part.box_low, part.box_up)
        merged = sharing.merge_shared(models, table, reuse_gradients=True, append=append)
        outs = [t for m in merged for t in m.fields()]
        torch.autograd.backward(outs, [torch.ones_like(t) for t in outs])
        for m in models:
            for t in m.fields():
                t.grad = None
        return table

    table = once()
    torch.cuda.synchronize()
    _capi.stage_timing(True)
    t0 = time.perf_counter()
    for _ in range(repeats):
        once()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / repeats
    ms = _capi.stage_timing_read()
    _capi.stage_timing(False)
    torch_ms = None
    if append:   # measured once, beside the appending variant
        torch_ms = _timed_ms(lambda: _sharing_by_tensor_expressions(models, part.box_low, part.box_up, dev), repeats)
    owned = float(sum(table.own))
    lent = float(table.counts.sum())
    merged_rows = owned + lent
    alg = {"straddler_select": 24.0 * owned + 4.0 * lent,
           "merge_rows": 2 * 236.0 * (lent if append else merged_rows) + 4.0 * lent,
           "merge_rows_backward": (248.0 + 2 * 248.0 + 4.0) * lent}
    out = {"owned_gaussians": int(owned), "lent_rows": int(lent), "submodels": K, "wall_ms_per_pass": round(wall_ms, 3),
           "own_rows": "in place, lent rows appended behind them" if append else "copied into the merged arrays"}
    if torch_ms is not None:
        # the same selection, merge and backward written as the reference writes them: boolean-mask
        # indexing per (source, destination) pair and torch.cat per field, differentiated by autograd
        out["tensor_expression_wall_ms_per_pass"] = round(torch_ms, 3)
    for name, (total, launches) in ms.items():
        per = total / repeats
        out[name] = {"ms_per_pass": round(per, 4), "launches_per_pass": launches / repeats,
                     "achieved_GBps": round(alg[name] / (per * 1e-3) / 1e9, 1) if name in alg and per > 0 else None}
        if out[name]["achieved_GBps"] is not None:
            out[name]["frac"] = round(out[name]["achieved_GBps"] / HBM_PEAK_GBS, 4)
    return out


def whole_iteration(scene, part, cam_d, rel, bg, streams, dev, repeats):
    """From the stored parameters and back to them: activation, sharing of the boundary Gaussians,
    render and composite, L1 + SSIM loss, backward through all of it, Adam.  Wall clock per iteration
    with the host included (learning rates scaled down so that the scene stays the workload it is);
    the activation kernels' own times from the library's stage events.  Not the metric of `value`,
    which is the rasterizer's forward + backward."""
    from retinags_amd import _capi
    from retinags_amd.harness import pipeline
    models = pipeline.stored_models_from_partition(scene, part, dev, spare_fraction=0.1)
    for m in models:
        for t in m.parameters():
            t.requires_grad_(True)
    optimisers = pipeline.make_stored_optimisers(models, scale=1e-3)
    H, W = cam_d.image_height, cam_d.image_width
    gt = torch.rand(3, H, W, generator=torch.Generator().manual_seed(11)).to(dev)
    run = lambda: pipeline.stored_training_iteration(models, optimisers, part, cam_d, rel, gt, bg, streams=streams)
    ms = _timed_ms(run, repeats)
    _capi.stage_timing(True)
    run()
    stage = _capi.stage_timing_read()
    _capi.stage_timing(False)
    n = float(sum(int(m.xyz.shape[0]) for m in models))

    def activations_by_tensor_expressions():
        import torch.nn.functional as F
        for m in models:
            outs = [torch.cat((m.features_dc, m.features_rest), dim=1), torch.exp(m.scaling), F.normalize(m.rotation),
                    torch.sigmoid(m.opacity)]
            torch.autograd.backward(outs, [torch.ones_like(o) for o in outs])
            for t in m.parameters():
                t.grad = None

    def activations_by_the_library():
        for m in models:
            shown = m.activated()
            outs = [shown.shs, shown.scales, shown.rotations, shown.opacity]
            torch.autograd.backward(outs, [torch.ones_like(o) for o in outs])
            for t in m.parameters():
                t.grad = None

    out = {"ms_per_iteration": round(ms, 3), "iterations_per_s": round(1e3 / ms, 2),
           "activation_fwd_bwd_wall_ms": round(_timed_ms(activations_by_the_library, repeats), 3),
           "activation_tensor_expression_wall_ms": round(_timed_ms(activations_by_tensor_expressions, repeats), 3),
           "steps": f"activate, select + merge straddlers (appended), render + composite, L1+SSIM loss, backward, "
                    f"Adam ({7 * len(models)} tensors)"}
    # algorithmic bytes: 224 in + 224 out per Gaussian forward (56 floats: SH, scale, rotation, opacity);
    # backward reads their gradients, the stored rotation and the activated scale / opacity, writes 224
    for name, per_gaussian in (("activate_forward", 448.0), ("activate_backward", 224.0 + 32.0 + 224.0)):
        if name in stage and stage[name][0] > 0:
            t = stage[name][0]
            out[name] = {"ms_per_iteration": round(t, 4), "launches": stage[name][1],
                         "achieved_GBps": round(per_gaussian * n / (t * 1e-3) / 1e9, 1),
                         "frac": round(per_gaussian * n / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def _timed_ms(fn, repeats):
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(repeats):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / repeats


def _sharing_by_tensor_expressions(models, box_low, box_up, dev):
    """What the kernels of the sharing stage replace, as stock tensor operations on the same GPU
    (for the timing beside them only; the checker of the tests is elsewhere)."""
    K = len(models)
    low = [torch.tensor(box_low[k], device=dev) for k in range(K)]
    up = [torch.tensor(box_up[k], device=dev) for k in range(K)]
    parts = [[m.fields()] for m in models]           # own rows first
    for s_id, m in enumerate(models):
        reach = (m.scales.max(dim=-1, keepdim=True).values * 3).clamp(min=0)
        hi, lo = m.means3D + reach, m.means3D - reach
        cand = ((hi >= up[s_id]) | (lo <= low[s_id])).any(dim=-1)
        cand_fields = [f[cand] for f in m.fields()]
        hi_c, lo_c = hi[cand], lo[cand]
        for d_id in range(K):
            if d_id == s_id:
                continue
            meets = ((hi_c >= low[d_id]) & (lo_c <= up[d_id])).all(dim=-1)
            parts[d_id].append([f[meets] for f in cand_fields])
    merged = [[torch.cat([p[f] for p in parts[d_id]], dim=0) for f in range(6)] for d_id in range(K)]
    outs = [t for m in merged for t in m]
    torch.autograd.backward(outs, [torch.ones_like(t) for t in outs])
    for m in models:
        for t in m.fields():
            t.grad = None


def _loss_by_tensor_expressions(image, gt, lambda_dssim):
    """L1 + SSIM as 11x11 grouped convolutions and elementwise operations, with autograd."""
    import torch.nn.functional as F
    g = torch.tensor([np.exp(-(x - 5) ** 2 / (2 * 1.5 ** 2)) for x in range(11)], dtype=torch.float32, device=image.device)
    g = (g / g.sum()).unsqueeze(1)
    window = (g @ g.t()).expand(3, 1, 11, 11).contiguous()
    blur = lambda t: F.conv2d(t.unsqueeze(0), window, padding=5, groups=3)
    mu1, mu2 = blur(image), blur(gt)
    s11, s22, s12 = blur(image * image) - mu1 * mu1, blur(gt * gt) - mu2 * mu2, blur(image * gt) - mu1 * mu2
    ssim = (((2 * mu1 * mu2 + 1e-4) * (2 * s12 + 9e-4)) / ((mu1 * mu1 + mu2 * mu2 + 1e-4) * (s11 + s22 + 9e-4))).mean()
    loss = (1 - lambda_dssim) * (image - gt).abs().mean() + lambda_dssim * (1 - ssim)
    loss.backward()
    image.grad = None


def training_stages(subs, H, W, dev, repeats):
    """Times the image loss (forward and backward) at the frame's size and one Adam step over the
    59 trainable floats (+1 untrained placeholder) of every Gaussian the submodels own, in the
    reference's seven parameter groups per submodel.  Not part of a step.  Algorithmic bytes: the
    loss reads image and ground truth and writes three derivative maps (20 B per pixel and channel),
    its backward reads the five and writes the gradient (24 B); Adam reads parameter, gradient and
    two moments and writes three of them (28 B per float)."""
    from retinags_amd import _capi
    from retinags_amd.loss import l1_ssim_loss
    from retinags_amd.optimizer import Adam
    gen = torch.Generator().manual_seed(4)
    gt = torch.rand(3, H, W, generator=gen).to(dev)
    image = (gt * 0.8 + 0.1 * torch.rand(3, H, W, generator=gen).to(dev)).requires_grad_(True)
    widths = [3, 3, 45, 1, 1, 3, 4]          # xyz, f_dc, f_rest, opacity, means2D_meta, scaling, rotation
    lrs = [0.00016, 0.0025, 0.0025 / 20.0, 0.05, 0.0, 0.005, 0.001]
    optimisers, floats = [], 0
    for s in subs:
        n = int(s.means3D.shape[0])
        params = [torch.nn.Parameter(torch.randn(n, w, device=dev) * 0.1) for w in widths]
        for p in params:
            p.grad = torch.randn_like(p) * 1e-3
        floats += n * sum(widths)
        optimisers.append(Adam([{"params": [p], "lr": lr} for p, lr in zip(params, lrs)], lr=0.0, eps=1e-15))

    def once():
        loss, _ = l1_ssim_loss(image, gt, 0.2)
        loss.backward()
        image.grad = None
        for o in optimisers:
            o.step()

    once()
    torch.cuda.synchronize()
    _capi.stage_timing(True)
    for _ in range(repeats):
        once()
    ms = _capi.stage_timing_read()
    _capi.stage_timing(False)
    loss_torch_ms = _timed_ms(lambda: _loss_by_tensor_expressions(image, gt, 0.2), repeats)

    def loss_once():
        loss, _ = l1_ssim_loss(image, gt, 0.2)
        loss.backward()
        image.grad = None
    loss_ms = _timed_ms(loss_once, repeats)
    adam_ms = _timed_ms(lambda: [o.step() for o in optimisers], repeats)
    stock = [torch.optim.Adam(o.param_groups, lr=0.0, eps=1e-15) for o in optimisers]
    adam_torch_ms = _timed_ms(lambda: [o.step() for o in stock], repeats)
    pixels = 3.0 * H * W
    alg = {"l1_ssim_forward": 20.0 * pixels, "l1_ssim_backward": 24.0 * pixels, "adam_step": 28.0 * floats}
    out = {"image": f"3x{H}x{W}", "adam_floats": floats,
           # wall clock per pass, host included, beside the same step written with stock tensor operations
           # (conv2d expression + autograd; torch.optim.Adam) on the same GPU
           "loss_fwd_bwd_wall_ms": round(loss_ms, 3), "loss_tensor_expression_wall_ms": round(loss_torch_ms, 3),
           "adam_wall_ms": round(adam_ms, 3), "adam_torch_optim_wall_ms": round(adam_torch_ms, 3)}
    for name, (total, launches) in ms.items():
        per = total / repeats
        out[name] = {"ms_per_pass": round(per, 4), "launches_per_pass": launches / repeats}
        if name in alg and per > 0:
            out[name]["achieved_GBps"] = round(alg[name] / (per * 1e-3) / 1e9, 1)
            out[name]["frac"] = round(out[name]["achieved_GBps"] / HBM_PEAK_GBS, 4)
    return out


def verify_timed_path(pipeline, R, _capi, cam_d, cam, subs, rel, bg, upstream, do_backward, streams):
    """One frame through the calls that were timed (every submodel of the frame in one call per stage:
    rgs_frame_forward_geom / _raster / rgs_frame_backward) against one call per submodel (rgs_forward_geom /
    rgs_forward_raster / rgs_backward) on the same inputs: instance counts, radii, images and n_contrib must agree bit
    for bit, the composited image too, and every gradient to GRADIENT_AGREEMENT relative L2 (the same atomic sums in
    another order; the line also carries what a repeat of the per-submodel calls differs from itself by)."""
    H, W = cam.image_height, cam.image_width
    related = [m for m in range(len(subs)) if rel[m] >= 0]
    for s in subs:
        for p in s.parameters():
            p.grad = None
    fields = ("means3D", "opacity", "scales", "rotations", "shs")
    grad_ctx = torch.enable_grad() if do_backward else torch.no_grad()
    with grad_ctx:
        frame = pipeline.render_frame(cam_d, subs, rel, bg, streams=streams, together=True, keep_workspaces=True)
        if do_backward:
            torch.autograd.backward([frame["render"]], [upstream])
    frame_grads = {m: {f: getattr(subs[m], f).grad for f in fields} for m in related} if do_backward else None
    for s in subs:
        for p in s.parameters():
            p.grad = None
    im = _capi.image_layout(W, H)
    e = torch.Tensor([])
    ok, mismatches, worst, floor = True, [], 0.0, 0.0
    with torch.no_grad():
        for m in related:
            s = subs[m]
            outs = R._rasterize_forward(bg, s.means3D.detach(), e, s.opacity.detach(), s.scales.detach(), s.rotations.detach(),
                                        1.0, e, cam_d.world_view_transform, cam_d.full_proj_transform, cam_d.projection_matrix_inv,
                                        s.range_low, s.range_up, cam.tanfovx, cam.tanfovy, H, W, s.shs.detach(), 3,
                                        cam_d.camera_center, False, False)
            Rn, geom, binning, img = frame["workspaces"][m]
            layer = frame["partial"][m]
            n0, n1 = im["n_contrib"], im["n_contrib"] + 4 * W * H
            same = (outs[0] == Rn and torch.equal(outs[4], layer["radii"]) and torch.equal(outs[1], layer["render"].detach())
                    and torch.equal(outs[2], layer["depth"].detach()) and torch.equal(outs[3], layer["alpha"].detach())
                    and torch.equal(outs[7][n0:n1], img[n0:n1]))
            if not same:
                ok = False
                mismatches.append(int(m))
            del outs
    if do_backward:
        with torch.enable_grad():
            again = pipeline.render_frame(cam_d, subs, rel, bg, together=False)
            ok = ok and torch.equal(again["render"], frame["render"])
            torch.autograd.backward([again["render"]], [upstream])
        for m in related:
            for f in fields:
                a, b = frame_grads[m][f], getattr(subs[m], f).grad
                err = float((a - b).double().norm() / b.double().norm().clamp_min(1e-300))
                worst = max(worst, err)
        # the noise floor of that comparison: the per-submodel calls against themselves, once more
        with torch.enable_grad():
            once_more = pipeline.render_frame(cam_d, subs, rel, bg, together=False)
            first = {m: {f: getattr(subs[m], f).grad for f in fields} for m in related}
            for s in subs:
                for p in s.parameters():
                    p.grad = None
            torch.autograd.backward([once_more["render"]], [upstream])
        for m in related:
            for f in fields:
                a, b = first[m][f], getattr(subs[m], f).grad
                floor = max(floor, float((a - b).double().norm() / b.double().norm().clamp_min(1e-300)))
        ok = ok and worst <= GRADIENT_AGREEMENT
        del again, once_more, first
        for s in subs:
            for p in s.parameters():
                p.grad = None
    return {"verified": bool(ok), "against": "one rgs_forward_geom / rgs_forward_raster" + (" / rgs_backward" if do_backward else "")
            + " call per submodel", "bit_for_bit": "instance counts, radii, colour, depth, alpha, n_contrib of every submodel"
            + (", composited image" if do_backward else ""), "submodels": len(related), "submodels_that_differ": mismatches,
            "worst_gradient_rel_l2": worst if do_backward else None, "gradient_rel_l2_allowed": GRADIENT_AGREEMENT if do_backward else None,
            # the same comparison between two runs of the per-submodel calls: what the order of the atomic adds alone does
            "gradient_rel_l2_of_a_repeat": floor if do_backward else None}


def cpu_render_baseline(subs, cam, rel, related, args):
    """The render (every related submodel's forward, then the compositing) on the CPU checker for a scene that lives
    on the device: one submodel is copied to the host at a time.  Bounded to about 25 s of wall time: if the submodels do
    not all fit, the figure is extrapolated from the share of the Gaussians that did, and says so."""
    from oracle import rgs_oracle as orc
    np32 = lambda t: np.ascontiguousarray(t.detach().cpu().numpy().astype(np.float32))
    threads = args.cpu_threads or min(16, orc.max_threads(), os.cpu_count() or 1)
    orc.set_threads(threads)
    order = sorted(related, key=lambda m: rel[m])
    total = sum(int(subs[m].means3D.shape[0]) for m in order)
    spent, seen, states = 0.0, 0, []
    try:
        for m in order:
            s = subs[m]
            arrays = [np32(t) for t in (s.means3D, s.opacity, s.shs, s.scales, s.rotations)]
            settings = orc.settings_from_camera(cam, s.range_low.cpu(), s.range_up.cpu(), torch.zeros(3))
            t0 = time.perf_counter()
            st = orc.forward(settings, arrays[0], arrays[1], shs=arrays[2], scales=arrays[3], rotations=arrays[4])
            spent += time.perf_counter() - t0
            states.append((st.color, st.depth, st.alpha))
            seen += arrays[0].shape[0]
            del arrays, st
            if spent > 25.0:
                break
        t0 = time.perf_counter()
        orc.composite_forward([c for c, _, _ in states], [d for _, d, _ in states], [a for _, _, a in states], np.zeros(3, np.float32))
        spent += time.perf_counter() - t0
    finally:
        orc.set_threads(1)
    whole = seen == total
    seconds = spent if whole else spent * total / max(seen, 1)
    return {"value": round(seconds * 1e3, 1), "unit": "ms/frame", "cores": threads, "kind": "port",
            "extrapolated": not whole,
            "sample": (f"the forward of {len(states)} of {len(order)} related submodels ({seen} of {total} Gaussians) and their "
                       f"compositing, {spent:.1f} s wall, C checker with OpenMP"
                       + ("" if whole else "; scaled by the share of the Gaussians")),
            "host_cpus": os.cpu_count()}


def cpu_baseline(scene, members, part, cam, rel, related, upstream, do_backward, args):
    """One full forward(+backward) of the same frame on the CPU checker, OpenMP over this
    host's cores.  Test infrastructure used as a measuring stick, never as the product path."""
    from oracle import rgs_oracle as orc
    oracle_settings = orc.settings_from_camera
    np32 = lambda t: np.ascontiguousarray(t.detach().cpu().numpy().astype(np.float32))
    threads = args.cpu_threads or min(16, orc.max_threads(), os.cpu_count() or 1)
    orc.set_threads(threads)
    order = sorted(related, key=lambda m: rel[m])
    bg = torch.zeros(3)
    xyz, opa, sc, rot, shs = (np32(scene[k]) for k in ("xyz", "opacity", "scales", "rotations", "shs"))
    if part is not None:
        lows, ups = part.box_low, part.box_up
    else:
        pad = 3.0 * float(scene["scales"].max()) + 1.0
        lows = [np32(scene["xyz"].min(dim=0).values - pad)]
        ups = [np32(scene["xyz"].max(dim=0).values + pad)]
    def iteration():
        t0 = time.perf_counter()
        states, sets = [], []
        for m in order:
            ids = members[m]
            s = oracle_settings(cam, torch.from_numpy(np.asarray(lows[m])), torch.from_numpy(np.asarray(ups[m])), bg)
            st = orc.forward(s, xyz[ids], opa[ids], shs=shs[ids], scales=sc[ids], rotations=rot[ids])
            states.append(st)
            sets.append(s)
        imgs = [st.color for st in states]
        deps = [st.depth for st in states]
        alps = [st.alpha for st in states]
        orc.composite_forward(imgs, deps, alps, np.zeros(3, np.float32))
        if do_backward:
            d_img, d_dep, d_alp = orc.composite_backward(imgs, deps, alps, np.zeros(3, np.float32), upstream)
            for k, st in enumerate(states):
                orc.backward(sets[k], st, d_img[k], d_dep[k], d_alp[k])
        return time.perf_counter() - t0

    times = [iteration()]
    # more iterations while they fit into about ten seconds of wall time; the median is reported
    while len(times) < 5 and sum(times) + times[0] < 10.0:
        times.append(iteration())
    dt = float(np.median(times))
    orc.set_threads(1)
    return {"value": round(1.0 / dt, 5), "unit": "it/s", "cores": threads, "kind": "port",
            "sample": f"{len(times)} full iteration(s) of the same frame, median {dt:.2f} s wall each "
                      f"({sum(times) * threads:.0f} core-seconds in all), C checker with OpenMP",
            "host_cpus": os.cpu_count()}


if __name__ == "__main__":
    main()
