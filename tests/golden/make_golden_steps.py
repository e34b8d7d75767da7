"""Writes tests/golden/neighbouring_steps_small.npz: seeded inputs and the CPU checkers' outputs for
the steps either side of the rasterizer (boundary-straddler row lists, L1 + SSIM loss with its
gradient, five Adam steps).  The reference holds no fixtures for these either; the vectors come from
oracle/sharing_oracle.py and oracle/training_oracle.py, which tests/test_scheduling_cpu.py and
tests/test_training_cpu.py pin.  Run: python tests/golden/make_golden_steps.py"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import sharing_oracle as so  # noqa: E402
from oracle import training_oracle as to  # noqa: E402


def main():
    rng = np.random.default_rng(2024)
    out = {}
    # three submodels side by side along x, Gaussians inside their own boxes, some reaching out
    low = np.float32([[-3, -1, -1], [-1, -1, -1], [1, -1, -1]])
    up = np.float32([[-1, 1, 1], [1, 1, 1], [3, 1, 1]])
    out["share/box_low"], out["share/box_up"] = low, up
    for m in range(3):
        n = 400 + 50 * m
        xyz = rng.uniform(low[m] + 0.001, up[m] - 0.001, (n, 3)).astype(np.float32)
        scales = np.exp(rng.normal(-3.2, 0.9, (n, 3))).astype(np.float32)
        out[f"share/xyz{m}"], out[f"share/scales{m}"] = xyz, scales
    for s in range(3):
        for d in range(3):
            if s != d:
                out[f"share/rows_{s}_{d}"] = so.straddler_rows(out[f"share/xyz{s}"], out[f"share/scales{s}"], low[s], up[s],
                                                               low[d], up[d]).astype(np.int64)
    # loss
    gt = rng.random((3, 41, 53)).astype(np.float32)
    image = np.clip(0.7 * gt + 0.2 * np.roll(gt, 3, axis=1) + 0.1 * rng.random(gt.shape), 0, 1).astype(np.float32)
    loss, l1, ssim, grad = to.l1_ssim(image, gt, 0.2)
    out["loss/image"], out["loss/gt"] = image, gt
    out["loss/values"] = np.float64([loss, l1, ssim])
    out["loss/grad"] = grad
    # Adam
    shapes = [(97, 3), (97, 15, 3), (97, 1), (97, 4)]
    lrs = [0.00016, 0.000125, 0.05, 0.001]
    params = [rng.normal(size=s).astype(np.float32) for s in shapes]
    grads = [[(rng.normal(size=s) * 1e-3).astype(np.float32) for s in shapes] for _ in range(5)]
    after = to.adam_reference(params, lrs, grads, eps=1e-15)
    out["adam/lrs"] = np.float64(lrs)
    for k, p in enumerate(params):
        out[f"adam/param{k}"] = p
        out[f"adam/after{k}"] = after[k]
        out[f"adam/exp_avg{k}"] = after[len(params) + k]
        out[f"adam/exp_avg_sq{k}"] = after[2 * len(params) + k]
        for t in range(5):
            out[f"adam/grad{t}_{k}"] = grads[t][k]
    path = os.path.join(HERE, "neighbouring_steps_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
