"""CPU restatement of the image loss of a training iteration and a wrapper of the optimiser the
reference uses, for the tests of the GPU loss and Adam kernels.

TEST INFRASTRUCTURE ONLY.  Tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package must not.

``l1_ssim`` follows utils/loss_utils.py:17-63 and loss_local
(parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:449-450) with torch's CPU
convolution in float64; its gradient is autograd's.  Pinned by tests/test_training_cpu.py:
SSIM against an implementation built on scipy.ndimage's separable Gaussian filter, SSIM(x, x) = 1,
the gradient against central differences.  ``adam_reference`` IS torch.optim.Adam (the reference's
optimiser, scene/gaussian_nn_module.py:443) run on the CPU, so it needs no pin; ``activate_reference``
likewise is the reference's own four tensor expressions with autograd.
"""
from __future__ import annotations

from math import exp
from typing import List, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F


def gaussian_window(window_size: int = 11, sigma: float = 1.5) -> torch.Tensor:
    """utils/loss_utils.py:23-25: float32 values, normalised in float32."""
    g = torch.Tensor([exp(-(x - window_size // 2) ** 2 / float(2 * sigma ** 2)) for x in range(window_size)])
    return g / g.sum()


def ssim_map(img1: torch.Tensor, img2: torch.Tensor, window_size: int = 11) -> torch.Tensor:
    """utils/loss_utils.py:27-58 for (C,H,W) inputs, evaluated in the inputs' dtype (use float64)."""
    channel = img1.size(-3)
    one = gaussian_window(window_size).unsqueeze(1)
    window = one.mm(one.t()).float().unsqueeze(0).unsqueeze(0).expand(channel, 1, window_size, window_size).contiguous()
    window = window.to(img1.dtype)
    a, b = img1.unsqueeze(0), img2.unsqueeze(0)
    conv = lambda t: F.conv2d(t, window, padding=window_size // 2, groups=channel)
    mu1, mu2 = conv(a), conv(b)
    mu1_sq, mu2_sq, mu1_mu2 = mu1.pow(2), mu2.pow(2), mu1 * mu2
    sigma1_sq = conv(a * a) - mu1_sq
    sigma2_sq = conv(b * b) - mu2_sq
    sigma12 = conv(a * b) - mu1_mu2
    C1, C2 = 0.01 ** 2, 0.03 ** 2
    return (((2 * mu1_mu2 + C1) * (2 * sigma12 + C2)) / ((mu1_sq + mu2_sq + C1) * (sigma1_sq + sigma2_sq + C2)))[0]


def l1_ssim(image: np.ndarray, gt: np.ndarray, lambda_dssim: float = 0.2, want_grad: bool = True):
    """Returns (loss, l1, ssim, d loss / d image) as float64 numpy values."""
    x = torch.tensor(np.asarray(image), dtype=torch.float64, requires_grad=want_grad)
    y = torch.tensor(np.asarray(gt), dtype=torch.float64)
    l1 = torch.abs(x - y).mean()
    s = ssim_map(x, y).mean()
    loss = (1.0 - lambda_dssim) * l1 + lambda_dssim * (1.0 - s)
    grad = None
    if want_grad:
        loss.backward()
        grad = x.grad.numpy()
    return float(loss.detach()), float(l1.detach()), float(s.detach()), grad


def activate_reference(features_dc, features_rest, scaling, rotation, opacity, grads=None):
    """The reference's activations as it writes them (scene/gaussian_nn_module.py:304-312, 373-394):
    torch.exp, torch.sigmoid, torch.nn.functional.normalize, torch.cat, on the CPU in float32.
    Returns (shs, scales, rotations, opacities) and, with `grads` (gradients of those four), the
    gradients of the five inputs by autograd."""
    leaves = [torch.tensor(np.asarray(a, dtype=np.float32), requires_grad=grads is not None)
              for a in (features_dc, features_rest, scaling, rotation, opacity)]
    dc, rest, sc, rot, op = leaves
    outs = (torch.cat((dc, rest), dim=1), torch.exp(sc), F.normalize(rot), torch.sigmoid(op))
    values = [o.detach().numpy().copy() for o in outs]
    if grads is None:
        return values, None
    torch.autograd.backward(outs, [torch.tensor(np.asarray(g, dtype=np.float32)) for g in grads])
    return values, [t.grad.numpy().copy() for t in leaves]


def adam_reference(params: Sequence[np.ndarray], lrs: Sequence[float], grads_per_step: Sequence[Sequence[np.ndarray]],
                   betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-15) -> List[np.ndarray]:
    """torch.optim.Adam on the CPU in float32: one parameter group per tensor, one step per entry of
    grads_per_step.  Returns the parameters after the last step."""
    ps = [torch.nn.Parameter(torch.tensor(np.asarray(p, dtype=np.float32))) for p in params]
    opt = torch.optim.Adam([{"params": [p], "lr": lr} for p, lr in zip(ps, lrs)], lr=0.0, betas=betas, eps=eps)
    for grads in grads_per_step:
        for p, g in zip(ps, grads):
            p.grad = torch.tensor(np.asarray(g, dtype=np.float32))
        opt.step()
    return [p.detach().numpy().copy() for p in ps] + [opt.state[p]["exp_avg"].numpy().copy() for p in ps] + \
           [opt.state[p]["exp_avg_sq"].numpy().copy() for p in ps]
