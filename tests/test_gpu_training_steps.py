"""The image loss and the Adam step on the GPU (rgs_l1_ssim_forward/backward, rgs_adam_step
through retinags_amd/loss.py and retinags_amd/optimizer.py) against the CPU checker.
Tolerances: loss values 2e-6 absolute (float32 sums of ~5e6 terms against float64), loss
gradient 1e-3 relative L2 (the gradient bar of the rasterizer), Adam 1e-6 relative per element
after several steps."""
import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import training_oracle as to

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _images(seed, C, H, W):
    rng = np.random.default_rng(seed)
    gt = rng.random((C, H, W)).astype(np.float32)
    image = np.clip(0.7 * gt + 0.2 * np.roll(gt, 2, axis=2) + 0.1 * rng.random((C, H, W)), 0, 1).astype(np.float32)
    return image, gt


@pytest.mark.parametrize("C,H,W", [(3, 64, 96), (3, 37, 45), (1, 16, 32), (3, 5, 7), (2, 131, 259)])
def test_loss_and_gradient_against_checker(C, H, W):
    from retinags_amd import loss as L
    image, gt = _images(C * 1000 + H, C, H, W)
    for lam in (0.2, 1.0, 0.0):
        want_loss, want_l1, want_ssim, want_grad = to.l1_ssim(image, gt, lam)
        x = torch.tensor(image, device=DEV, requires_grad=True)
        y = torch.tensor(gt, device=DEV)
        loss, l1 = L.l1_ssim_loss(x, y, lam)
        (loss * 3.0).backward()
        assert abs(float(loss.detach()) - want_loss) < 2e-6 and abs(float(l1) - want_l1) < 2e-6
        assert abs(float(L.ssim(x.detach(), y)) - want_ssim) < 2e-6
        assert abs(float(L.l1_loss(x.detach(), y)) - want_l1) < 2e-6
        assert rel_l2(x.grad.cpu().numpy(), 3.0 * want_grad) < 1e-3
    # identical images: SSIM exactly at its maximum, L1 zero, and a zero L1 gradient (sign(0) = 0)
    x = torch.tensor(gt, device=DEV, requires_grad=True)
    loss, l1 = L.l1_ssim_loss(x, torch.tensor(gt, device=DEV), 0.2)
    loss.backward()
    assert float(l1) == 0.0 and abs(float(loss.detach())) < 1e-6 and float(x.grad.abs().max()) < 1e-6


def test_loss_is_reproducible_and_batched_planes_are_independent():
    from retinags_amd import loss as L
    image, gt = _images(7, 3, 90, 130)
    x, y = torch.tensor(image, device=DEV), torch.tensor(gt, device=DEV)
    a = [float(L.l1_ssim_loss(x, y)[0]) for _ in range(3)]
    assert a[0] == a[1] == a[2]
    xb = torch.stack([x, x.flip(-1)]).requires_grad_(True)
    yb = torch.stack([y, y.flip(-1)])
    lb, _ = L.l1_ssim_loss(xb, yb)
    lb.backward()
    assert abs(float(lb.detach()) - a[0]) < 1e-6
    assert torch.allclose(xb.grad[0], xb.grad[1].flip(-1), atol=1e-9)


def test_loss_rejects_host_tensors_and_shape_mismatch():
    from retinags_amd import loss as L
    with pytest.raises(RuntimeError):
        L.l1_ssim_loss(torch.zeros(3, 8, 8), torch.zeros(3, 8, 8))
    with pytest.raises(RuntimeError):
        L.l1_ssim_loss(torch.zeros(3, 8, 8, device=DEV), torch.zeros(3, 8, 9, device=DEV))


def test_adam_against_torch_on_the_cpu():
    """The reference's parameter groups (scene/gaussian_nn_module.py:433-441) at a small size,
    five steps, against torch.optim.Adam on the CPU; includes the group with learning rate 0."""
    from retinags_amd.optimizer import Adam
    n = 1237
    rng = np.random.default_rng(5)
    shapes = [(n, 3), (n, 1, 3), (n, 15, 3), (n, 1), (n, 1), (n, 3), (n, 4)]
    lrs = [0.00016, 0.0025, 0.0025 / 20.0, 0.05, 0.0, 0.005, 0.001]
    params = [rng.normal(size=s).astype(np.float32) for s in shapes]
    steps = [[(rng.normal(size=s) * 10.0 ** rng.uniform(-6, 0)).astype(np.float32) for s in shapes] for _ in range(5)]
    steps[2][3][:] = 0.0                                  # a step without gradient signal for one group
    want = to.adam_reference(params, lrs, steps, eps=1e-15)
    ps = [torch.nn.Parameter(torch.tensor(p, device=DEV)) for p in params]
    opt = Adam([{"params": [p], "lr": lr, "name": str(k)} for k, (p, lr) in enumerate(zip(ps, lrs))], lr=0.0, eps=1e-15)
    for grads in steps:
        for p, g in zip(ps, grads):
            p.grad = torch.tensor(g, device=DEV)
        opt.step()
        opt.zero_grad(set_to_none=True)
    got = [p.detach().cpu().numpy() for p in ps] + [opt.state[p]["exp_avg"].cpu().numpy() for p in ps] + \
          [opt.state[p]["exp_avg_sq"].cpu().numpy() for p in ps]
    for k, (g, w) in enumerate(zip(got, want)):
        assert np.abs(g - w).max() <= 1e-6 * max(1.0, np.abs(w).max()), k
        assert rel_l2(g, w) < 1e-6, k
    assert np.array_equal(got[4], params[4])              # learning rate 0 leaves the tensor as it was
    assert all(opt.state[p]["step"] == 5 for p in ps)


def test_adam_handles_odd_sizes_and_many_tensors():
    from retinags_amd.optimizer import Adam
    rng = np.random.default_rng(6)
    sizes = [1, 2, 3, 5, 4095, 4096, 4097, 8191] + [17] * 20      # more than one launch's worth of tensors
    params = [rng.normal(size=s).astype(np.float32) for s in sizes]
    grads = [[rng.normal(size=s).astype(np.float32) for s in sizes] for _ in range(2)]
    want = to.adam_reference(params, [0.01] * len(sizes), grads, eps=1e-8)
    base = torch.zeros(sum(sizes) + 64, device=DEV)
    ps, at = [], 1                                                   # start off a 16-byte boundary
    for p in params:
        view = base[at:at + p.size]
        view.copy_(torch.tensor(p))
        ps.append(torch.nn.Parameter(view))
        at += p.size
    opt = Adam(ps, lr=0.01, eps=1e-8)
    for g in grads:
        for p, gi in zip(ps, g):
            p.grad = torch.tensor(gi, device=DEV)
        opt.step()
    for k, p in enumerate(ps):
        assert np.abs(p.detach().cpu().numpy() - want[k]).max() <= 2e-6, k
    assert float(base[0]) == 0.0 and float(base[at:].abs().max()) == 0.0     # nothing written outside the tensors


def test_golden_vectors_of_the_neighbouring_steps():
    """The committed fixtures (tests/golden/neighbouring_steps_small.npz) through the C ABI: row lists
    bit for bit, loss and gradient, five Adam steps."""
    import os
    from helpers import ROOT
    from retinags_amd import loss as L, sharing
    from retinags_amd.optimizer import Adam
    z = np.load(os.path.join(ROOT, "tests", "golden", "neighbouring_steps_small.npz"))
    dev = lambda a: torch.tensor(a, device=DEV)
    models = []
    for m in range(3):
        xyz = dev(z[f"share/xyz{m}"])
        n = xyz.shape[0]
        models.append(sharing.SharedGSInfo(xyz, torch.zeros_like(xyz), torch.zeros(n, 1, device=DEV), dev(z[f"share/scales{m}"]),
                                           torch.zeros(n, 4, device=DEV), torch.zeros(n, 16, 3, device=DEV)))
    table = sharing.select_straddlers(models, z["share/box_low"], z["share/box_up"])
    for s in range(3):
        for d in range(3):
            if s != d:
                want = z[f"share/rows_{s}_{d}"]
                assert table.counts[s, d] == len(want)
                if len(want):
                    assert np.array_equal(table.rows[(s, d)].cpu().numpy().astype(np.int64), want)
    x = dev(z["loss/image"]).requires_grad_(True)
    loss, l1 = L.l1_ssim_loss(x, dev(z["loss/gt"]), 0.2)
    loss.backward()
    assert abs(float(loss.detach()) - z["loss/values"][0]) < 2e-6 and abs(float(l1) - z["loss/values"][1]) < 2e-6
    assert rel_l2(x.grad.cpu().numpy(), z["loss/grad"]) < 1e-3
    ps = [torch.nn.Parameter(dev(z[f"adam/param{k}"])) for k in range(4)]
    opt = Adam([{"params": [p], "lr": float(lr)} for p, lr in zip(ps, z["adam/lrs"])], lr=0.0, eps=1e-15)
    for t in range(5):
        for k, p in enumerate(ps):
            p.grad = dev(z[f"adam/grad{t}_{k}"])
        opt.step()
    for k, p in enumerate(ps):
        assert rel_l2(p.detach().cpu().numpy(), z[f"adam/after{k}"]) < 1e-6
        assert rel_l2(opt.state[p]["exp_avg_sq"].cpu().numpy(), z[f"adam/exp_avg_sq{k}"]) < 1e-6


def test_activation_and_its_backward_against_the_tensor_expressions():
    """rgs_activate_forward / rgs_activate_backward against exp, sigmoid, normalize and cat with autograd
    (scene/gaussian_nn_module.py:373-394), incl. a zero quaternion, rows behind for appending, and
    outputs without a gradient."""
    from retinags_amd.activation import activate_gaussians
    rng = np.random.default_rng(14)
    for n, rest, spare in ((1003, 15, 0), (257, 15, 64), (64, 0, 8), (5, 8, 0)):
        dc = rng.normal(size=(n, 1, 3)).astype(np.float32)
        fr = rng.normal(size=(n, rest, 3)).astype(np.float32)
        sc = rng.normal(-4, 1, size=(n, 3)).astype(np.float32)
        rot = rng.normal(size=(n, 4)).astype(np.float32)
        rot[0] = 0.0                                   # normalize leaves a zero vector at zero
        op = rng.normal(0, 2, size=(n, 1)).astype(np.float32)
        g = [rng.normal(size=s).astype(np.float32) for s in ((n, 1 + rest, 3), (n, 3), (n, 4), (n, 1))]
        want, want_grads = to.activate_reference(dc, fr, sc, rot, op, g)
        leaves = [torch.tensor(a, device=DEV, requires_grad=True) for a in (dc, fr, sc, rot, op)]
        xyz = torch.zeros(n, 3, device=DEV)
        info = activate_gaussians(xyz, *leaves, spare_rows=spare)
        got = [info.shs, info.scales, info.rotations, info.opacity]
        assert info.means3D is xyz and float(info.means2D.abs().sum()) == 0.0
        assert np.array_equal(got[0].detach().cpu().numpy(), want[0])
        for a, b in zip(got[1:], want[1:]):
            assert np.abs(a.detach().cpu().numpy() - b).max() <= 2e-6 * max(1.0, np.abs(b).max())
        if spare:
            assert all(t.untyped_storage().nbytes() >= (n + spare) * t[0].numel() * 4 for t in got)
        torch.autograd.backward(got, [torch.tensor(x, device=DEV) for x in g])
        for leaf, w in zip(leaves, want_grads):
            assert rel_l2(leaf.grad.cpu().numpy()[1:], w[1:]) < 1e-5      # row 0: the zero quaternion
        assert torch.isfinite(leaves[3].grad[0]).all()
    # only some outputs take part in the loss
    leaves = [torch.tensor(a, device=DEV, requires_grad=True) for a in (dc, fr, sc, rot, op)]
    info = activate_gaussians(torch.zeros(n, 3, device=DEV), *leaves)
    info.scales.sum().backward()
    assert leaves[0].grad is None and leaves[3].grad is None
    assert torch.allclose(leaves[2].grad, torch.exp(leaves[2].detach()), rtol=1e-5)
