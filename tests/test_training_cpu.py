"""Pins of the CPU checker for the image loss (oracle/training_oracle.py): SSIM against an
implementation that shares nothing with it but the definition, and the gradient against central
differences."""
import numpy as np
import pytest
import torch

from oracle import training_oracle as to


def _images(seed, C=3, H=37, W=45):
    rng = np.random.default_rng(seed)
    gt = rng.random((C, H, W))
    # a smoothed, shifted version of the ground truth plus noise: SSIM well inside (0, 1)
    image = np.clip(0.7 * gt + 0.2 * np.roll(gt, 2, axis=2) + 0.1 * rng.random((C, H, W)), 0, 1)
    return image, gt


def _ssim_by_ndimage(img1, img2):
    """Windowed means by scipy's separable Gaussian filter (radius 5 = 11 taps, zero outside)."""
    from scipy.ndimage import gaussian_filter
    blur = lambda a: np.stack([gaussian_filter(p, sigma=1.5, radius=5, mode="constant", cval=0.0) for p in a])
    mu1, mu2 = blur(img1), blur(img2)
    s11 = blur(img1 * img1) - mu1 ** 2
    s22 = blur(img2 * img2) - mu2 ** 2
    s12 = blur(img1 * img2) - mu1 * mu2
    C1, C2 = 1e-4, 9e-4
    return ((2 * mu1 * mu2 + C1) * (2 * s12 + C2)) / ((mu1 ** 2 + mu2 ** 2 + C1) * (s11 + s22 + C2))


def test_ssim_of_the_checker_against_scipy_filters():
    """Pins ssim_map (utils/loss_utils.py:39-63)."""
    image, gt = _images(1)
    got = to.ssim_map(torch.tensor(image), torch.tensor(gt)).numpy()
    want = _ssim_by_ndimage(image, gt)
    assert got.shape == want.shape
    # the checker's window is rounded to float32 as the reference's is; scipy's is float64
    assert np.abs(got - want).max() < 5e-6
    assert 0.2 < got.mean() < 0.95


def test_ssim_closed_cases():
    image, _ = _images(2)
    same = to.ssim_map(torch.tensor(image), torch.tensor(image)).numpy()
    assert np.abs(same - 1.0).max() < 1e-12
    # constant images a and b: every windowed variance is zero inside the image's interior
    a, b = np.full((1, 30, 30), 0.25), np.full((1, 30, 30), 0.75)
    inner = to.ssim_map(torch.tensor(a), torch.tensor(b)).numpy()[0, 5:-5, 5:-5]
    one = to.gaussian_window().unsqueeze(1)
    w = float(one.mm(one.t()).double().sum())    # the float32 window does not sum to exactly 1
    m1, m2 = 0.25 * w, 0.75 * w
    s11, s22, s12 = 0.0625 * w - m1 * m1, 0.5625 * w - m2 * m2, 0.1875 * w - m1 * m2
    expect = (2 * m1 * m2 + 1e-4) * (2 * s12 + 9e-4) / ((m1 * m1 + m2 * m2 + 1e-4) * (s11 + s22 + 9e-4))
    assert np.abs(inner - expect).max() < 1e-9
    loss, l1, s, _ = to.l1_ssim(a, b, 0.2, want_grad=False)
    assert abs(l1 - 0.5) < 1e-12 and abs(loss - (0.8 * 0.5 + 0.2 * (1 - s))) < 1e-12


def test_loss_gradient_of_the_checker_against_central_differences():
    image, gt = _images(3, C=2, H=19, W=23)
    loss, _, _, grad = to.l1_ssim(image, gt, 0.2)
    rng = np.random.default_rng(0)
    for _ in range(25):
        c, i, j = rng.integers(0, 2), rng.integers(0, 19), rng.integers(0, 23)
        h = 1e-6
        up, down = image.copy(), image.copy()
        up[c, i, j] += h
        down[c, i, j] -= h
        fd = (to.l1_ssim(up, gt, 0.2, want_grad=False)[0] - to.l1_ssim(down, gt, 0.2, want_grad=False)[0]) / (2 * h)
        assert abs(fd - grad[c, i, j]) < 1e-8 + 1e-5 * abs(fd)
