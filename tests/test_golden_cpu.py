"""The committed vectors in tests/golden/ are reproduced by the CPU checker bit for bit
(integer stages) and to rounding (float stages): a change to the checker that alters any
result shows up here before it can silently move the target of the GPU parity tests."""
import os

import numpy as np

from helpers import ROOT, orc


def load_cases():
    z = np.load(os.path.join(ROOT, "tests", "golden", "half_gaussian_small.npz"))
    cases = {}
    for key in z.files:
        c, k = key.split("/", 1)
        cases.setdefault(c, {})[k] = z[key]
    return cases


def settings_of(c):
    W, H = (int(v) for v in c["size"])
    return orc.Settings(image_height=H, image_width=W, tanfovx=float(c["tanfov"][0]), tanfovy=float(c["tanfov"][1]),
                        bg=c["bg"], scale_modifier=1.0, viewmatrix=c["viewmatrix"], projmatrix=c["projmatrix"],
                        projmatrix_inv=c["projmatrix_inv"], range_low=c["range_low"], range_up=c["range_up"],
                        sh_degree=3, campos=c["campos"])


def test_checker_reproduces_golden_vectors():
    for name, c in load_cases().items():
        s = settings_of(c)
        st = orc.forward(s, c["xyz"], c["opacity"], shs=c["shs"], scales=c["scales"], rotations=c["rotations"])
        for k in ("radii", "tiles_touched", "keys", "point_list", "ranges", "n_contrib"):
            assert np.array_equal(getattr(st, k), c[k]), (name, k)
        for k in ("xy", "depths", "color", "depth", "alpha"):
            assert np.array_equal(getattr(st, k), c[k]), (name, k)
        g = orc.backward(s, st, c["g_color"], c["g_depth"], c["g_alpha"])
        for k, v in g.items():
            assert np.allclose(v, c["grad_" + k], rtol=1e-6, atol=1e-9), (name, k)
        assert (st.radii > 0).sum() > 100 and (st.radii == 0).sum() >= 20


def load_steps():
    return np.load(os.path.join(ROOT, "tests", "golden", "neighbouring_steps_small.npz"))


def test_checkers_of_the_neighbouring_steps_reproduce_their_golden_vectors():
    from oracle import sharing_oracle as so
    from oracle import training_oracle as to
    z = load_steps()
    low, up = z["share/box_low"], z["share/box_up"]
    lent = 0
    for s in range(3):
        for d in range(3):
            if s != d:
                rows = so.straddler_rows(z[f"share/xyz{s}"], z[f"share/scales{s}"], low[s], up[s], low[d], up[d])
                assert np.array_equal(rows, z[f"share/rows_{s}_{d}"]), (s, d)
                lent += len(rows)
    assert lent > 30 and len(z["share/rows_0_2"]) < len(z["share/rows_0_1"])
    loss, l1, ssim, grad = to.l1_ssim(z["loss/image"], z["loss/gt"], 0.2)
    assert np.allclose([loss, l1, ssim], z["loss/values"], rtol=0, atol=1e-12)
    assert np.allclose(grad, z["loss/grad"], rtol=1e-9, atol=1e-15)
    n = 4
    params = [z[f"adam/param{k}"] for k in range(n)]
    grads = [[z[f"adam/grad{t}_{k}"] for k in range(n)] for t in range(5)]
    after = to.adam_reference(params, list(z["adam/lrs"]), grads, eps=1e-15)
    for k in range(n):
        assert np.allclose(after[k], z[f"adam/after{k}"], rtol=1e-6, atol=1e-9)
        assert np.allclose(after[n + k], z[f"adam/exp_avg{k}"], rtol=1e-6, atol=1e-12)
        assert np.allclose(after[2 * n + k], z[f"adam/exp_avg_sq{k}"], rtol=1e-6, atol=1e-15)
