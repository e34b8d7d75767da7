"""Stand-alone binning primitives and the compositor of the HIP library, through the C ABI,
against numpy / the CPU checker.  Integer results are bit-exact."""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import np32, orc, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def gpu_sort_pairs(keys, vals, end_bit):
    from retinags_amd import _capi
    n = keys.shape[0]
    k_in = torch.from_numpy(keys.view(np.int64).copy()).to(DEV)
    v_in = torch.from_numpy(vals.view(np.int32).copy()).to(DEV)
    k_out, v_out = torch.empty_like(k_in), torch.empty_like(v_in)
    temp = torch.empty(max(_capi.lib.rgs_sort_temp_bytes(n), 4), dtype=torch.uint8, device=DEV)
    _capi.check(_capi.lib.rgs_sort_pairs(_capi.ptr(k_in), _capi.ptr(k_out), _capi.ptr(v_in), _capi.ptr(v_out), n,
                                         end_bit, _capi.ptr(temp), _stream()))
    torch.cuda.synchronize()
    return k_out.cpu().numpy().view(np.uint64), v_out.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("n,end_bit", [(0, 45), (1, 45), (63, 43), (4095, 43), (4096, 45), (4097, 45), (20001, 49),
                                        (300000, 45), (1 << 20, 43), (100000, 64), (50000, 8), (50000, 1), (77777, 33)])
def test_sort_pairs_matches_numpy_stable_sort(n, end_bit):
    g = np.random.default_rng(n + end_bit)
    keys = g.integers(0, 2 ** 63, size=n, dtype=np.uint64) * np.uint64(2) + g.integers(0, 2, size=n, dtype=np.uint64)
    if n:
        keys[: n // 3] &= np.uint64(0xFFFFF)                    # many equal compared bits -> stability matters
        keys[n // 3: n // 2] = keys[n // 3]                      # long run of identical keys
    vals = g.integers(0, 2 ** 32, size=n, dtype=np.uint32)
    ko, vo = gpu_sort_pairs(keys, vals, end_bit)
    mask = np.uint64((1 << end_bit) - 1) if end_bit < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
    order = np.argsort(keys & mask, kind="stable")
    assert np.array_equal(ko, keys[order])
    assert np.array_equal(vo, vals[order])


def test_sort_pairs_tile_depth_keys_like_the_rasterizer():
    """Keys shaped like the rasterizer's: 13 bits of tile id over positive float depth bits."""
    g = np.random.default_rng(5)
    n = 2_000_003
    tiles = g.integers(0, 6500, size=n, dtype=np.uint64)
    depth = g.uniform(0.2, 30.0, size=n).astype(np.float32).view(np.uint32).astype(np.uint64)
    keys = (tiles << np.uint64(32)) | depth
    vals = np.arange(n, dtype=np.uint32)
    ko, vo = gpu_sort_pairs(keys, vals, 45)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(ko, keys[order]) and np.array_equal(vo, vals[order])


@pytest.mark.parametrize("n", [0, 1, 255, 256, 257, 65536, 1_000_001])
def test_inclusive_sum_matches_cumsum(n):
    from retinags_amd import _capi
    g = np.random.default_rng(n)
    x = g.integers(0, 50, size=n, dtype=np.uint32)
    if n > 10:
        x[3] = 4_000_000_000  # wraps like the reference's uint32 scan
    xi = torch.from_numpy(x.view(np.int32).copy()).to(DEV)
    out = torch.empty_like(xi)
    temp = torch.empty(max(_capi.lib.rgs_scan_temp_bytes(n), 4), dtype=torch.uint8, device=DEV)
    _capi.check(_capi.lib.rgs_inclusive_sum(_capi.ptr(xi), _capi.ptr(out), n, _capi.ptr(temp), _stream()))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), np.cumsum(x.astype(np.uint64)).astype(np.uint32))
    assert np.array_equal(out.cpu().numpy().view(np.uint32), orc.inclusive_sum(x))


@pytest.mark.parametrize("K,H,W,with_bg", [(1, 17, 23, True), (4, 259, 400, True), (16, 64, 64, False), (33, 40, 56, True),
                                            (64, 16, 16, True), (70, 24, 24, True)])
def test_compositor_forward_and_backward(K, H, W, with_bg):
    from retinags_amd import composite_partial_images
    g = torch.Generator().manual_seed(K * 1000 + H)
    imgs = [torch.rand(3, H, W, generator=g) for _ in range(K)]
    deps = [torch.rand(1, H, W, generator=g) * 5 for _ in range(K)]
    # More than 64 layers are folded in groups through (1 - transmittance), which keeps
    # transmittances only down to float32 resolution; thin layers keep them well above it.
    alps = [torch.rand(1, H, W, generator=g) * (0.1 if K > 64 else 1.0) for _ in range(K)]
    if K <= 64:
        alps[0][0, 0, 0] = 1.0
    bg = torch.tensor([0.25, 0.5, 0.75]) if with_bg else None
    gi, gd, ga = torch.randn(3, H, W, generator=g), torch.randn(1, H, W, generator=g), torch.randn(1, H, W, generator=g)
    bg_np = np32(bg) if with_bg else np.zeros(3, np.float32)
    want = orc.composite_forward([np32(t) for t in imgs], [np32(t) for t in deps], [np32(t) for t in alps], bg_np)
    wdi, wdd, wda = orc.composite_backward([np32(t) for t in imgs], [np32(t) for t in deps], [np32(t) for t in alps],
                                           bg_np, np32(gi), np32(gd), np32(ga))
    leaf = lambda ts: [t.to(DEV).requires_grad_(True) for t in ts]
    li, ld, la = leaf(imgs), leaf(deps), leaf(alps)
    img, dep, alp = composite_partial_images(li, ld, la, None if bg is None else bg.to(DEV))
    torch.autograd.backward([img, dep, alp], [gi.to(DEV), gd.to(DEV), ga.to(DEV)])
    torch.cuda.synchronize()
    for got, w in zip((img, dep, alp), want):
        assert np.abs(got.detach().cpu().numpy() - w).max() <= 1e-4 * max(1.0, float(np.abs(w).max()))
    for k in range(K):
        assert rel_l2(li[k].grad.cpu().numpy(), wdi[k]) <= 1e-4
        assert rel_l2(ld[k].grad.cpu().numpy(), wdd[k]) <= 1e-4
        assert rel_l2(la[k].grad.cpu().numpy(), wda[k]) <= 1e-4


def test_compositor_colour_only_gradient_and_ordering_rule():
    """blender_render_result composites by ascending relation value and skips negatives."""
    from retinags_amd import blender_render_result
    g = torch.Generator().manual_seed(3)
    H, W = 20, 30
    res = {m: {"render": torch.rand(3, H, W, generator=g).to(DEV).requires_grad_(True),
               "depth": torch.rand(1, H, W, generator=g).to(DEV), "alpha": torch.rand(1, H, W, generator=g).to(DEV)}
           for m in (0, 1, 2)}
    rel = np.array([2, -1, 0, 1])
    res3 = {"render": torch.rand(3, H, W, generator=g).to(DEV), "depth": torch.rand(1, H, W, generator=g).to(DEV),
            "alpha": torch.rand(1, H, W, generator=g).to(DEV)}
    pool = {0: res[0], 2: res[2], 3: res3}
    bg = torch.tensor([0.1, 0.2, 0.3], device=DEV)
    out = blender_render_result(pool, rel, bg)
    order = [2, 3, 0]
    want = orc.composite_forward([np32(pool[m]["render"]) for m in order], [np32(pool[m]["depth"]) for m in order],
                                 [np32(pool[m]["alpha"]) for m in order], np32(bg))
    assert np.abs(out["render"].detach().cpu().numpy() - want[0]).max() <= 1e-5
    assert np.abs(out["alpha"].detach().cpu().numpy() - want[2]).max() <= 1e-5
    out["render"].sum().backward()
    assert res[0]["render"].grad is not None and res[1]["render"].grad is None
    with pytest.raises(RuntimeError, match="NUM_RELATED"):
        blender_render_result({0: res[0]}, rel, bg)
