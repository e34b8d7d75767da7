"""The scheduler routines either side of the rasterizer, on the CPU: which submodels a camera
sees and in which order (retinags_amd/harness/partition.py against oracle/sharing_oracle.py),
and what pins that checker: linear programming for the hull test, pairwise split-plane
constraints for the order, a scalar loop for the straddler selection."""
import math

import numpy as np
import pytest
import torch

from helpers import scenes
from oracle import sharing_oracle as so
from retinags_amd.harness import partition


def random_camera(rng, width=160, height=100, look_near=None):
    eye = rng.uniform(-6, 6, 3)
    target = eye + rng.normal(size=3) if look_near is None else np.asarray(look_near) + rng.normal(size=3) * 2.0
    up = rng.normal(size=3)
    return scenes.look_at_camera(eye, target, up, width, height, float(rng.uniform(30, 100)))


def random_box(rng):
    c = rng.uniform(-6, 6, 3)
    h = np.exp(rng.uniform(-2.5, 1.5, 3))
    return (c - h).astype(np.float32), (c + h).astype(np.float32)


def signed_gap(box_vs, frustum_vs):
    """Independent of any hull: the two bodies share a point iff some convex combination of the
    box's vertices equals one of the frustum's.  Solved as a linear program that also reports
    how far the bodies are from the other answer: minimise t such that the combinations differ by
    at most t in every coordinate."""
    from scipy.optimize import linprog
    nb, nf = len(box_vs), len(frustum_vs)
    # variables: lambda (nb), mu (nf), t
    c = np.zeros(nb + nf + 1)
    c[-1] = 1.0
    D = np.concatenate((box_vs.T, -frustum_vs.T), axis=1)            # (3, nb+nf)
    A_ub = np.concatenate((np.concatenate((D, -np.ones((3, 1))), axis=1),
                           np.concatenate((-D, -np.ones((3, 1))), axis=1)), axis=0)
    b_ub = np.zeros(6)
    A_eq = np.zeros((2, nb + nf + 1))
    A_eq[0, :nb] = 1.0
    A_eq[1, nb:nb + nf] = 1.0
    res = linprog(c, A_ub=A_ub, b_ub=b_ub, A_eq=A_eq, b_eq=np.ones(2),
                  bounds=[(0, None)] * (nb + nf) + [(0, None)], method="highs")
    assert res.status == 0
    return res.x[-1]


def test_hull_test_of_the_checker_against_linear_programming():
    """Pins is_overlapping_spacebox_view (parallel_utils/grid_utils/utils.py:115-137)."""
    rng = np.random.default_rng(11)
    seen = {True: 0, False: 0}
    for _ in range(150):
        low, up = random_box(rng)
        cam = random_camera(rng, look_near=(low + up) / 2 if rng.random() < 0.5 else None)
        wvt = cam.world_view_transform.numpy()
        z_far = float(rng.choice([8.0, 1000.0]))
        box = so.box_in_view_space(low, up, wvt).astype(np.float64)
        fr = so.frustum_vertices(cam.FoVx, cam.FoVy, 0.01, z_far).astype(np.float64)
        gap = signed_gap(box, fr)
        got = so.is_overlapping_spacebox_view(low, up, wvt, cam.FoVx, cam.FoVy, 0.01, z_far)
        if gap > 1e-6:
            assert not got
        elif gap < 1e-9:          # between the two, a contact within rounding may go either way
            assert got
        seen[got] += 1
    assert seen[True] > 20 and seen[False] > 20


def test_hull_test_closed_cases():
    cam = scenes.look_at_camera((0, 0, 0), (0, 0, 1), (0, -1, 0), 200, 100, 90.0)   # looks down +z, tan x = 1
    wvt = cam.world_view_transform.numpy()
    tany = math.tan(cam.FoVy / 2)
    call = lambda lo, hi, **kw: so.is_overlapping_spacebox_view(np.float32(lo), np.float32(hi), wvt, cam.FoVx, cam.FoVy, **kw)
    assert call((-1, -1, 2), (1, 1, 3))                       # dead ahead
    assert not call((-1, -1, -3), (1, 1, -2))                 # behind
    assert not call((5.5, -1, 2), (7, 1, 5))                  # x > z everywhere
    assert call((4.5, -1, 2), (7, 1, 5))                      # reaches x < z at z = 5
    assert not call((-1, -1, 12), (1, 1, 13), z_far=10.0)     # beyond the far plane
    assert call((-1, -1, 9), (1, 1, 13), z_far=10.0)
    assert not call((-0.1, 3 * tany + 0.2, 2), (0.1, 3 * tany + 1, 3))   # below the lower side plane
    assert call((-50, -50, -50), (50, 50, 50))                # camera inside the box
    # a box that passes between camera and a side edge: no vertex of either inside the other
    assert call((-30, -0.05, 4), (30, 0.05, 4.1))


def test_separating_axes_agree_with_the_checker():
    """boxes_overlap_view against the reference's hull predicate on random boxes and cameras."""
    rng = np.random.default_rng(5)
    disagreements, n_true = 0, 0
    for _ in range(60):
        boxes = [random_box(rng) for _ in range(12)]
        cam = random_camera(rng, look_near=(boxes[0][0] + boxes[0][1]) / 2 if rng.random() < 0.6 else None)
        low = np.stack([b[0] for b in boxes])
        up = np.stack([b[1] for b in boxes])
        z_far = float(rng.choice([6.0, 1000.0]))
        got = partition.boxes_overlap_view(low, up, cam, 0.01, z_far)
        wvt = cam.world_view_transform.numpy()
        for k in range(len(boxes)):
            want = so.is_overlapping_spacebox_view(low[k], up[k], wvt, cam.FoVx, cam.FoVy, 0.01, z_far)
            n_true += want
            if want != bool(got[k]):
                # only a contact within rounding may be seen differently
                box = so.box_in_view_space(low[k], up[k], wvt).astype(np.float64)
                fr = so.frustum_vertices(cam.FoVx, cam.FoVy, 0.01, z_far).astype(np.float64)
                assert signed_gap(box, fr) < 1e-5
                disagreements += 1
    assert disagreements <= 2 and 100 < n_true < 620


def test_frustum_vertices_match_the_checker():
    cam = scenes.look_at_camera((1, 2, 3), (0, 0, 0), (0, 0, 1), 320, 200, 70.0)
    for near, far in ((None, None), (0.001, 50.0), (0.5, 1e9)):
        a = partition.view_frustum_vertices(cam, near, far)
        b = so.frustum_vertices(cam.FoVx, cam.FoVy, near, far)
        assert a.dtype == np.float32 and np.array_equal(a, b)


def _splits_of(part):
    out = {}
    for path, node in part.nodes.items():
        if node.is_leaf or node.split_position is None:
            continue
        d = node.split_dim
        out[path] = (d, node.split_position * part.grid.voxel[d] + part.grid.low[d])
    return out


def test_order_of_the_checker_respects_every_split_plane():
    """Pins relation_vector (scene_utils.py:220-264): for two leaves that part ways at an inner
    node, the one on the camera's side of that node's split plane is composited first."""
    scene, _, _ = scenes.make_config("C1", shrink=400)
    part = partition.partition_scene(scene["xyz"], scene["scales"], 3)
    paths = [l.path for l in part.leaves]
    splits = _splits_of(part)
    rng = np.random.default_rng(2)
    for _ in range(20):
        center = rng.uniform(-12, 12, 3)
        rel = so.relation_vector(center, paths, splits, [True] * len(paths))
        assert sorted(rel) == list(range(len(paths)))
        for a in range(len(paths)):
            for b in range(a + 1, len(paths)):
                n = 0
                while paths[a][n] == paths[b][n]:
                    n += 1
                dim, where = splits[paths[a][:n]]
                camera_in_right = center[dim] > where
                a_in_right = paths[a][n] == "1"
                assert (rel[a] < rel[b]) == (a_in_right == camera_in_right)
    # unseen submodels keep their rank out of the vector; nothing seen -> all zero
    rel = so.relation_vector((0, 0, 5), paths, splits, [i % 2 == 0 for i in range(len(paths))])
    assert (rel[1::2] == -1).all() and (rel[0::2] >= 0).all()
    assert (so.relation_vector((0, 0, 5), paths, splits, [False] * len(paths)) == 0).all()


def test_relation_vector_against_the_checker():
    scene, cam0, _ = scenes.make_config("C1", shrink=400)
    rng = np.random.default_rng(9)
    for depth in (2, 3):
        part = partition.partition_scene(scene["xyz"], scene["scales"], depth)
        paths = [l.path for l in part.leaves]
        splits = _splits_of(part)
        cams = [cam0] + [random_camera(rng) for _ in range(12)]
        some_unseen = 0
        for cam in cams:
            wvt = cam.world_view_transform.numpy()
            overlaps = [so.is_overlapping_spacebox_view(part.box_low[m], part.box_up[m], wvt, cam.FoVx, cam.FoVy, 0.01, 1000.0)
                        for m in range(len(paths))]
            want = so.relation_vector(cam.camera_center.numpy(), paths, splits, overlaps)
            got = partition.relation_vector(part, cam, 0.01, 1000.0)
            assert np.array_equal(want, got)
            some_unseen += int((want < 0).any())
        assert some_unseen > 0


def test_straddler_selection_of_the_checker_against_a_scalar_loop():
    """Pins straddler_rows (result_aggregator.py:76-85, 103-106)."""
    rng = np.random.default_rng(3)
    n = 500
    xyz = rng.uniform(-1, 1, (n, 3)).astype(np.float32)
    xyz[:, 0] = -np.abs(xyz[:, 0])
    scales = np.exp(rng.normal(-3.5, 0.8, (n, 3))).astype(np.float32)
    src_low, src_up = np.float32([-1.5, -1.5, -1.5]), np.float32([0, 1.5, 1.5])
    dst_low, dst_up = np.float32([0, -1.5, -1.5]), np.float32([1, 0.2, 1.5])
    got = so.straddler_rows(xyz, scales, src_low, src_up, dst_low, dst_up)
    want = []
    for i in range(n):
        r = max(np.float32(3) * max(scales[i]), np.float32(0))
        hi = [np.float32(xyz[i, a] + r) for a in range(3)]
        lo = [np.float32(xyz[i, a] - r) for a in range(3)]
        leaves_source = any(hi[a] >= src_up[a] or lo[a] <= src_low[a] for a in range(3))
        meets = all(hi[a] >= dst_low[a] and lo[a] <= dst_up[a] for a in range(3))
        if leaves_source and meets:
            want.append(i)
    assert 5 < len(want) < n // 2 and list(got) == want
    # a Gaussian deep inside its own box is never lent, however close the destination
    assert len(so.straddler_rows(np.float32([[-0.5, 0, 0]]), np.float32([[0.01, 0.01, 0.01]]), src_low, src_up, src_low, src_up)) == 0
    # negative "scales" reach nowhere (clamp at 0) but a centre on a face still counts
    assert list(so.straddler_rows(np.float32([[0.0, 0, 0]]), np.float32([[-1, -1, -1]]), src_low, src_up, dst_low, dst_up)) == [0]


def test_merge_of_the_checker_and_its_adjoint():
    """merge_fields / merge_backward: <merge(x), g> == <x, merge_backward(g)>, own rows first."""
    rng = np.random.default_rng(4)
    counts = [7, 5, 9]
    models = [{"means3D": rng.normal(size=(c, 3)).astype(np.float32), "shs": rng.normal(size=(c, 16, 3)).astype(np.float32)}
              for c in counts]
    lent = {(s, d): np.sort(rng.choice(counts[s], size=rng.integers(0, counts[s]), replace=False))
            for s in range(3) for d in range(3) if s != d}
    for dst in range(3):
        blocks = so.merged_rows(counts, lent, dst)
        merged = so.merge_fields(models, blocks)
        assert np.array_equal(merged["means3D"][:counts[dst]], models[dst]["means3D"])
        total = counts[dst] + sum(len(lent[(s, dst)]) for s in range(3) if s != dst)
        assert merged["shs"].shape == (total, 16, 3)
        g = {n: rng.normal(size=v.shape).astype(np.float32) for n, v in merged.items()}
        back = so.merge_backward(g, blocks, [{n: v.shape for n, v in m.items()} for m in models])
        lhs = sum(float((merged[n].astype(np.float64) * g[n]).sum()) for n in merged)
        rhs = sum(float((models[s][n].astype(np.float64) * back[s][n]).sum()) for s in range(3) for n in merged)
        assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))


def test_partition_by_tensor_operations_matches_the_numpy_partition():
    """partition_scene_on_device (used for the scenes too large for the host) on the CPU device: same
    grid loads, boxes, owners and member lists as partition_scene, also when taken in several passes."""
    for name, shrink in (("C1", 100.0), ("C3", 600.0), ("C4", 2000.0)):
        scene, _, cfg = scenes.make_config(name, "cpu", shrink, geometry_only=True)
        host = partition.partition_scene(scene["xyz"], scene["scales"], cfg["bvh_depth"])
        other = partition.partition_scene_on_device(scene["xyz"], scene["scales"], cfg["bvh_depth"], rows_per_pass=20_000)
        assert np.array_equal(host.grid.load, other.grid.load)
        assert np.array_equal(host.box_low, other.box_low) and np.array_equal(host.box_up, other.box_up)
        assert np.array_equal(host.owner, other.owner.numpy())
        assert all(np.array_equal(a, b.numpy()) for a, b in zip(host.members, other.members))


def test_morton_order_is_a_permutation_that_keeps_neighbours_together():
    """The Z-order storage offered for a submodel's Gaussians: every point once, ties in index order, and points that
    are consecutive in the order lie far closer together on average than points that are consecutive as given."""
    import torch
    from retinags_amd.harness import partition
    g = torch.Generator().manual_seed(3)
    xyz = torch.rand(20_000, 3, generator=g) * torch.tensor([20.0, 20.0, 0.5])
    order = partition.morton_order(xyz)
    assert order.dtype == torch.long and torch.equal(torch.sort(order).values, torch.arange(20_000))
    step_given = (xyz[1:] - xyz[:-1]).norm(dim=1).mean()
    step_sorted = (xyz[order][1:] - xyz[order][:-1]).norm(dim=1).mean()
    assert float(step_sorted) < 0.1 * float(step_given)
    same = torch.zeros(7, 3)
    assert torch.equal(partition.morton_order(same), torch.arange(7))          # stable
    assert partition.morton_order(torch.zeros(0, 3)).numel() == 0
