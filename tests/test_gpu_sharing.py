"""Boundary straddlers on the GPU (rgs_straddler_select, rgs_merge_rows, rgs_merge_rows_backward
through retinags_amd/sharing.py) against the CPU checker: row lists and merged rows bit for bit,
gradients to float32 rounding of at most K additions."""
import numpy as np
import pytest
import torch

from helpers import np32, scenes
from oracle import sharing_oracle as so

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NAMES = ("means3D", "means2D", "opacity", "scales", "rotations", "shs")


def _setup(shrink, depth, scale_shift=0.0, spare_fraction=0.0):
    from retinags_amd.harness import partition, pipeline
    scene, cam, _ = scenes.make_config("C1", shrink=shrink)
    if scale_shift:
        scene["scales"] = scene["scales"] * float(np.exp(scale_shift))
    part = partition.partition_scene(scene["xyz"], scene["scales"], depth)
    models = pipeline.owned_models_from_partition(scene, part, DEV, spare_fraction)
    return scene, cam, part, models


def _host_fields(models):
    return [{n: np32(getattr(m, n)) for n in NAMES} for m in models]


@pytest.mark.parametrize("shrink,depth,scale_shift", [(40, 2, 0.0), (150, 3, 1.0), (400, 4, 2.0)])
def test_row_lists_against_checker(shrink, depth, scale_shift):
    from retinags_amd import sharing
    scene, cam, part, models = _setup(shrink, depth, scale_shift)
    K = len(models)
    table = sharing.select_straddlers(models, part.box_low, part.box_up)
    host = _host_fields(models)
    lent_total = 0
    for s in range(K):
        for d in range(K):
            if s == d:
                assert table.counts[s, d] == 0
                continue
            want = so.straddler_rows(host[s]["means3D"], host[s]["scales"], part.box_low[s], part.box_up[s],
                                     part.box_low[d], part.box_up[d])
            assert table.counts[s, d] == len(want), (s, d)
            if len(want):
                assert np.array_equal(table.rows[(s, d)].cpu().numpy().astype(np.int64), want), (s, d)
            lent_total += len(want)
    assert lent_total > 50
    # the scene-level restatement of the harness names the same Gaussians in the same order
    own_ids = [np.nonzero(part.owner == k)[0] for k in range(K)]
    for d in range(K):
        ids = [own_ids[d]] + [own_ids[s][table.rows[(s, d)].cpu().numpy()] for s in range(K) if (s, d) in table.rows]
        assert np.array_equal(np.concatenate(ids), part.members[d])


def test_truncated_lists_are_redone_with_room():
    from retinags_amd import sharing
    scene, cam, part, models = _setup(100, 2, 1.5)
    full = sharing.select_straddlers(models, part.box_low, part.box_up)
    assert full.counts.max() > 16
    tight = sharing.select_straddlers(models, part.box_low, part.box_up, capacity=16)
    assert np.array_equal(full.counts, tight.counts)
    for key, rows in full.rows.items():
        assert torch.equal(rows, tight.rows[key])


def test_one_submodel_empty_submodel_and_distant_boxes():
    """Nothing to lend: a single submodel, a submodel without Gaussians, boxes that are far apart."""
    from retinags_amd import sharing
    g = torch.Generator().manual_seed(2)

    def model(n, centre):
        xyz = (torch.rand(n, 3, generator=g) - 0.5 + torch.tensor(centre)).to(DEV)
        return sharing.SharedGSInfo(xyz, torch.zeros_like(xyz), torch.rand(n, 1, generator=g).to(DEV),
                                    (torch.rand(n, 3, generator=g) * 0.01).to(DEV), torch.randn(n, 4, generator=g).to(DEV),
                                    torch.randn(n, 16, 3, generator=g).to(DEV))

    one = [model(500, (0.0, 0.0, 0.0))]
    table = sharing.select_straddlers(one, [[-1, -1, -1]], [[1, 1, 1]])
    assert table.counts.tolist() == [[0]] and not table.rows
    merged = sharing.merge_shared(one, table)
    assert all(torch.equal(a, b) for a, b in zip(merged[0].fields(), one[0].fields()))

    models = [model(300, (0.0, 0.0, 0.0)), model(0, (10.0, 0.0, 0.0)), model(200, (20.0, 0.0, 0.0))]
    low = [[-1, -1, -1], [9, -1, -1], [19, -1, -1]]
    up = [[1, 1, 1], [11, 1, 1], [21, 1, 1]]
    table = sharing.select_straddlers(models, low, up)
    assert int(table.counts.sum()) == 0
    for m in models:
        for t in m.fields():
            t.requires_grad_(True)
    merged = sharing.merge_shared(models, table)
    assert [len(m) for m in merged] == [300, 0, 200]
    torch.autograd.backward([merged[0].shs, merged[2].means3D], [torch.ones_like(merged[0].shs), torch.ones_like(merged[2].means3D)])
    assert float(models[0].shs.grad.min()) == 1.0 and float(models[2].means3D.grad.min()) == 1.0
    assert models[1].shs.grad is None or models[1].shs.grad.numel() == 0
    # a Gaussian of submodel 0 that reaches into submodel 2's box is lent to it and to nobody else
    with torch.no_grad():
        models[0].scales[7] = 7.0
    table = sharing.select_straddlers(models, low, up)
    assert table.counts.tolist() == [[0, 1, 1], [0, 0, 0], [0, 0, 0]]
    assert table.rows[(0, 2)].tolist() == [7] and table.rows[(0, 1)].tolist() == [7]
    torch.cuda.synchronize()


def test_merge_and_its_backward_against_checker():
    from retinags_amd import sharing
    scene, cam, part, models = _setup(60, 2, 1.0)
    K = len(models)
    for m in models:
        for t in m.fields():
            t.requires_grad_(True)
    table = sharing.select_straddlers(models, part.box_low, part.box_up)
    merged = sharing.merge_shared(models, table)
    host = _host_fields(models)
    lent = {(s, d): (table.rows[(s, d)].cpu().numpy() if (s, d) in table.rows else np.zeros(0, np.int64))
            for s in range(K) for d in range(K) if s != d}
    gen = torch.Generator().manual_seed(3)
    blocks, ups = [], []
    for d in range(K):
        blocks.append(so.merged_rows(table.own, lent, d))
        want = so.merge_fields(host, blocks[d])
        for n in NAMES:
            got = getattr(merged[d], n).detach().cpu().numpy()
            assert got.shape == want[n].shape and np.array_equal(got, want[n]), (d, n)
        ups.append({n: torch.randn(getattr(merged[d], n).shape, generator=gen) for n in NAMES})
    torch.autograd.backward([getattr(merged[d], n) for d in range(K) for n in NAMES],
                            [ups[d][n].to(DEV) for d in range(K) for n in NAMES])
    torch.cuda.synchronize()
    shapes = [{n: v.shape for n, v in h.items()} for h in host]
    want = [{n: np.zeros(s, np.float32) for n, s in sh.items()} for sh in shapes]
    for d in range(K):
        back = so.merge_backward({n: ups[d][n].numpy() for n in NAMES}, blocks[d], shapes)
        for s in range(K):
            for n in NAMES:
                want[s][n] += back[s][n]
    for s in range(K):
        for n in NAMES:
            got = getattr(models[s], n).grad.cpu().numpy()
            assert np.abs(got - want[s][n]).max() <= 1e-5, (s, n)


def test_in_place_gradients_match_copies():
    from retinags_amd import sharing
    scene, cam, part, models = _setup(100, 2, 1.0)
    K = len(models)
    for m in models:
        for t in m.fields():
            t.requires_grad_(True)
    table = sharing.select_straddlers(models, part.box_low, part.box_up)
    results = []
    for reuse in (False, True):
        for m in models:
            for t in m.fields():
                t.grad = None
        merged = sharing.merge_shared(models, table, reuse_gradients=reuse)
        gen = torch.Generator().manual_seed(8)
        outs = [getattr(merged[d], n) for d in range(K) for n in NAMES]
        torch.autograd.backward(outs, [torch.randn(o.shape, generator=gen).to(DEV) for o in outs])
        torch.cuda.synchronize()
        results.append([t.grad.clone() for m in models for t in m.fields()])
    for a, b in zip(*results):
        assert torch.equal(a, b)


def test_lent_rows_appended_in_place_match_the_copying_merge():
    """append=True leaves a submodel's own rows where they are and writes the lent rows behind
    them; merged values and every gradient are those of the copying merge."""
    from retinags_amd import sharing
    scene, cam, part, models = _setup(100, 2, 1.0, spare_fraction=0.2)
    K = len(models)
    for m in models:
        for t in m.fields():
            t.requires_grad_(True)
    table = sharing.select_straddlers(models, part.box_low, part.box_up)
    values, grads = [], []
    for append in (False, True):
        for m in models:
            for t in m.fields():
                t.grad = None
        merged = sharing.merge_shared(models, table, reuse_gradients=append, append=append)
        if append:
            assert all(a.data_ptr() == b.data_ptr() for m, g in zip(models, merged) for a, b in zip(m.fields(), g.fields()))
        values.append([t.detach().clone() for g in merged for t in g.fields()])
        gen = torch.Generator().manual_seed(12)
        outs = [t for g in merged for t in g.fields()]
        torch.autograd.backward(outs, [torch.randn(o.shape, generator=gen).to(DEV) for o in outs])
        torch.cuda.synchronize()
        grads.append([t.grad.clone() for m in models for t in m.fields()])
    assert all(torch.equal(a, b) for a, b in zip(*values))
    assert all(torch.equal(a, b) for a, b in zip(*grads))
    # without room behind the rows the request is refused
    tight = [sharing.SharedGSInfo(*[t.detach().clone() for t in m.fields()]) for m in models]
    with pytest.raises(RuntimeError, match="no room"):
        sharing.merge_shared(tight, table, append=True)


def test_frame_through_shared_rows_matches_frame_from_host_lists():
    """The rendered, composited, differentiated frame is the same whether every submodel's input
    was put together on the host from the scene or on the GPU from what its neighbours lend."""
    from retinags_amd import sharing
    from retinags_amd.harness import partition, pipeline
    scene, cam, part, models = _setup(60, 2, 0.5)
    rel = partition.relation_vector(part, cam)
    cam_d = cam.to(DEV)
    bg = torch.tensor([0.1, 0.2, 0.3], device=DEV)
    up = (torch.randn(3, cam.image_height, cam.image_width, generator=torch.Generator().manual_seed(1)) * 1e-2).to(DEV)

    subs_host = [s.requires_grad_(True) for s in pipeline.submodels_from_partition(scene, part, DEV)]
    a = pipeline.render_frame(cam_d, subs_host, rel, bg)
    torch.autograd.backward([a["render"]], [up])

    for m in models:
        for t in m.fields():
            t.requires_grad_(True)
    table = sharing.select_straddlers(models, part.box_low, part.box_up)
    merged = sharing.merge_shared(models, table, reuse_gradients=True)
    b = pipeline.render_frame(cam_d, pipeline.submodels_from_shared(merged, part, DEV), rel, bg)
    torch.autograd.backward([b["render"]], [up])
    torch.cuda.synchronize()
    assert torch.equal(a["render"], b["render"]) and torch.equal(a["alpha"], b["alpha"])

    # gradient of a scene Gaussian = sum over the submodels that render it
    n = scene["xyz"].shape[0]
    own_ids = [np.nonzero(part.owner == k)[0] for k in range(len(models))]
    for name, field in (("means3D", "means3D"), ("opacity", "opacity"), ("scales", "scales"), ("rotations", "rotations"), ("shs", "shs")):
        want = torch.zeros((n,) + tuple(getattr(models[0], field).shape[1:]), device=DEV)
        got = torch.zeros_like(want)
        for k in range(len(models)):
            want.index_add_(0, torch.from_numpy(part.members[k]).to(DEV), getattr(subs_host[k], name).grad)
            got[torch.from_numpy(own_ids[k]).to(DEV)] = getattr(models[k], field).grad
        scale = float(want.abs().max())
        assert float((got - want).abs().max()) <= 1e-4 * max(scale, 1e-12), name
    # the screen-space gradient reaches the lender's placeholder too
    assert all(m.means2D.grad is not None and torch.isfinite(m.means2D.grad).all() for m in models)
    assert any(float(m.means2D.grad.abs().sum()) > 0 for m in models)
