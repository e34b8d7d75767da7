"""Boundary straddlers: what every submodel lends to its neighbours, and a submodel's merged
input (its own Gaussians first, then the lent ones in ascending lender id).

Host side of rgs_straddler_select / rgs_merge_rows / rgs_merge_rows_backward (include/rgs.h).
It does what gather_SharedGSInfo_pool + merge_SharedGSInfo do in the reference
(parallel_utils/basic_parallel_trainer/result_aggregator.py:55-160, 263-288) for submodels that
live on one GPU, without materialising a (source, destination) tensor set per pair: the
selection yields row lists, the merge reads the sources through them once, and the backward
adds the gradients of lent rows straight onto the lender's gradients.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _capi
from ._capi import check, lib, ptr

FIELDS = ("means3D", "means2D", "opacity", "scales", "rotations", "shs")


class SharedGSInfo:
    """The six tensors a submodel shows its renderer and its neighbours
    (parallel_utils/basic_parallel_trainer/task_utils.py:230-247): activated values, N rows each."""

    def __init__(self, means3D: torch.Tensor, means2D: torch.Tensor, opacity: torch.Tensor, scales: torch.Tensor,
                 rotations: torch.Tensor, shs: torch.Tensor) -> None:
        self.means3D = means3D
        self.means2D = means2D
        self.opacity = opacity
        self.scales = scales
        self.rotations = rotations
        self.shs = shs

    def fields(self) -> List[torch.Tensor]:
        return [getattr(self, n) for n in FIELDS]

    def __len__(self) -> int:
        return int(self.means3D.shape[0])


class StraddlerTable:
    """counts[src, dst] lent rows and, for each pair with any, their row numbers within the
    source (ascending, uint32 stored as int32 on the device)."""

    def __init__(self, counts: np.ndarray, rows: Dict[Tuple[int, int], torch.Tensor], own: List[int]) -> None:
        self.counts = counts
        self.rows = rows
        self.own = own

    def merged_size(self, dst: int) -> int:
        return self.own[dst] + int(self.counts[:, dst].sum())


def _stream(device) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_device_rows(t: torch.Tensor, width, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a device tensor: there is no host implementation")
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous float32")
    if tuple(t.shape[1:]) != tuple(width):
        raise RuntimeError(f"{name} has shape {tuple(t.shape)}, expected (N, {', '.join(map(str, width))})")


def select_straddlers(models: Sequence[SharedGSInfo], box_low, box_up, capacity: Optional[int] = None) -> StraddlerTable:
    """models[m] is submodel m with box (box_low[m], box_up[m]) in world units, (K,3) each.
    One pass over every submodel's means and scales; one device-to-host copy for all counts."""
    K = len(models)
    if K > _capi.MAX_SHARE_BOXES:
        raise RuntimeError(f"{K} submodels: at most {_capi.MAX_SHARE_BOXES} per call")
    low = np.ascontiguousarray(np.asarray(box_low, dtype=np.float32).reshape(K, 3))
    up = np.ascontiguousarray(np.asarray(box_up, dtype=np.float32).reshape(K, 3))
    fp = C.POINTER(C.c_float)
    as_fp = lambda a: a.ctypes.data_as(fp)
    device = models[0].means3D.device
    stream = _stream(device)
    own = [len(m) for m in models]
    for m in models:
        _require_device_rows(m.means3D, (3,), "means3D")
        _require_device_rows(m.scales, (3,), "scales")
    counts_dev = torch.empty((K, K), dtype=torch.int32, device=device)
    caps = [min(n, capacity if capacity is not None else n // 8 + 4096) for n in own]
    lists = [torch.empty((K, caps[s]), dtype=torch.int32, device=device) for s in range(K)]

    def run(src: int) -> None:
        n = own[src]
        scratch = torch.empty(max(1, lib.rgs_straddler_scratch_bytes(n, K)), dtype=torch.uint8, device=device)
        check(lib.rgs_straddler_select(n, ptr(models[src].means3D), ptr(models[src].scales), as_fp(low[src]), as_fp(up[src]),
                                       K, as_fp(low), as_fp(up), src, C.c_void_p(counts_dev[src].data_ptr()),
                                       ptr(lists[src]), caps[src], C.c_void_p(scratch.data_ptr()), stream))

    for src in range(K):
        run(src)
    counts = counts_dev.cpu().numpy().astype(np.int64)
    for src in range(K):
        if counts[src].max(initial=0) > caps[src]:       # a list was cut short: once more with room for the longest
            caps[src] = int(counts[src].max())
            lists[src] = torch.empty((K, caps[src]), dtype=torch.int32, device=device)
            run(src)
    rows = {(s, d): lists[s][d, :counts[s, d]] for s in range(K) for d in range(K) if counts[s, d] > 0}
    return StraddlerTable(counts, rows, own)


def _segments_for(dst: int, table: StraddlerTable) -> List[Tuple[int, Optional[torch.Tensor], int]]:
    """(source, row list or None for the destination's own rows, count), in merge order."""
    out = [(dst, None, table.own[dst])]
    for src in range(len(table.own)):
        if src != dst and table.counts[src, dst] > 0:
            out.append((src, table.rows[(src, dst)], int(table.counts[src, dst])))
    return out


def _room_behind(t: torch.Tensor, rows: int) -> bool:
    """Does the allocation t lives in continue for `rows` rows of t's width past t's first row?"""
    width = int(np.prod(t.shape[1:])) if t.dim() > 1 else 1
    return (t.storage_offset() + rows * width) * t.element_size() <= t.untyped_storage().nbytes()


def _grown(t: torch.Tensor, rows: int) -> torch.Tensor:
    """A tensor over the same memory as t with `rows` rows: t's own rows and the room behind them."""
    width = tuple(t.shape[1:])
    stride = tuple(t.stride())
    return torch.empty(0, dtype=t.dtype, device=t.device).set_(t.untyped_storage(), t.storage_offset(), (rows,) + width, stride)


class _MergeShared(torch.autograd.Function):
    """All destinations at once, so that a lender's gradient is written in one place: its own
    rows' gradient plus what every borrower adds."""

    @staticmethod
    def forward(ctx, table: StraddlerTable, reuse_gradients: bool, append: bool, *flat):
        K = len(table.own)
        models = [flat[6 * m:6 * m + 6] for m in range(K)]
        device = flat[0].device
        stream = _stream(device)
        sh_shape = tuple(models[0][5].shape[1:])
        sh_floats = int(np.prod(sh_shape)) if sh_shape else 0
        outs = []
        for dst in range(K):
            P = table.merged_size(dst)
            if append:
                # the lent rows go behind the destination's own rows, which stay where they are
                for f, t in enumerate(models[dst]):
                    if not _room_behind(t, P):
                        raise RuntimeError(f"submodel {dst}: no room for {P - table.own[dst]} lent rows behind its "
                                           f"{FIELDS[f]}; allocate the field with spare rows or merge with append=False")
                merged = [_grown(t, P) for t in models[dst]]
                merged[1][table.own[dst]:].zero_()
                segs = _segments_for(dst, table)[1:]
                first = table.own[dst]
            else:
                merged = [torch.empty((P, 3), device=device), torch.zeros((P, 3), device=device),
                          torch.empty((P, 1), device=device), torch.empty((P, 3), device=device),
                          torch.empty((P, 4), device=device), torch.empty((P,) + sh_shape, device=device)]
                segs = _segments_for(dst, table)
                first = 0
            arr = (_capi.SharedRows * len(segs))()
            for k, (src, rows, count) in enumerate(segs):
                m3, _, op, sc, ro, sh = models[src]
                arr[k] = _capi.SharedRows(m3.data_ptr(), op.data_ptr(), sc.data_ptr(), ro.data_ptr(), sh.data_ptr(),
                                          rows.data_ptr() if rows is not None else None, count)
            check(lib.rgs_merge_rows(len(segs), arr, first, sh_floats, ptr(merged[0]), ptr(merged[2]), ptr(merged[3]),
                                     ptr(merged[4]), ptr(merged[5]), stream))
            outs.extend(merged)
        ctx.table = table
        ctx.reuse = reuse_gradients
        ctx.sh_floats = sh_floats
        ctx.shapes = [tuple(t.shape) for t in flat]
        ctx.device = device
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        table, K = ctx.table, len(ctx.table.own)
        stream = _stream(ctx.device)
        # a lender's gradient starts as the gradient of its own rows in its own merged arrays
        out: List[Optional[torch.Tensor]] = []
        for m in range(K):
            for f in range(6):
                g = grads[6 * m + f]
                if g is None:
                    out.append(torch.zeros(ctx.shapes[6 * m + f], device=ctx.device))
                else:
                    g = g.contiguous()[:table.own[m]]
                    out.append(g if ctx.reuse else g.clone())
        for dst in range(K):
            segs = _segments_for(dst, table)[1:]
            if not segs or all(grads[6 * dst + f] is None for f in range(6)):
                continue
            arr = (_capi.SharedGrads * len(segs))()
            for k, (src, rows, count) in enumerate(segs):
                arr[k] = _capi.SharedGrads(*[out[6 * src + f].data_ptr() for f in range(6)], rows.data_ptr(), count)
            g = [grads[6 * dst + f] for f in range(6)]
            g = [None if t is None else t.contiguous() for t in g]
            check(lib.rgs_merge_rows_backward(len(segs), arr, table.own[dst], ctx.sh_floats, *[ptr(t) for t in g], stream))
        return (None, None, None) + tuple(out)


def merge_shared(models: Sequence[SharedGSInfo], table: StraddlerTable, reuse_gradients: bool = False,
                 append: bool = False) -> List[SharedGSInfo]:
    """Every submodel's merged input (merge_SharedGSInfo, result_aggregator.py:263-288, for all
    destinations), differentiable with respect to every field of every submodel.

    append: instead of copying a submodel's own rows into new arrays, write the lent rows into
    the memory right behind them and return tensors over both.  Every field of every submodel
    must then sit in an allocation with that much room behind its rows (with_spare_rows makes
    such tensors); the merged tensors alias the submodel's own, and the room behind is
    overwritten by every merge.  Autograd does not know of that aliasing (the merged tensors are
    built over the inputs' storage, so the inputs' version counters do not guard them): the
    inputs must not be updated in place, and no other merge may run, between this call and the
    backward of everything that was rendered from its result.

    reuse_gradients: the backward returns the incoming gradient buffers of the merged arrays,
    with the borrowers' rows added in place, instead of copies.  Only for callers that do not
    read the merged arrays' gradients afterwards (no retain_grad on them)."""
    for m in models:
        for name, width in (("means3D", (3,)), ("means2D", (3,)), ("opacity", (1,)), ("scales", (3,)), ("rotations", (4,))):
            _require_device_rows(getattr(m, name), width, name)
        _require_device_rows(m.shs, tuple(models[0].shs.shape[1:]), "shs")
    flat = [t for m in models for t in m.fields()]
    outs = _MergeShared.apply(table, reuse_gradients, append, *flat)
    return [SharedGSInfo(*outs[6 * m:6 * m + 6]) for m in range(len(models))]


def with_spare_rows(t: torch.Tensor, spare: int) -> torch.Tensor:
    """A copy of t (N rows) at the start of an allocation of N + spare rows, for merge_shared(append=True)."""
    room = torch.empty((t.shape[0] + spare,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
    room[:t.shape[0]].copy_(t)
    return room[:t.shape[0]]
