"""Per-graph split of an adjacency into dense bit blocks and a sparse rest (graph preprocessing,
an extension of cuda/util.py:5-11 of the reference, which caches CSR / CSC / COO once per graph).

On power-law graphs the cells (row i, column j) with expected density deg(i) * cnt(j) / nnz above a
percent or so hold a large part of all edges.  With rows and columns ranked by falling slot count that
region is a staircase: row block b (256 consecutive row ranks) gets the columns of rank below
``extent[b]``.  Inside it an edge is one bit and the copy_u aggregation a 0/1 x int8 matrix product
(tango_spmm_csr_copy_u_dense); everything else stays a CSR.  The split changes no result: integer
sums are exact in any order.
"""
import ctypes
import os

import numpy as np
import torch

from . import _lib
from ._lib import check

ROWS = 256   # rows of a row block
UNIT = 256   # mask columns of a unit


def default_tau():
    """Density above which a cell is worth a bit: a cell costs the matrix cores about 0.9 % of what a gathered
    edge costs the gather kernel, at 64 columns as at 256 (measured on the 114.8 M-edge benchmark graph, where
    0.009 .. 0.011 give the shortest epochs: 4.83 / 4.81 / 4.80 / 4.82 ms at 0.008 / 0.009 / 0.010 / 0.011);
    TANGO_DENSE_TAU overrides, 0 switches the dense blocks off."""
    return float(os.environ.get("TANGO_DENSE_TAU", "0.010"))


class DensePlan:
    """Device tensors of one orientation's split plus the C struct that points at them."""

    def __init__(self, **kw):
        self.__dict__.update(kw)
        s = _lib.DensePlan()
        s.rows, s.num_src = self.rows, self.num_src
        s.dense_rows, s.dense_cols = self.row_blocks * ROWS, self.dense_cols
        s.row_blocks, s.num_groups = self.row_blocks, self.seg_ptr.numel() - 1
        s.num_groups2, s.num_shared = self.seg_ptr2.numel() - 1, self.shared_blocks.numel()
        for name in ("col_ids", "row_slot", "row_order", "mask_off", "mask", "seg_ptr", "segs", "seg_ptr2", "segs2", "shared_blocks",
                     "res_indptr", "res_indices"):
            t = getattr(self, name)
            setattr(s, name, t.data_ptr() if t is not None and t.numel() else None)
        s.res_nnz, s.res_max_row = self.res_indices.numel(), self.res_max_row
        self.struct = s
        self.ref = ctypes.byref(s)


# what a segment costs beside its units, in units of work: its prologue and flush; the atomic flush of a shared block
SEGMENT_COST = 1.8
SHARED_COST = 1.3


def _segments(units, groups, min_piece=4):
    """Deals the units of every row block over ``groups`` workgroups so that all finish together (a launch lasts
    as long as its slowest workgroup).  Blocks of less than 0.8 of a fair share stay whole and go, heaviest first,
    to the least loaded workgroup; the longer blocks are then poured into what room is left below a common level,
    cut where a workgroup is full (several workgroups then add into such a block's partial sums).  Returns (seg_ptr, segs [(row block, first unit, units, shared)], shared_blocks)
    as numpy."""
    total = int(units.sum())
    groups = max(1, min(groups, total))
    fair = total / groups
    whole = sorted(((n, b) for b, n in enumerate(units.tolist()) if 0 < n <= 0.8 * fair), reverse=True)
    cut = sorted(((n, b) for b, n in enumerate(units.tolist()) if n > 0.8 * fair), reverse=True)
    load = np.zeros(groups)
    per_group = [[] for _ in range(groups)]
    for n, b in whole:
        g = int(np.argmin(load))
        per_group[g].append((b, 0, n, 0))
        load[g] += n + SEGMENT_COST
    piece_cost = SEGMENT_COST + SHARED_COST
    need = sum(n for n, _ in cut)

    def room(level):
        r = np.floor(level - load - piece_cost)
        r[r < min_piece] = 0
        return r

    lo, hi = 0.0, float(load.max() + need + piece_cost + min_piece)
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        if room(mid).sum() >= need:
            hi = mid
        else:
            lo = mid
    left = room(hi).astype(np.int64)
    order = [int(g) for g in np.argsort(-left, kind="stable") if left[g] > 0]
    gi = 0
    for n, b in cut:
        a = 0
        while n > 0:
            if gi < len(order):
                g = order[gi]
                take = int(min(n, left[g]))
                if 0 < n - take < min_piece:  # no sliver of a block: this workgroup takes it too
                    take = n
                left[g] -= take
                if left[g] < min_piece:
                    gi += 1
            else:  # rounding leftovers
                g = int(np.argmin(load))
                take = n
            per_group[g].append((b, a, take, 1))
            load[g] += take + piece_cost
            a += take
            n -= take
    pieces = {}
    for lst in per_group:
        for b, _, _, _ in lst:
            pieces[b] = pieces.get(b, 0) + 1
    shared = sorted(b for b, k in pieces.items() if k > 1)
    seg_ptr = np.zeros(groups + 1, dtype=np.int32)
    segs = []
    for g, lst in enumerate(per_group):
        lst.sort(key=lambda it: -it[2])  # the longest piece first
        segs.extend((b, a, n, 1 if pieces[b] > 1 else 0) for b, a, n, _ in lst)
        seg_ptr[g + 1] = len(segs)
    return seg_ptr, np.asarray(segs, dtype=np.int32).reshape(-1, 4), np.asarray(shared, dtype=np.int32)


def build_dense_plan(indptr, indices, num_src, tau=None, groups=256, sort_rest=True, min_share=0.05, min_extent=None):
    """Splits the CSR (indptr int64 [rows + 1], indices int32 / int64 [nnz], gathered rows < num_src).
    Returns a DensePlan, or None when fewer than ``min_share`` of the slots would become bits."""
    tau = default_tau() if tau is None else float(tau)
    min_extent = int(os.environ.get("TANGO_DENSE_MIN_EXTENT", "4096")) if min_extent is None else int(min_extent)
    min_extent = max(min_extent, UNIT)
    rows = indptr.numel() - 1
    nnz = indices.numel()
    if tau <= 0 or rows <= 0 or nnz == 0:
        return None
    dev = indptr.device
    row_deg = torch.diff(indptr)
    col_cnt = torch.bincount(indices, minlength=num_src)
    row_order = torch.argsort(row_deg, descending=True, stable=True)
    col_order = torch.argsort(col_cnt, descending=True, stable=True)
    rd = row_deg[row_order].cpu().numpy().astype(np.float64)
    cc = col_cnt[col_order].cpu().numpy().astype(np.float64)
    extents = []
    for b in range((rows + ROWS - 1) // ROWS):
        mean_deg = rd[b * ROWS:(b + 1) * ROWS].mean()
        if mean_deg <= 0:
            break
        cols = int(np.searchsorted(-cc, -(tau * nnz / mean_deg), side="left"))  # columns with cnt * deg / nnz > tau
        ext = cols // UNIT * UNIT
        if ext < min_extent:  # a block's partial sums cost a write and a read of 256 rows whatever its extent
            break
        extents.append(ext)
    if not extents:
        return None
    extents = np.asarray(extents, dtype=np.int64)
    # expected number of slots inside the blocks under the density model
    covered = sum(np.minimum(1.0, rd[b * ROWS:(b + 1) * ROWS].mean() * cc[:e] / nnz).sum() * ROWS for b, e in enumerate(extents))
    if covered < min_share * nnz:
        return None
    row_blocks = len(extents)
    row_rank = torch.empty(rows, dtype=torch.int32, device=dev)
    row_rank[row_order] = torch.arange(rows, dtype=torch.int32, device=dev)
    col_rank = torch.empty(num_src, dtype=torch.int32, device=dev)
    col_rank[col_order] = torch.arange(num_src, dtype=torch.int32, device=dev)
    mask_words = extents * (ROWS // 32)
    mask_off = np.concatenate([[0], np.cumsum(mask_words)[:-1]]).astype(np.int64)
    mask = torch.zeros(int(mask_words.sum()), dtype=torch.int32, device=dev)
    mask_off_t = torch.from_numpy(mask_off).to(dev)
    extent_t = torch.from_numpy(extents.astype(np.int32)).to(dev)
    keep = torch.empty(nnz, dtype=torch.uint8, device=dev)
    kept = torch.empty(rows, dtype=torch.int32, device=dev)
    idx_bits = 32 if indices.dtype == torch.int32 else 64
    stream = torch.cuda.current_stream(dev).cuda_stream
    check(_lib.lib().tango_spmm_dense_mask_build(indptr.data_ptr(), indices.data_ptr(), idx_bits, rows,
                                                 row_rank.data_ptr(), col_rank.data_ptr(), extent_t.data_ptr(),
                                                 mask_off_t.data_ptr(), row_blocks, mask.data_ptr(), keep.data_ptr(),
                                                 kept.data_ptr(), stream), "dense_mask_build")
    res_indices = indices[keep.bool()].to(torch.int32)
    res_indptr = torch.zeros(rows + 1, dtype=torch.int64, device=dev)
    torch.cumsum(kept, 0, out=res_indptr[1:])
    if sort_rest and res_indices.numel():
        # inside a row, popular sources first: rows walked at the same time then ask for the same lines
        row_of = torch.repeat_interleave(torch.arange(rows, device=dev), kept.long())
        key = row_of * num_src + col_rank[res_indices.long()].long()
        del row_of
        res_indices = res_indices[torch.argsort(key)]
        del key
    del keep
    seg_ptr, segs, shared = _segments(extents // UNIT, groups)
    seg_ptr2, segs2, shared2 = _segments(extents // UNIT, 2 * groups)
    shared = np.union1d(shared, shared2).astype(np.int32)
    row_slot = torch.where(row_rank < row_blocks * ROWS, row_rank, torch.full_like(row_rank, -1))
    # the gather kernel takes the rows in rank order: the rows that share a wavefront are then about equally long
    # (ordering by the number of slots left to it instead was measured: the same times)
    return DensePlan(
        row_order=row_order.to(torch.int32).contiguous(),
        rows=rows, num_src=int(num_src), row_blocks=row_blocks, dense_cols=int(extents.max()),
        tau=tau, nnz=nnz,
        col_ids=col_order[:int(extents.max())].to(torch.int32).contiguous(), row_slot=row_slot.contiguous(),
        mask_off=mask_off_t, mask=mask, seg_ptr=torch.from_numpy(seg_ptr).to(dev),
        segs=torch.from_numpy(segs).to(dev).contiguous(), seg_ptr2=torch.from_numpy(seg_ptr2).to(dev),
        segs2=torch.from_numpy(segs2).to(dev).contiguous(), shared_blocks=torch.from_numpy(shared).to(dev),
        res_indptr=res_indptr, res_indices=res_indices.contiguous(),
        res_max_row=int(kept.max().item()) if rows else 0,
        cells=int((extents * ROWS).sum()))
