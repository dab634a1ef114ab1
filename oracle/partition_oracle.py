"""CPU restatement of the block-level partitioner and the degree sort.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.

What is restated here (reference files, relative to the upstream tree):

* the per-degree lookup tables            block_level_partition.py:7-21
* the walk over the degree-sorted rows    block_level_partition.py:48-103
* the on-disk ``.block4`` layout          block_level_partition.py:105-106
* how the kernel reads each field back    spmm_accel.cu:21-28,34

Two independent formulations are kept on purpose: ``partition_walk`` is a
row-at-a-time state machine (small inputs), ``partition_closed_form`` is a
vectorised numpy formula (large inputs, the 16 golden ``.block4`` files).
They are checked against each other and both against the golden files.

Pinned by: the 16 ``.block4`` files the reference ships (every degree 1..384
occurs in them, 1,510 distinct degrees above 384 including the exact multiples
768, 1152 and 5376), brute force on tiny inputs, and table known-answers.

The degree sort is not in the reference (only its output files are consumed,
block_level_partition.py:31-32,38); the golden files show ascending order with
zero-degree rows first.  The tie-break is this build's choice: stable, i.e.
ties keep original row order.  ``degree_sort`` is therefore *defined* by
``numpy.argsort(kind="stable")``; it is pinned by sortedness + stability
properties, not by a reference vector.
"""
from __future__ import annotations

import numpy as np

DEG_BOUND = 384          # block_level_partition.py:7, spmm_accel.cu:11
SLICES_PER_BLOCK = 12    # block_level_partition.py:8, spmm_accel.cu:12
SLICE_NZ = DEG_BOUND // SLICES_PER_BLOCK   # 32 non-zeros per slice


def slice_tables():
    """Return (w_nz, rows_per_block) indexed by degree 0..DEG_BOUND.

    block_level_partition.py:12-21 fills the tables for degrees 1..191 with
    split factors 1,2,3,4,6; degrees 192..384 fall off the table and take the
    defaults of lines 56-63 (32 non-zeros per slice, one row per block).
    """
    w_nz = np.zeros(DEG_BOUND + 1, dtype=np.int64)
    rows = np.zeros(DEG_BOUND + 1, dtype=np.int64)
    for d in range(1, DEG_BOUND + 1):
        if d < DEG_BOUND // 2:
            split = next(f for f in (1, 2, 3, 4, 6) if f * SLICE_NZ >= d)
            w_nz[d] = -(-d // split)
            rows[d] = SLICES_PER_BLOCK // split
        else:
            w_nz[d] = SLICE_NZ
            rows[d] = 1
    return w_nz, rows


def _degrees(indptr):
    indptr = np.asarray(indptr)
    if indptr.ndim != 1 or indptr.size < 1:
        raise ValueError("indptr must be a 1-D array with at least one entry")
    return np.diff(indptr.astype(np.int64))


def partition_walk(indptr):
    """Row-at-a-time restatement (block_level_partition.py:48-103).

    Returns an int32 array of shape [B, 4] = (degree, row_begin, loc_begin,
    info).  Works on any row order: a block groups consecutive rows of equal
    degree, rows of degree 0 emit nothing.
    """
    deg = _degrees(indptr)
    w_tab, r_tab = slice_tables()
    n = deg.size
    out = []
    row = 0
    loc = 0
    while row < n:
        d = int(deg[row])
        if d == 0:
            row += 1
            continue
        if d <= DEG_BOUND:
            cap = int(r_tab[d])
            taken = 1
            while taken < cap and row + taken < n and deg[row + taken] == d:
                taken += 1
            out.append((d, row, loc, (int(w_tab[d]) << 16) + taken))
            row += taken
            loc += taken * d
        else:
            done = 0
            while done < d:
                seg = min(DEG_BOUND, d - done)
                out.append((d, row, loc, seg))
                loc += seg
                done += seg
            row += 1
    return np.asarray(out, dtype=np.int32).reshape(-1, 4)


def partition_closed_form(indptr):
    """Vectorised restatement: same result as ``partition_walk``.

    For a row r of degree d in 1..384 inside a maximal run of equal-degree
    rows that starts at s: r opens a block iff (r - s) % rows[d] == 0, and
    the block holds min(rows[d], run_end - r) rows.  A row with d > 384 opens
    ceil(d / 384) blocks of 384 non-zeros, the last one shorter unless d is a
    multiple of 384.  loc_begin is the running count of non-zeros.
    """
    deg = _degrees(indptr)
    n = deg.size
    if n == 0:
        return np.zeros((0, 4), dtype=np.int32)
    w_tab, r_tab = slice_tables()
    rid = np.arange(n, dtype=np.int64)
    head = np.ones(n, dtype=bool)
    head[1:] = deg[1:] != deg[:-1]
    run_start = np.maximum.accumulate(np.where(head, rid, 0))
    head_pos = np.flatnonzero(head)
    run_id = np.cumsum(head) - 1
    run_end = np.append(head_pos[1:], n)[run_id]
    loc = np.concatenate(([0], np.cumsum(deg)[:-1]))

    short = (deg >= 1) & (deg <= DEG_BOUND)
    dcl = np.clip(deg, 0, DEG_BOUND)
    cap = r_tab[dcl]
    opens = short & ((rid - run_start) % np.maximum(cap, 1) == 0)
    long_ = deg > DEG_BOUND
    nseg = np.where(long_, -(-deg // DEG_BOUND), 0)
    per_row = np.where(opens, 1, nseg)

    src = np.repeat(rid, per_row)                  # row that emits each block
    first = np.concatenate(([0], np.cumsum(per_row)[:-1]))
    k = np.arange(src.size, dtype=np.int64) - first[src]   # segment number
    d_src = deg[src]
    is_long = d_src > DEG_BOUND
    n_rows = np.minimum(cap[src], run_end[src] - src)
    seg_len = np.minimum(DEG_BOUND, d_src - k * DEG_BOUND)
    info = np.where(is_long, seg_len, (w_tab[np.clip(d_src, 0, DEG_BOUND)] << 16) + n_rows)
    out = np.stack([d_src, src, loc[src] + k * DEG_BOUND, info], axis=1)
    return out.astype(np.int32)


def decode_block4(block4):
    """Invert the metadata the way the kernel reads it (spmm_accel.cu:21-28).

    Returns (row_begin, n_rows, row_nz, loc_begin, is_long) per block.
    """
    b = np.asarray(block4, dtype=np.int64).reshape(-1, 4)
    deg, row, loc, info = b[:, 0], b[:, 1], b[:, 2], b[:, 3]
    is_long = deg > DEG_BOUND
    n_rows = np.where(is_long, 1, info & 0xFFFF)
    row_nz = np.where(is_long, info, deg)
    return row, n_rows, row_nz, loc, is_long


def degrees_from_block4(block4, n_rows_total=None):
    """Recover the degree sequence a ``.block4`` file was built from.

    Rows not covered by any block have degree 0 (block_level_partition.py:
    52-53 emits nothing for them).  ``n_rows_total`` extends the sequence with
    trailing zero-degree rows; by default it ends at the last covered row.
    """
    b = np.asarray(block4, dtype=np.int64).reshape(-1, 4)
    row, n_rows, _, _, is_long = decode_block4(b)
    last = int((row + n_rows).max()) if b.size else 0
    n = last if n_rows_total is None else int(n_rows_total)
    deg = np.zeros(n, dtype=np.int64)
    first_seg = np.ones(b.shape[0], dtype=bool)
    first_seg[1:] = ~(is_long[1:] & (row[1:] == row[:-1]))
    for r, c, d in zip(row[first_seg], n_rows[first_seg], b[first_seg, 0]):
        deg[r:r + c] = d
    return deg


def indptr_from_degrees(deg):
    deg = np.asarray(deg, dtype=np.int64)
    out = np.zeros(deg.size + 1, dtype=np.int64)
    np.cumsum(deg, out=out[1:])
    if out[-1] >= 2 ** 31:
        raise ValueError("nnz does not fit int32")
    return out.astype(np.int32)


def degree_sort(indptr):
    """perm[new_row] = old_row, ascending degree, ties by original row id."""
    return np.argsort(_degrees(indptr), kind="stable").astype(np.int32)


def permute_csr(indptr, indices, values, perm):
    """Rows of the CSR taken in the order ``perm`` (columns are not relabelled)."""
    indptr = np.asarray(indptr, dtype=np.int64)
    perm = np.asarray(perm, dtype=np.int64)
    deg = np.diff(indptr)[perm]
    new_indptr = np.zeros(perm.size + 1, dtype=np.int64)
    np.cumsum(deg, out=new_indptr[1:])
    src = np.repeat(indptr[:-1][perm] - new_indptr[:-1], deg) + np.arange(new_indptr[-1])
    return (new_indptr.astype(np.int32), np.asarray(indices)[src],
            None if values is None else np.asarray(values)[src])


N_COLUMN_GROUPS = 8


def column_group(col, groups=N_COLUMN_GROUPS):
    """Which column group a column belongs to (groups of 8 consecutive columns,
    round-robin over ``groups`` = 8, 16, 32 or 64).  This is the build's own
    layout rule for the rows it cuts into pieces; upstream has no counterpart
    (it never reorders the non-zeros of a row), so it is pinned by its
    definition and by the SpMM result being unchanged."""
    return (np.asarray(col) >> 3) & (groups - 1)


GROUP_MIN_PIECE = 96


def row_groups(d, forced=0):
    """Column groups a split row of degree d is stored in: 8, doubled while a group
    would still get about 96 of the row's non-zeros, at most 64; ``forced``
    (8..64) overrides.  Definition of this build (no upstream counterpart)."""
    if forced:
        return forced
    g = N_COLUMN_GROUPS
    while g < 64 and d // (2 * g) >= GROUP_MIN_PIECE:
        g *= 2
    return g


def group_long_rows(indptr, indices, values, threshold=DEG_BOUND, groups=0):
    """Stable partition of the non-zeros of every row with degree > threshold
    (the launch plan's unit size, 384 unless the plan uses smaller units) by
    column_group() into row_groups() groups (``groups`` = 0: chosen per row);
    all other rows are left as they are."""
    indptr = np.asarray(indptr, dtype=np.int64)
    indices = np.array(indices, copy=True)
    values = None if values is None else np.array(values, copy=True)
    for r in np.flatnonzero(np.diff(indptr) > threshold):
        a, b = indptr[r], indptr[r + 1]
        order = np.argsort(column_group(indices[a:b], row_groups(int(b - a), groups)), kind="stable")
        indices[a:b] = indices[a:b][order]
        if values is not None:
            values[a:b] = values[a:b][order]
    return indices, values


def block4_to_bytes(block4):
    """Raw little-endian int32, [deg,row,loc,info] interleaved per block
    (block_level_partition.py:105-106)."""
    return np.ascontiguousarray(block4, dtype="<i4").tobytes()
