"""Shared builders for the tests (inputs only; no product code paths)."""
from __future__ import annotations

import numpy as np

import __graft_entry__ as entry
from oracle import partition_oracle as po


def package():
    return entry.load_package()


def degree_mix(seed=0, n_long=3, zeros=5, shuffle=True):
    """Row degrees that hit every regime of the partition rule: zeros, each
    slice-table boundary, 192..384 (one row per block), exact multiples of 384
    and a few long rows."""
    rng = np.random.default_rng(seed)
    deg = [0] * zeros
    for d in (1, 2, 3, 12, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 160, 191, 192, 193,
              256, 383, 384):
        deg += [d] * int(rng.integers(1, 15))
    deg += [1] * 40 + [2] * 30 + [5] * 13
    deg += [385, 768, 1152, 1000][:n_long] if n_long <= 4 else [385, 768, 1152, 1000] + list(
        rng.integers(400, 3000, n_long - 4))
    deg = np.asarray(deg, dtype=np.int64)
    if shuffle:
        deg = rng.permutation(deg)
    return deg


def graph_from_degrees(deg, n_cols=None, seed=0, value_mode="uniform"):
    pkg = package()
    deg = np.asarray(deg, dtype=np.int64)
    n_cols = int(n_cols or max(int(deg.max(initial=1)) + 7, deg.size))
    return pkg.synthetic.random_csr(deg.size, n_cols, deg, seed=seed, value_mode=value_mode)


def expected_preprocess(indptr, indices, values, unit=384, groups=0):
    """(perm, sorted indptr/indices/values, block4) from the CPU oracle; ``unit`` is
    the launch plan's unit size (rows above it are stored grouped by column group)."""
    perm = po.degree_sort(indptr)
    sip, six, sval = po.permute_csr(indptr, indices, values, perm)
    six, sval = po.group_long_rows(sip, six, sval, unit, groups)
    return perm, sip, six, sval, po.partition_closed_form(sip)
