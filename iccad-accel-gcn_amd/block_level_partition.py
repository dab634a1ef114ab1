"""The block-level partition stage, driven through the C ABI.

Counterpart of upstream's block_level_partition.py script: for every
``<graphs>/<stem>.config`` it reads ``<stem>.new_indptr`` (raw int32, rows
already in ascending-degree order, :31-32), partitions it and writes
``<out>/<stem>.block4`` as interleaved little-endian int32 quadruples
(degree, row_begin, loc_begin, info) (:105-106).  The partition itself runs as
HIP kernels (``accel_partition_gpu``); ``backend="host"`` selects the library's
explicit host routine instead (``accel_partition_host``) and is never chosen
implicitly.

CLI:  python -m ... block_level_partition [--graphs ./graphs] [--out ./block_level_meta]
"""
from __future__ import annotations

import argparse
import ctypes as C
from pathlib import Path

import numpy as np

from . import _lib
from ._lib import check, lib, ptr


def partition(indptr, backend: str = "gpu") -> np.ndarray:
    """block4 metadata [B, 4] (int32) for the row order given."""
    ip = _lib.as_i32(indptr)
    if ip.ndim != 1 or ip.size < 1:
        raise _lib.AccelError(_lib.ERR_ARG, "indptr must be a 1-D array with at least one entry")
    fn = {"gpu": lib().accel_partition_gpu, "host": lib().accel_partition_host}[backend]
    n = C.c_int64(0)
    rows = ip.size - 1
    # size: at most one block per row plus one per 384 non-zeros
    cap = rows + int(ip[-1]) // _lib.DEG_BOUND + 1 if rows else 0
    out = np.empty((max(cap, 1), 4), dtype=np.int32)
    check(fn(ptr(ip, C.c_int32), rows, ptr(out, C.c_int32), cap, C.byref(n)))
    if n.value > cap:
        raise _lib.AccelError(_lib.ERR_META, f"partition produced {n.value} blocks, capacity {cap}")
    return out[: n.value].copy()


def degree_sort(indptr) -> np.ndarray:
    """perm[new_row] = old_row, ascending degree, ties by row id (host routine)."""
    ip = _lib.as_i32(indptr)
    perm = np.empty(ip.size - 1, dtype=np.int32)
    check(lib().accel_degree_sort_host(ptr(ip, C.c_int32), ip.size - 1, ptr(perm, C.c_int32)))
    return perm


def write_block4(path, block4) -> None:
    b = np.ascontiguousarray(block4, dtype="<i4").reshape(-1)
    check(lib().accel_file_write(str(path).encode(), ptr(b), b.size))


def read_raw_i32(path) -> np.ndarray:
    n = C.c_int64(0)
    check(lib().accel_file_count(str(path).encode(), C.byref(n)))
    out = np.empty(n.value, dtype=np.int32)
    check(lib().accel_file_read(str(path).encode(), ptr(out), n.value))
    return out


def run_stage(graphs_dir="./graphs/", out_dir="./block_level_meta/", backend="gpu", verbose=True):
    """Partition every graph that has a ``.config`` file; returns {stem: n_blocks}."""
    graphs_dir, out_dir = Path(graphs_dir), Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    done = {}
    for cfg in sorted(graphs_dir.glob("*.config")):
        stem = cfg.stem
        indptr = read_raw_i32(graphs_dir / f"{stem}.new_indptr")
        b4 = partition(indptr, backend=backend)
        write_block4(out_dir / f"{stem}.block4", b4)
        done[stem] = b4.shape[0]
        if verbose:
            print(stem)
            print(indptr.size - 1, int(indptr[-1]))
    return done


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--graphs", default="./graphs/")
    ap.add_argument("--out", default="./block_level_meta/")
    ap.add_argument("--backend", choices=("gpu", "host"), default="gpu")
    a = ap.parse_args(argv)
    run_stage(a.graphs, a.out, a.backend)


if __name__ == "__main__":
    main()
