"""Writes iccad-accel-gcn_amd/data/upstream_degrees.json: the degree sequence of each
of the reference's benchmark graphs, as (degree, row count) pairs in ascending degree
order.

The sequences are read out of the golden ``.block4`` metadata kept next to this
script (degree, first row and row count of every block; rows that no block covers
have degree 0).  Run from the repository root:
    python tests/golden/make_upstream_degrees.py
"""
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(Path(__file__).resolve().parent))
import block4_codec  # noqa: E402


def degrees(b):
    b = b.astype(np.int64)
    is_long = b[:, 0] > 384
    first = np.ones(len(b), dtype=bool)
    first[1:] = ~(is_long[1:] & (b[1:, 1] == b[:-1, 1]))      # one entry per long row
    b = b[first]
    n_rows_blk = np.where(b[:, 0] > 384, 1, b[:, 3] & 0xFFFF)
    n = int((b[:, 1] + n_rows_blk).max())
    deg = np.zeros(n, dtype=np.int64)
    start = np.repeat(b[:, 1], n_rows_blk)
    within = np.arange(n_rows_blk.sum()) - np.repeat(np.cumsum(n_rows_blk) - n_rows_blk, n_rows_blk)
    deg[start + within] = np.repeat(b[:, 0], n_rows_blk)
    return deg


def main():
    out = {}
    for name in block4_codec.names():
        d, c = np.unique(degrees(block4_codec.load(name)), return_counts=True)
        out[name] = [[int(a), int(b)] for a, b in zip(d, c)]
    path = ROOT / "iccad-accel-gcn_amd" / "data" / "upstream_degrees.json"
    path.write_text(json.dumps(out, separators=(",", ":")) + "\n")
    print(path, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
