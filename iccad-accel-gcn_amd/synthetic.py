"""Seeded synthetic graphs and dense operands for the five benchmark workloads.

The upstream datasets (graphs/*.new_indptr, *.new_indices; README.md:44-53) are
a download and are not available offline, so every workload is generated here
with ``numpy.random.default_rng``.  All graphs come out as CSR with int32
``indptr``/``indices`` (columns sorted and unique within a row) and fp32 values.
Row ids are shuffled so that the degree sort has real work to do.

Directed power-law graphs are Chung-Lu by edge sampling: every edge draws its
source and its destination independently with probability proportional to the
node weight w_i = c * (rank_i + i0) ** (-1 / (gamma - 1)); c and i0 are solved
so that the weights sum to the requested edge count and the largest weight is
the requested maximum degree.  Duplicate edges are merged, so nnz is whatever
the generator yields (it is reported, never assumed).

GCN normalisation: val_ij = 1 / sqrt(d_i * d_j) where d is the row degree of
the matrix being normalised (self-loops included when they are added).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

GRAPH_SEED = 0
X_SEED = 1


@dataclass
class Graph:
    name: str
    indptr: np.ndarray      # int32 [rows + 1]
    indices: np.ndarray     # int32 [nnz]
    values: np.ndarray      # float32 [nnz]
    n_rows: int
    n_cols: int

    @property
    def nnz(self) -> int:
        return int(self.indptr[-1])


# ----------------------------------------------------------------------------
# power-law weights with an analytic inverse CDF
# ----------------------------------------------------------------------------
def _solve_i0(n, total, w_max, alpha):
    """i0 such that c*(i+i0)^-alpha sums (integral) to ``total`` with w_0 = w_max."""
    def peak(i0):
        e = 1.0 - alpha
        integral = ((n + i0) ** e - i0 ** e) / e
        return total / integral * i0 ** (-alpha)
    lo, hi = 1e-3, float(n)
    for _ in range(200):
        mid = (lo * hi) ** 0.5
        if peak(mid) > w_max:
            lo = mid
        else:
            hi = mid
    return (lo * hi) ** 0.5


def _draw_ranks(rng, count, n, i0, alpha, chunk=1 << 24):
    """``count`` node ranks in [0, n) with P(i) ~ integral_i^{i+1} (x+i0)^-alpha dx."""
    e = 1.0 - alpha
    a, b = i0 ** e, (n + i0) ** e
    out = np.empty(count, dtype=np.int64)
    for s in range(0, count, chunk):
        u = rng.random(min(chunk, count - s))
        x = (a + u * (b - a)) ** (1.0 / e) - i0
        np.clip(x, 0, n - 1, out=x)
        out[s:s + u.size] = x.astype(np.int64)
    return out


def _csr_from_edges(src, dst, n_rows, n_cols):
    """Merge duplicates, sort columns inside rows; returns int32 indptr, indices."""
    key = (src.astype(np.int64) << 32) | dst.astype(np.int64)
    del src, dst
    key.sort(kind="stable")
    if key.size:
        keep = np.ones(key.size, dtype=bool)
        keep[1:] = key[1:] != key[:-1]
        key = key[keep]
    rows = (key >> 32).astype(np.int64)
    cols = (key & 0xFFFFFFFF).astype(np.int32)
    counts = np.bincount(rows, minlength=n_rows)
    indptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(counts, out=indptr[1:])
    assert indptr[-1] < 2 ** 31, "nnz does not fit int32"
    return indptr.astype(np.int32), cols


def _gcn_values(indptr, indices):
    deg = np.diff(indptr).astype(np.float64)
    inv = 1.0 / np.sqrt(np.maximum(deg, 1.0))
    rows = np.repeat(np.arange(deg.size), np.diff(indptr))
    return (inv[rows] * inv[indices]).astype(np.float32)


def _with_self_loops(src, dst, n):
    loop = np.arange(n, dtype=np.int64)
    return np.concatenate([src, loop]), np.concatenate([dst, loop])


def chung_lu_directed(name, n, n_edges, gamma, max_degree, seed=GRAPH_SEED, self_loops=True):
    rng = np.random.default_rng(seed)
    alpha = 1.0 / (gamma - 1.0)
    i0 = _solve_i0(n, n_edges, max_degree, alpha)
    relabel = rng.permutation(n)
    src = relabel[_draw_ranks(rng, n_edges, n, i0, alpha)]
    dst = relabel[_draw_ranks(rng, n_edges, n, i0, alpha)]
    if self_loops:
        src, dst = _with_self_loops(src, dst, n)
    indptr, indices = _csr_from_edges(src, dst, n, n)
    return Graph(name, indptr, indices, _gcn_values(indptr, indices), n, n)


# ----------------------------------------------------------------------------
# the five workloads
# ----------------------------------------------------------------------------
def cfg1(seed=GRAPH_SEED):
    """10,000 nodes, ~100k undirected edges, Chung-Lu gamma=2.5, symmetrised,
    self-loops, GCN-normalised."""
    n, e, gamma = 10_000, 100_000, 2.5
    rng = np.random.default_rng(seed)
    alpha = 1.0 / (gamma - 1.0)
    i0 = _solve_i0(n, 2 * e, 400, alpha)
    relabel = rng.permutation(n)
    u = relabel[_draw_ranks(rng, e, n, i0, alpha)]
    v = relabel[_draw_ranks(rng, e, n, i0, alpha)]
    keep = u != v
    u, v = u[keep], v[keep]
    src, dst = _with_self_loops(np.concatenate([u, v]), np.concatenate([v, u]), n)
    indptr, indices = _csr_from_edges(src, dst, n, n)
    return Graph("cfg1", indptr, indices, _gcn_values(indptr, indices), n, n)


def cfg2(seed=GRAPH_SEED):
    """170,000 nodes, ~2.3M directed edges, gamma=2.3, max degree ~15k, self-loops."""
    return chung_lu_directed("cfg2", 170_000, 2_300_000, 2.3, 24_000, seed)


def cfg3(seed=GRAPH_SEED, n=233_000, scale=1.0):
    """233,000 nodes, ~114M edges, lognormal degree (mu=5.5, sigma=1.2) capped at
    21,000; destinations drawn proportionally to the same degree weights;
    val = 1/sqrt(d_i d_j), no self-loops.  ``scale`` < 1 shrinks the degrees
    (tests use it; the benchmark uses 1)."""
    rng = np.random.default_rng(seed)
    want = np.minimum(rng.lognormal(5.5, 1.2, n) * scale, 21_000 * scale)
    want = np.maximum(np.rint(want), 1).astype(np.int64)
    cdf = np.cumsum(want / want.sum())
    cdf[-1] = 1.0
    src = np.repeat(np.arange(n, dtype=np.int64), want)
    dst = np.empty(src.size, dtype=np.int64)
    for s in range(0, src.size, 1 << 24):
        u = rng.random(min(1 << 24, src.size - s))
        dst[s:s + u.size] = np.searchsorted(cdf, u, side="right")
    np.clip(dst, 0, n - 1, out=dst)
    indptr, indices = _csr_from_edges(src, dst, n, n)
    return Graph("cfg3", indptr, indices, _gcn_values(indptr, indices), n, n)


def cfg4(seed=GRAPH_SEED, n=2_450_000, n_edges=124_000_000, max_degree=17_000):
    """2.45M nodes, ~124M directed edges, gamma=2.1, mean degree ~50, max ~17k,
    self-loops, GCN-normalised."""
    g = chung_lu_directed("cfg4", n, n_edges, 2.1, max_degree, seed)
    return g


def cfg5(seed=GRAPH_SEED, n=1_000_000, n_hubs=64, hub_lo=50_000, hub_hi=200_000,
         tail_edges=25_500_000):
    """1M nodes: 64 hub rows with 50k-200k neighbours each, every other row has a
    Zipf(1.8) degree (more than half of them degree 1) truncated so that the
    tail holds ~22M edges; destinations follow a rank**-0.8 popularity with the
    hubs as the most popular nodes; val ~ U(0,1]."""
    rng = np.random.default_rng(seed)
    # truncated Zipf(1.8): pick the cut-off K that gives the wanted mean degree
    want_mean = tail_edges / (n - n_hubs)
    ks = np.arange(1, 2_000_001, dtype=np.float64)
    pmf_all = ks ** -1.8
    mean_k = np.cumsum(ks * pmf_all) / np.cumsum(pmf_all)
    K = int(np.searchsorted(mean_k, want_mean)) + 1
    K = min(K, hub_lo - 1, n // 4)
    cdf = np.cumsum(pmf_all[:K] / pmf_all[:K].sum())
    cdf[-1] = 1.0
    deg = np.searchsorted(cdf, rng.random(n), side="right").astype(np.int64) + 1
    relabel = rng.permutation(n)            # rank -> node id; ranks 0..63 are the hubs
    hubs = relabel[:n_hubs]
    deg[hubs] = rng.integers(hub_lo, hub_hi + 1, n_hubs)
    alpha = 0.8
    i0 = 1.0
    is_hub = np.zeros(n, dtype=bool)
    is_hub[hubs] = True
    tail_deg = np.where(is_hub, 0, deg)
    src = [np.repeat(np.arange(n, dtype=np.int64), tail_deg)]
    dst = [relabel[_draw_ranks(rng, src[0].size, n, i0, alpha)]]
    for h in hubs:                          # hubs keep their full, distinct neighbour count
        d = int(deg[h])
        cols = np.unique(_draw_ranks(rng, 3 * d, n, i0, alpha))
        while cols.size < d:
            cols = np.unique(np.concatenate([cols, _draw_ranks(rng, 3 * d, n, i0, alpha)]))
        cols = rng.permutation(cols)[:d]
        src.append(np.full(d, h, dtype=np.int64))
        dst.append(relabel[cols])
    src, dst = np.concatenate(src), np.concatenate(dst)
    indptr, indices = _csr_from_edges(src, dst, n, n)
    values = (1.0 - rng.random(indices.size, dtype=np.float32)).astype(np.float32)
    return Graph("cfg5", indptr, indices, values, n, n)


def hub_graph_small(seed=GRAPH_SEED, n=6_000, n_hubs=4, hub_lo=900, hub_hi=2_500, tail_edges=30_000):
    """A few-thousand-row graph with the shape of cfg5 (hubs that span several
    384-non-zero segments, a majority of degree-1 rows); for parity tests."""
    g = cfg5(seed, n=n, n_hubs=n_hubs, hub_lo=hub_lo, hub_hi=hub_hi, tail_edges=tail_edges)
    g.name = "hub_small"
    return g


# ----------------------------------------------------------------------------
# graphs with the degree sequences of upstream's own benchmark set
# ----------------------------------------------------------------------------
def upstream_graph_names():
    return sorted(_upstream_degrees())


def _upstream_degrees():
    import json
    from pathlib import Path
    return json.loads((Path(__file__).resolve().parent / "data" / "upstream_degrees.json").read_text())


def upstream_degree_sequence(name):
    """Row degrees (ascending) of one of upstream's 16 published graphs (README.md:42
    lists them), as its block_level_meta/<name>.block4 file encodes them."""
    runs = np.asarray(_upstream_degrees()[name], dtype=np.int64)
    return np.repeat(runs[:, 0], runs[:, 1])


def fixture_graph(name, seed=0, sigma=0):
    """A graph with exactly the degree sequence of one of upstream's benchmark graphs, rows
    in shuffled order, values GCN-normalised.  The real edge lists are a download that is
    not available offline, so the columns are synthetic: uniform random (sigma = 0), or,
    to model a vertex order with locality, row id + N(0, sigma) (duplicates inside a row
    merge, so such a graph has slightly fewer non-zeros)."""
    deg = upstream_degree_sequence(name)
    n = deg.size
    rng = np.random.default_rng(seed)
    deg = rng.permutation(deg)
    src = np.repeat(np.arange(n, dtype=np.int64), deg)
    if sigma > 0:
        dst = np.clip(src + np.rint(rng.standard_normal(src.size) * sigma).astype(np.int64), 0, n - 1)
    else:
        dst = rng.integers(0, n, size=src.size, dtype=np.int64)
    indptr, indices = _csr_from_edges(src, dst, n, n)
    return Graph(name, indptr, indices, _gcn_values(indptr, indices), n, n)


def uniform_graph(n_rows, degree, n_cols, seed=0):
    """Every row has `degree` non-zeros with columns uniform over n_cols (repeats
    allowed): a probe of the gather rate for an X of a chosen size."""
    rng = np.random.default_rng(seed)
    indptr = (np.arange(n_rows + 1, dtype=np.int64) * degree).astype(np.int32)
    indices = rng.integers(0, n_cols, size=n_rows * degree).astype(np.int32)
    values = rng.random(n_rows * degree, dtype=np.float32)
    return Graph(f"uniform:{n_rows}:{degree}:{n_cols}", indptr, indices, values, n_rows, n_cols)


def columns_by_popularity(g):
    """The same matrix with its columns renumbered by descending number of non-zeros (the
    most referenced column becomes column 0): what a caller would get by ordering the rows
    of X by popularity.  Columns inside a row are left in the order of the old numbering."""
    count = np.bincount(g.indices, minlength=g.n_cols)
    order = np.argsort(-count, kind="stable")                  # new id -> old id
    new_of_old = np.empty(g.n_cols, dtype=np.int32)
    new_of_old[order] = np.arange(g.n_cols, dtype=np.int32)
    return Graph("bypopularity:" + g.name, g.indptr, new_of_old[g.indices], g.values, g.n_rows, g.n_cols)


def workload(spec):
    """cfg1..cfg5, fixture:<name>, local:<name>:<sigma>, uniform:<rows>:<degree>:<cols>, or
    bypopularity:<any of these> for the same matrix with columns renumbered by popularity."""
    if spec in WORKLOADS:
        return WORKLOADS[spec]()
    kind, _, rest = spec.partition(":")
    if kind == "bypopularity":
        return columns_by_popularity(workload(rest))
    if kind == "fixture":
        return fixture_graph(rest)
    if kind == "local":
        name, sigma = rest.rsplit(":", 1)
        return fixture_graph(name, sigma=int(sigma))
    if kind == "uniform":
        n_rows, degree, n_cols = (int(v) for v in rest.split(":"))
        return uniform_graph(n_rows, degree, n_cols)
    raise ValueError(f"unknown workload {spec}")


def export_upstream_layout(spec_or_graph, graphs_dir, name=None):
    """Write a workload the way upstream's programs read their datasets (main.cu:62-65,
    block_level_partition.py:26-32): ``<name>.config`` (presence only), ``<name>.new_indptr``
    and ``<name>.new_indices`` as raw little-endian int32, rows in ascending degree order
    (ties keep their order), and ``<name>.graph.ptrdump`` / ``<name>.graph.edgedump``, the
    same matrix with its rows in the workload's own order (column ids are the same in both
    pairs).  Values are not part of the layout (upstream fills ones, main.cu:114).  The
    adjacency must be square.  Returns the stem written."""
    from pathlib import Path
    g = workload(spec_or_graph) if isinstance(spec_or_graph, str) else spec_or_graph
    if g.n_rows != g.n_cols:
        raise ValueError("upstream's layout assumes a square adjacency")
    name = name or g.name.replace(":", "-")
    deg = np.diff(g.indptr).astype(np.int64)
    perm = np.argsort(deg, kind="stable")
    sip = np.zeros(g.n_rows + 1, dtype=np.int64)
    np.cumsum(deg[perm], out=sip[1:])
    # gather the rows in the new order
    starts = g.indptr[:-1].astype(np.int64)[perm]
    src = np.repeat(starts - sip[:-1], deg[perm]) + np.arange(int(sip[-1]), dtype=np.int64)
    out = Path(graphs_dir)
    out.mkdir(parents=True, exist_ok=True)
    (out / f"{name}.config").write_text("")
    sip.astype("<i4").tofile(out / f"{name}.new_indptr")
    g.indices[src].astype("<i4").tofile(out / f"{name}.new_indices")
    np.asarray(g.indptr).astype("<i4").tofile(out / f"{name}.graph.ptrdump")
    np.asarray(g.indices).astype("<i4").tofile(out / f"{name}.graph.edgedump")
    return name


WORKLOADS = {"cfg1": cfg1, "cfg2": cfg2, "cfg3": cfg3, "cfg4": cfg4, "cfg5": cfg5}
# column counts each workload is swept over; the first entry is the default
WORKLOAD_N = {"cfg1": (32,), "cfg2": (64, 16, 32, 128), "cfg3": (64, 32, 128),
              "cfg4": (64, 16, 100), "cfg5": (256,)}


def dense_operand(name, n_rows, n_cols, seed=X_SEED):
    """X for a workload: N(0,1) for cfg5, U[-1,1] otherwise; fp32, C-contiguous."""
    rng = np.random.default_rng(seed)
    if name == "cfg5" or name == "hub_small":
        return rng.standard_normal((n_rows, n_cols), dtype=np.float32)
    x = rng.random((n_rows, n_cols), dtype=np.float32)
    x *= 2.0
    x -= 1.0
    return x


def random_csr(n_rows, n_cols, degrees, seed=0, value_mode="uniform"):
    """Small CSR with prescribed row degrees (tests).  Columns are distinct and
    sorted inside each row."""
    rng = np.random.default_rng(seed)
    degrees = np.minimum(np.asarray(degrees, dtype=np.int64), n_cols)
    indptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(degrees, out=indptr[1:])
    indices = np.empty(indptr[-1], dtype=np.int32)
    for r in range(n_rows):
        d = int(degrees[r])
        if d == 0:
            continue
        if d * 4 > n_cols:
            cols = rng.permutation(n_cols)[:d]
        else:
            cols = np.unique(rng.integers(0, n_cols, size=2 * d + 8))
            while cols.size < d:
                cols = np.unique(np.concatenate([cols, rng.integers(0, n_cols, size=2 * d + 8)]))
            cols = rng.permutation(cols)[:d]
        indices[indptr[r]:indptr[r + 1]] = np.sort(cols)
    if value_mode == "ones":
        values = np.ones(indices.size, dtype=np.float32)
    else:
        values = (rng.random(indices.size, dtype=np.float32) * 2 - 1).astype(np.float32)
    return Graph("random", indptr.astype(np.int32), indices, values, n_rows, n_cols)
