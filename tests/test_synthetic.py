"""The seeded workload generators: shape, determinism, CSR well-formedness."""
import numpy as np
import pytest

from oracle import spmm_oracle as so


def well_formed(g):
    assert g.indptr.dtype == np.int32 and g.indices.dtype == np.int32 and g.values.dtype == np.float32
    assert g.indptr[0] == 0 and g.indptr[-1] == g.indices.size == g.values.size
    d = np.diff(g.indptr)
    assert np.all(d >= 0)
    assert g.indices.min() >= 0 and g.indices.max() < g.n_cols
    rows = np.repeat(np.arange(g.n_rows), d)
    key = rows.astype(np.int64) * g.n_cols + g.indices
    assert np.all(np.diff(key) > 0), "columns must be sorted and unique inside a row"


def test_cfg1_matches_its_description(pkg):
    g = pkg.synthetic.cfg1()
    well_formed(g)
    assert g.n_rows == 10_000 and 190_000 < g.nnz < 215_000
    A = so.csr(g.indptr, g.indices, g.values, g.n_cols)
    assert abs(A - A.T).max() < 1e-7                      # symmetrised
    assert np.all(A.diagonal() > 0)                       # self-loops
    d = np.diff(g.indptr)
    r = 1234
    cols = g.indices[g.indptr[r]:g.indptr[r + 1]]
    expect = 1.0 / np.sqrt(d[r] * d[cols].astype(np.float64))
    assert np.allclose(g.values[g.indptr[r]:g.indptr[r + 1]], expect, rtol=1e-6)
    g2 = pkg.synthetic.cfg1()
    assert np.array_equal(g.indices, g2.indices) and np.array_equal(g.values, g2.values)


def test_cfg2_shape(pkg):
    g = pkg.synthetic.cfg2()
    well_formed(g)
    d = np.diff(g.indptr)
    assert g.n_rows == 170_000 and 2.2e6 < g.nnz < 2.6e6
    assert 8_000 < d.max() < 20_000 and (d > 384).sum() > 50
    assert np.any(np.diff(d) < 0)                         # not degree-sorted on input


def test_hub_graph_small_shape(pkg):
    g = pkg.synthetic.hub_graph_small()
    well_formed(g)
    d = np.diff(g.indptr)
    assert (d > 384).sum() >= 4 and (d == 1).sum() > g.n_rows // 3
    assert g.values.min() > 0 and g.values.max() <= 1


def test_dense_operand(pkg):
    X = pkg.synthetic.dense_operand("cfg2", 100, 16)
    assert X.dtype == np.float32 and X.flags.c_contiguous and X.min() >= -1 and X.max() <= 1
    assert np.array_equal(X, pkg.synthetic.dense_operand("cfg2", 100, 16))
    Z = pkg.synthetic.dense_operand("cfg5", 2000, 8)
    assert abs(Z.mean()) < 0.05 and abs(Z.std() - 1) < 0.05


def _bench_module():
    import importlib.util
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
    spec = importlib.util.spec_from_file_location("bench_under_test", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_bench_fixture_graphs_keep_the_golden_degree_sequence(pkg):
    """bench.py's fixture:<g> and local:<g>:<sigma> workloads: the degree sequence is the one
    the golden .block4 file of <g> encodes; local columns stay near the row id."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import block4_codec
    from oracle import partition_oracle as po
    bench = _bench_module()
    golden = block4_codec.load("pubmed")
    want = np.sort(po.degrees_from_block4(golden))
    g = bench.fixture_graph(pkg, "pubmed")
    well_formed(g)
    # duplicates inside a row merge, so a row may fall slightly short of its target degree
    got = np.sort(np.diff(g.indptr))
    assert got.size == want.size and np.all(got <= want) and got.sum() >= 0.999 * want.sum()
    loc = bench.fixture_graph(pkg, "pubmed", sigma=50)
    well_formed(loc)
    rows = np.repeat(np.arange(loc.n_rows), np.diff(loc.indptr))
    assert np.percentile(np.abs(loc.indices - rows), 99) <= 3 * 50 + 1
    assert np.abs(g.indices - np.repeat(np.arange(g.n_rows), np.diff(g.indptr))).mean() > 1000


def test_bench_uniform_probe_graph(pkg):
    bench = _bench_module()
    g = bench.uniform_graph(pkg, 1000, 7, 300)
    assert g.n_rows == 1000 and g.n_cols == 300 and g.nnz == 7000
    assert np.all(np.diff(g.indptr) == 7) and g.indices.min() >= 0 and g.indices.max() < 300
