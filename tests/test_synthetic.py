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


def test_packaged_degree_sequences_are_the_golden_ones(pkg):
    """data/upstream_degrees.json against the golden .block4 files it was read from."""
    import block4_codec
    from oracle import partition_oracle as po
    assert pkg.synthetic.upstream_graph_names() == block4_codec.names()
    for name in block4_codec.names():
        want = np.sort(po.degrees_from_block4(block4_codec.load(name)))
        assert np.array_equal(pkg.synthetic.upstream_degree_sequence(name), want), name


def test_fixture_graphs_keep_the_degree_sequence(pkg):
    """fixture:<g> and local:<g>:<sigma> workloads: the degree sequence is the one upstream's
    .block4 file of <g> encodes; local columns stay near the row id."""
    syn = pkg.synthetic
    want = syn.upstream_degree_sequence("pubmed")
    g = syn.workload("fixture:pubmed")
    well_formed(g)
    # duplicates inside a row merge, so a row may fall slightly short of its target degree
    got = np.sort(np.diff(g.indptr))
    assert got.size == want.size and np.all(got <= want) and got.sum() >= 0.999 * want.sum()
    loc = syn.workload("local:pubmed:50")
    well_formed(loc)
    rows = np.repeat(np.arange(loc.n_rows), np.diff(loc.indptr))
    assert np.percentile(np.abs(loc.indices - rows), 99) <= 3 * 50 + 1
    assert np.abs(g.indices - np.repeat(np.arange(g.n_rows), np.diff(g.indptr))).mean() > 1000
    with pytest.raises(ValueError):
        syn.workload("nothing:1")


def test_uniform_probe_graph(pkg):
    g = pkg.synthetic.workload("uniform:1000:7:300")
    assert g.n_rows == 1000 and g.n_cols == 300 and g.nnz == 7000
    assert np.all(np.diff(g.indptr) == 7) and g.indices.min() >= 0 and g.indices.max() < 300


def test_bench_workload_cache_and_traffic_record(pkg, tmp_path):
    """bench.py keeps generated workloads between runs, and reports recorded HBM traffic only
    when it was taken with the kernel sources that are running."""
    import json
    import os
    bench = _bench_module()
    g1, cached1 = bench.load_workload(pkg.synthetic, "cfg1", str(tmp_path))
    g2, cached2 = bench.load_workload(pkg.synthetic, "cfg1", str(tmp_path))
    assert not cached1 and cached2
    assert np.array_equal(g1.indptr, g2.indptr) and np.array_equal(g1.indices, g2.indices)
    assert np.array_equal(g1.values, g2.values) and (g1.n_rows, g1.n_cols) == (g2.n_rows, g2.n_cols)
    assert bench.load_workload(pkg.synthetic, "cfg1", "")[1] is False
    # every committed traffic entry names the sources it was measured with
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    entries = json.load(open(os.path.join(root, "profiles", "spmm_gather_traffic.json")))
    now = bench.kernel_source_hash()
    assert len(now) == 16
    for key, e in entries.items():
        if key.startswith("_"):
            continue
        wl, n = key.rsplit("/N", 1)
        value, note = bench.recorded_traffic(wl, int(n))
        if e.get("source_sha16") == now:
            assert value == e and note is None and value["traffic_bytes"] > 0 and 0 < value["l2_hit_rate"] < 1
        else:
            assert value is None and "taken with kernel sources" in note
    assert bench.recorded_traffic("cfg1", 7) == (None, "this workload was not profiled")
    # the ceilings of the bench line: the probe's two rates come from the same committed file
    rates = bench.probe_rates(64)
    assert rates == entries["_probe_rates_GBps"]["N64"] and bench.probe_rates(16) == entries["_probe_rates_GBps"]["N16"]
    assert bench.probe_rates(100) == rates and bench.probe_rates(20) == entries["_probe_rates_GBps"]["N32"]
    alg, delivered = 2_256_466_672, 125_258_334 * 64 * 4          # the headline workload
    all_hits, at_rate = bench.ceilings(alg, delivered, 0.3057, rates)
    assert abs(all_hits - 0.234) < 5e-4 and abs(at_rate - 0.0815) < 5e-4
    assert bench.ceilings(alg, delivered, 1.0, rates)[1] == pytest.approx(all_hits)
    assert bench.ceilings(alg, delivered, None, rates) == (all_hits, None)
    assert bench.ceilings(alg, delivered, 0.3, None) == (None, None)


def test_export_in_upstreams_layout(pkg, tmp_path):
    """<name>.config / .new_indptr / .new_indices: degree-sorted rows, raw int32, the same matrix."""
    from oracle import partition_oracle as po
    syn = pkg.synthetic
    g = syn.workload("fixture:pubmed")
    name = syn.export_upstream_layout(g, tmp_path / "graphs")
    assert name == "pubmed" and (tmp_path / "graphs" / "pubmed.config").exists()
    ip = np.fromfile(tmp_path / "graphs" / "pubmed.new_indptr", dtype="<i4")
    ix = np.fromfile(tmp_path / "graphs" / "pubmed.new_indices", dtype="<i4")
    perm = po.degree_sort(g.indptr)
    sip, six, _ = po.permute_csr(g.indptr, g.indices, g.values, perm)
    assert np.array_equal(ip, sip) and np.array_equal(ix, six)
    assert np.all(np.diff(np.diff(ip)) >= 0)


def test_columns_by_popularity_is_the_same_matrix(pkg):
    syn = pkg.synthetic
    g = syn.cfg1()
    p = syn.workload("bypopularity:cfg1")
    count = np.bincount(p.indices, minlength=p.n_cols)
    assert np.all(np.diff(count) <= 0)                     # column 0 is the most referenced
    # the same product once X is permuted the same way
    X = syn.dense_operand("cfg1", g.n_cols, 4)
    old_count = np.bincount(g.indices, minlength=g.n_cols)
    order = np.argsort(-old_count, kind="stable")
    Y0 = so.csr(g.indptr, g.indices, g.values, g.n_cols) @ X
    Y1 = so.csr(p.indptr, p.indices, p.values, p.n_cols) @ X[order]
    assert np.allclose(Y0, Y1, rtol=1e-5, atol=1e-6)
