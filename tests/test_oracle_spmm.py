"""Pins the CPU SpMM oracle (scipy product, fp64 scaling, C restatement, and
the emulation of the reference kernel's block4 decomposition)."""
import numpy as np
import pytest

import helpers
from oracle import c_oracle, partition_oracle as po, spmm_oracle as so


def dense_of(g):
    A = np.zeros((g.n_rows, g.n_cols), dtype=np.float64)
    for r in range(g.n_rows):
        for p in range(g.indptr[r], g.indptr[r + 1]):
            A[r, g.indices[p]] += float(g.values[p])
    return A


@pytest.mark.parametrize("seed,N", [(0, 1), (1, 7), (2, 32)])
def test_against_dense_brute_force(seed, N):
    rng = np.random.default_rng(seed)
    g = helpers.graph_from_degrees(rng.integers(0, 12, size=40), n_cols=30, seed=seed)
    X = rng.standard_normal((g.n_cols, N)).astype(np.float32)
    ref = dense_of(g) @ X.astype(np.float64)
    R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
    assert np.allclose(R, ref, rtol=0, atol=1e-12)
    assert np.allclose(S, np.abs(dense_of(g)) @ np.abs(X.astype(np.float64)), rtol=0, atol=1e-12)
    for Y in (so.spmm_scipy32(g.indptr, g.indices, g.values, X),
              c_oracle.spmm_csr_f32(g.indptr, g.indices, g.values, X)):
        assert so.scaled_error(Y, R, S) <= so.TOL
    R2, S2 = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
    assert np.allclose(R2, R, rtol=1e-13, atol=1e-13) and np.allclose(S2, S, rtol=1e-13, atol=1e-13)


def test_closed_forms():
    deg = helpers.degree_mix(seed=1)
    g = helpers.graph_from_degrees(deg, seed=1, value_mode="ones")
    ones = np.ones((g.n_cols, 4), dtype=np.float32)
    for Y in (so.spmm_scipy32(g.indptr, g.indices, g.values, ones),
              c_oracle.spmm_csr_f32(g.indptr, g.indices, g.values, ones)):
        assert np.array_equal(Y, np.repeat(deg[:, None], 4, axis=1).astype(np.float32))
    n = 50                                      # identity matrix returns X
    ip = np.arange(n + 1, dtype=np.int32)
    ix = np.arange(n, dtype=np.int32)
    X = np.random.default_rng(0).standard_normal((n, 5)).astype(np.float32)
    assert np.array_equal(so.spmm_scipy32(ip, ix, np.ones(n, np.float32), X), X)
    assert np.array_equal(c_oracle.spmm_csr_f32(ip, ix, np.ones(n, np.float32), X), X)


def test_c_restatement_matches_scipy_bitwise_order():
    # both accumulate in CSR order in fp32, so they agree to the last bit
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=2), seed=2)
    X = np.random.default_rng(2).uniform(-1, 1, (g.n_cols, 16)).astype(np.float32)
    assert np.array_equal(c_oracle.spmm_csr_f32(g.indptr, g.indices, g.values, X),
                          so.spmm_scipy32(g.indptr, g.indices, g.values, X))


@pytest.mark.parametrize("N", [1, 16, 33])
def test_block4_decomposition_computes_the_product(N):
    """The metadata means what the reference kernel decodes it to mean
    (spmm_accel.cu:21-28,34,47-48): summing the slices it describes gives A X."""
    g = helpers.graph_from_degrees(np.sort(helpers.degree_mix(seed=3)), seed=3)
    X = np.random.default_rng(3).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    b4 = po.partition_closed_form(g.indptr)
    Y = c_oracle.spmm_block4(b4, g.indices, g.values, X, g.n_rows)
    R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
    assert so.scaled_error(Y, R, S) <= so.TOL
    # a corrupted field must be noticed: shift one block's loc_begin
    bad = b4.copy()
    bad[len(bad) // 2, 2] += 1
    Yb = c_oracle.spmm_block4(bad, g.indices, g.values, X, g.n_rows)
    assert so.scaled_error(Yb, R, S) > so.TOL


def test_scaled_error_catches_a_dropped_term():
    g = helpers.graph_from_degrees([50] * 20, n_cols=200, seed=4)
    X = np.random.default_rng(4).uniform(-1, 1, (g.n_cols, 8)).astype(np.float32)
    R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
    v = g.values.copy()
    v[7] = 0.0
    assert so.scaled_error(so.spmm_scipy32(g.indptr, g.indices, v, X), R, S) > 100 * so.TOL
    assert so.scaled_error(so.spmm_scipy32(g.indptr, g.indices, g.values, X), R, S) <= so.TOL


def test_threaded_fp64_oracle_is_the_same_routine_on_row_ranges():
    import helpers
    from oracle import c_oracle
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=1, n_long=20), seed=1)
    X = np.random.default_rng(0).standard_normal((g.n_cols, 20)).astype(np.float32)
    R1, S1 = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
    R2, S2 = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X, threads=5)
    assert np.array_equal(R1, R2) and np.array_equal(S1, S2)
    R3, S3 = c_oracle.spmm_csr_f64(g.indptr[50:201], g.indices, g.values, X, threads=3)   # a slab of rows
    assert np.array_equal(R3, R1[50:200]) and np.array_equal(S3, S1[50:200])


def test_dense_product_oracle():
    rng = np.random.default_rng(5)
    X = rng.standard_normal((9, 6)).astype(np.float32)
    W = rng.standard_normal((6, 4)).astype(np.float32)
    R, S = so.dense_fp64(X, W)
    ref = np.zeros((9, 4)); ref_abs = np.zeros((9, 4))
    for i in range(9):
        for j in range(4):
            for k in range(6):
                ref[i, j] += float(X[i, k]) * float(W[k, j])
                ref_abs[i, j] += abs(float(X[i, k])) * abs(float(W[k, j]))
    assert np.allclose(R, ref, rtol=0, atol=1e-13) and np.allclose(S, ref_abs, rtol=0, atol=1e-13)
    assert np.array_equal(so.dense_fp64(X, np.eye(6, dtype=np.float32))[0], X.astype(np.float64))
    assert np.allclose(so.dense_fp64(X, np.ones((6, 3), np.float32))[0], X.astype(np.float64).sum(1)[:, None])
    assert so.check_dense((X.astype(np.float64) @ W).astype(np.float32), X, W) <= so.TOL
    Wt = W.copy(); Wt[2, 1] = 0.0                          # a dropped term is noticed
    assert so.check_dense((X @ Wt).astype(np.float32), X, W) > 100 * so.TOL
    assert so.check_dense((X[:, ::-1] @ W).astype(np.float32), X, W) > 100 * so.TOL      # a transposed index
