"""The comparison baselines (rocSPARSE CSR SpMM, neighbour-partition kernel with
atomics) compute the same product as the operator, so their timings compare like
with like.  They live in their own library and are never part of the operator."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers
from oracle import spmm_oracle as so

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def baselines(gpu):
    path = os.path.join(os.path.dirname(str(gpu._lib.LIB_PATH)), "libaccelgcn_baselines.so")
    assert os.path.exists(path), "baselines library not built (run __graft_entry__.build())"
    L = C.CDLL(path)
    L.baseline_last_error.restype = C.c_char_p
    L.baseline_neighbor_partition_last_error.restype = C.c_char_p
    return L


@pytest.mark.parametrize("N", [16, 64, 100])
def test_neighbor_partition_baseline_computes_the_product(gpu, baselines, N):
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=3, n_long=4, zeros=5), seed=3)
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    bufs = [gpu.DeviceBuffer.from_numpy(a) for a in (g.indices, g.values, X)]
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    dY.fill_u32(0x7FC00000)                                  # NaN: the baseline must clear it itself
    ms = (C.c_float * 3)()
    pre, parts = C.c_float(0), C.c_int64(0)
    indptr = np.ascontiguousarray(g.indptr, dtype=np.int32)
    rc = baselines.baseline_neighbor_partition_spmm(
        indptr.ctypes.data_as(C.c_void_p), C.c_void_p(bufs[0].address), C.c_void_p(bufs[1].address),
        C.c_int64(g.n_rows), C.c_int64(g.nnz), C.c_void_p(bufs[2].address), C.c_void_p(dY.address),
        C.c_int32(N), 0, 1, 3, ms, C.byref(pre), C.byref(parts))
    assert rc == 0, baselines.baseline_neighbor_partition_last_error().decode()
    ps = max(1, g.nnz // g.n_rows)
    assert parts.value == int(np.sum(-(-np.diff(g.indptr.astype(np.int64)) // ps)))   # spmm_gnna.cu:27-33
    Y = dY.to_numpy(np.float32, (g.n_rows, N))
    assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL
    assert all(t > 0 for t in ms)
    for b in bufs + [dY]:
        b.close()


def test_rocsparse_baseline_computes_the_product(gpu, baselines):
    N = 32
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=4, n_long=2), seed=4)
    X = np.random.default_rng(4).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    bufs = [gpu.DeviceBuffer.from_numpy(a) for a in (g.indptr, g.indices, g.values, X)]
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    ms = (C.c_float * 2)()
    pre = C.c_float(0)
    rc = baselines.baseline_rocsparse_spmm(
        C.c_void_p(bufs[0].address), C.c_void_p(bufs[1].address), C.c_void_p(bufs[2].address),
        C.c_int64(g.n_rows), C.c_int64(g.n_cols), C.c_int64(g.nnz), C.c_void_p(bufs[3].address),
        C.c_void_p(dY.address), C.c_int32(N), 0, 1, 2, ms, C.byref(pre))
    assert rc == 0, baselines.baseline_last_error().decode()
    Y = dY.to_numpy(np.float32, (g.n_rows, N))
    assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL
    for b in bufs + [dY]:
        b.close()


def test_gather_probe_runs(gpu, baselines):
    """The pure-gather measurement probe: argument checks and a small run."""
    baselines.baseline_gather_probe_last_error.restype = C.c_char_p
    ms, gathered, stored = C.c_float(0), C.c_double(0), C.c_double(0)
    for stores in (0, 1, 2):
        rc = baselines.baseline_gather_probe(C.c_int64(1000), C.c_int32(64), C.c_int32(8), C.c_int32(4),
                                             C.c_int32(stores), C.c_int32(1), C.byref(ms), C.byref(gathered),
                                             C.byref(stored))
        assert rc == 0, baselines.baseline_gather_probe_last_error().decode()
        assert ms.value > 0 and gathered.value == 65536 * 4 * 8 * 256.0
        assert (stored.value > 0) == (stores != 0)
    assert baselines.baseline_gather_probe(C.c_int64(1000), C.c_int32(48), C.c_int32(8), C.c_int32(4), C.c_int32(0),
                                           C.c_int32(1), C.byref(ms), None, None) != 0      # N must be 16, 64 or 256


def test_rocblas_baseline_computes_the_dense_product(gpu, baselines):
    baselines.baseline_rocblas_last_error.restype = C.c_char_p
    rng = np.random.default_rng(8)
    rows, K, N = 1000, 48, 40
    X = rng.uniform(-1, 1, (rows, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    dX, dW, dZ = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(W), gpu.DeviceBuffer(rows * N * 4)
    ms, queued = (C.c_float * 2)(), C.c_float(0)
    rc = baselines.baseline_rocblas_sgemm(C.c_void_p(dX.address), C.c_void_p(dW.address), C.c_void_p(dZ.address),
                                          C.c_int64(rows), C.c_int32(K), C.c_int32(N), 1, 2, ms, C.byref(queued))
    assert rc == 0, baselines.baseline_rocblas_last_error().decode()
    assert so.check_dense(dZ.to_numpy(np.float32, (rows, N)), X, W) <= so.TOL
    assert all(t > 0 for t in ms) and queued.value > 0
    for b in (dX, dW, dZ):
        b.close()
