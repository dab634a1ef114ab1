"""Z = X W on the fp32 matrix cores (accel_dense_xw) and the GCN layer built from it and
the sparse product, against fp64 products through the C ABI.  Tolerance: the scaled error
of the sparse product's tests, max |Z - R| / |X| |W| <= 1e-5."""
import ctypes as C

import numpy as np
import pytest

import helpers
from oracle import spmm_oracle as so

pytestmark = pytest.mark.gpu

CANARY = np.float32(-12345.5)


def run_dense(gpu, X, W, ldx=0, ldz=0, x_offset=0):
    """Operands placed in larger buffers filled with a canary: X rows ldx apart starting
    x_offset floats into its buffer, Z rows ldz apart with a guard band on both sides."""
    rows, K = X.shape
    N = W.shape[1]
    sx, sz = ldx or K, ldz or N
    xbuf = np.full(x_offset + max(rows, 1) * sx + 8, 7.25, np.float32)
    for r in range(rows):
        xbuf[x_offset + r * sx: x_offset + r * sx + K] = X[r]
    guard = 64
    zbuf = np.full(guard + max(rows, 1) * sz + guard, CANARY, np.float32)
    dX, dW, dZ = gpu.DeviceBuffer.from_numpy(xbuf), gpu.DeviceBuffer.from_numpy(W), gpu.DeviceBuffer.from_numpy(zbuf)
    try:
        gpu.dense_xw(dX.address + 4 * x_offset, dW, dZ.address + 4 * guard, rows, K, N, ldx, ldz)
        gpu._lib.check(gpu.lib().accel_stream_sync(None))
        out = dZ.to_numpy(np.float32, (zbuf.size,))
    finally:
        dX.close(); dW.close(); dZ.close()
    assert np.all(out[:guard] == CANARY) and np.all(out[guard + (rows - 1) * sz + N if rows else guard:] == CANARY), \
        "written outside Z"
    body = out[guard: guard + rows * sz].reshape(rows, sz) if rows else np.zeros((0, sz), np.float32)
    if sz > N and rows:
        pad = body[:-1, N:] if rows > 1 else np.zeros((0, 0))
        assert np.all(pad == CANARY), "padding columns of Z written"
    Z = np.stack([out[guard + r * sz: guard + r * sz + N] for r in range(rows)]) if rows else np.zeros((0, N), np.float32)
    return Z


SHAPES = [(1, 1, 1), (1, 32, 32), (31, 3, 7), (32, 16, 16), (33, 31, 33), (127, 32, 64), (128, 33, 64),
          (129, 64, 100), (300, 100, 128), (257, 128, 130), (500, 200, 256), (1000, 128, 64), (5003, 96, 17),
          (64, 515, 9), (2049, 128, 16), (200, 36, 300), (100, 4, 5), (100, 2, 3), (50, 20, 40), (700, 100, 64)]


@pytest.mark.parametrize("rows,K,N", SHAPES)
def test_dense_product_against_fp64(gpu, rows, K, N):
    rng = np.random.default_rng(rows * 1000 + K * 10 + N)
    X = rng.uniform(-1, 1, (rows, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    Z = run_dense(gpu, X, W)
    assert so.check_dense(Z, X, W) <= so.TOL


@pytest.mark.parametrize("x_offset", [0, 1, 2, 3])
@pytest.mark.parametrize("ldx,ldz", [(0, 0), (132, 72), (129, 65), (128, 64)])
def test_strides_and_alignments(gpu, x_offset, ldx, ldz):
    """Rows of X at every 4-byte alignment (only 16-byte aligned rows take the vector path),
    rows of X and Z with strides; what lies between the rows is neither used nor written."""
    rng = np.random.default_rng(17 + x_offset)
    rows, K, N = 333, 128, 64
    X = rng.uniform(-1, 1, (rows, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    Z = run_dense(gpu, X, W, ldx=ldx, ldz=ldz, x_offset=x_offset)
    assert so.check_dense(Z, X, W) <= so.TOL


def test_closed_forms(gpu):
    rng = np.random.default_rng(3)
    X = rng.standard_normal((777, 48)).astype(np.float32)
    assert np.array_equal(run_dense(gpu, X, np.eye(48, dtype=np.float32)), X)            # identity: exact
    Z = run_dense(gpu, np.ones((100, 37), np.float32), np.ones((37, 5), np.float32))
    assert np.array_equal(Z, np.full((100, 5), 37, np.float32))
    # one non-zero weight picks one column of X, scaled: exact in fp32
    W = np.zeros((48, 70), np.float32); W[13, 69] = 2.0
    Z = run_dense(gpu, X, W)
    assert np.array_equal(Z[:, 69], 2 * X[:, 13]) and not Z[:, :69].any()


def test_a_large_tall_product(gpu):
    """The shape the layer has on a large graph: a million rows, streamed once."""
    rng = np.random.default_rng(11)
    rows, K, N = 1_000_003, 128, 64
    X = rng.uniform(-1, 1, (rows, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    Z = gpu.dense_xw_numpy(X, W)
    idx = np.concatenate([np.arange(0, 4096), rng.integers(0, rows, 20000), np.arange(rows - 4096, rows)])
    assert so.check_dense(Z[idx], X[idx], W) <= so.TOL
    assert np.isfinite(Z).all()
    # column sums of Z = (1^T X) W: every row counted once
    lhs = Z.astype(np.float64).sum(0)
    rhs = X.astype(np.float64).sum(0) @ W.astype(np.float64)
    scale = np.abs(X.astype(np.float64)).sum(0) @ np.abs(W.astype(np.float64))
    assert np.max(np.abs(lhs - rhs) / scale) <= so.TOL


def test_argument_errors(gpu):
    L = gpu.lib()
    X = gpu.DeviceBuffer(64 * 16 * 4); W = gpu.DeviceBuffer(16 * 8 * 4); Z = gpu.DeviceBuffer(64 * 8 * 4)
    E = gpu._lib
    def call(x, w, z, rows, K, N, ldx=0, ldz=0):
        return L.accel_dense_xw(x, w, z, rows, K, N, ldx, ldz, None)
    assert call(X.address, W.address, Z.address, 64, 16, 8) == 0
    assert call(X.address, W.address, Z.address, 0, 16, 8) == 0                          # no rows: nothing to do
    assert call(X.address, W.address, Z.address, -1, 16, 8) == E.ERR_ARG
    assert call(X.address, W.address, Z.address, 64, 0, 8) == E.ERR_ARG
    assert call(X.address, W.address, Z.address, 64, 16, 0) == E.ERR_ARG
    assert call(X.address, W.address, Z.address, 64, 16, 8, 15, 0) == E.ERR_ARG          # ldx < K
    assert call(X.address, W.address, Z.address, 64, 16, 8, 0, 7) == E.ERR_ARG           # ldz < N
    assert call(None, W.address, Z.address, 64, 16, 8) == E.ERR_ARG
    assert call(X.address, W.address, Z.address, 65, 16, 8) == E.ERR_ARG                 # X and Z too small for 65 rows
    assert "needs" in gpu._lib.last_error()
    assert call(X.address, W.address, Z.address, 64, 16, 9) == E.ERR_ARG                 # W too small
    assert call(X.address, W.address, X.address, 64, 16, 8) == E.ERR_ARG                 # Z overlaps X
    assert "overlaps" in gpu._lib.last_error()
    host = np.zeros(64 * 16, np.float32)
    assert call(host.ctypes.data, W.address, Z.address, 64, 16, 8) == E.ERR_ARG      # a host array
    gpu._lib.check(L.accel_stream_sync(None))
    X.close(); W.close(); Z.close()


@pytest.mark.parametrize("K,N,relu,with_bias", [(64, 32, True, True), (100, 64, True, False), (33, 17, False, True)])
def test_gcn_layer(gpu, K, N, relu, with_bias):
    """Y = act(A (X W) + bias) in two launches against the same in fp64."""
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=K, n_long=5, zeros=4), seed=K)
    rng = np.random.default_rng(K)
    X = rng.uniform(-1, 1, (g.n_cols, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32) if with_bias else None
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    layer = gpu.GcnLayer(op, W, b, relu=relu)
    Y = layer.forward_numpy(X)
    # reference in fp64 end to end; the scale multiplies the magnitudes through both products
    Z64, Zabs = so.dense_fp64(X, W)
    R, _ = so.spmm_fp64(g.indptr, g.indices, g.values, Z64)
    _, S = so.spmm_fp64(g.indptr, g.indices, np.abs(g.values), Zabs)
    if b is not None:
        R = R + b.astype(np.float64); S = S + np.abs(b.astype(np.float64))
    if relu:
        R = np.maximum(R, 0)
    # two roundings of an fp32 chain: twice the single-product bound
    assert so.scaled_error(Y, R, S) <= 2 * so.TOL
    layer.close(); op.close()


def test_dense_product_in_a_captured_graph(gpu):
    """The launch allocates nothing and asks nothing of a capturing stream."""
    hip = C.CDLL("libamdhip64.so.7")
    for name in ("hipStreamCreate", "hipStreamDestroy", "hipStreamSynchronize", "hipStreamBeginCapture",
                 "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch", "hipGraphExecDestroy", "hipGraphDestroy"):
        getattr(hip, name).restype = C.c_int
    rng = np.random.default_rng(21)
    rows, K, N = 4000, 64, 64
    X = rng.uniform(-1, 1, (rows, K)).astype(np.float32)
    W = rng.standard_normal((K, N)).astype(np.float32)
    dX, dW, dZ = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(W), gpu.DeviceBuffer(rows * N * 4)
    s = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(s)) == 0
    graph, ex = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(s, 0) == 0
    gpu.dense_xw(dX, dW, dZ, rows, K, N, stream=s.value)
    assert hip.hipStreamEndCapture(s, C.byref(graph)) == 0
    assert hip.hipGraphInstantiate(C.byref(ex), graph, None, None, 0) == 0
    for rep in range(3):
        X2 = (X * (rep + 1)).astype(np.float32)
        gpu._lib.check(gpu.lib().accel_memcpy_h2d(dX.address, X2.ctypes.data, X2.nbytes))
        dZ.fill_u32(0x7FC00000)
        gpu._lib.check(gpu.lib().accel_stream_sync(None))
        assert hip.hipGraphLaunch(ex, s) == 0
        assert hip.hipStreamSynchronize(s) == 0
        assert so.check_dense(dZ.to_numpy(np.float32, (rows, N)), X2, W) <= so.TOL
    hip.hipGraphExecDestroy(ex); hip.hipGraphDestroy(graph); hip.hipStreamDestroy(s)
    dX.close(); dW.close(); dZ.close()


def test_layer_and_wrapper_argument_errors(gpu):
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=5, n_long=1), seed=5)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    W = np.ones((8, 4), np.float32)
    with pytest.raises(gpu.AccelError):
        gpu.GcnLayer(op, np.zeros((0, 4), np.float32))                       # empty weights
    with pytest.raises(gpu.AccelError):
        gpu.GcnLayer(op, W, bias=np.zeros(5, np.float32))                    # bias of the wrong length
    layer = gpu.GcnLayer(op, W, bias=np.zeros(4, np.float32))
    with pytest.raises(gpu.AccelError):
        layer.forward_numpy(np.zeros((g.n_cols, 9), np.float32))             # features of the wrong width
    with pytest.raises(gpu.AccelError):
        gpu.dense_xw(np.zeros((4, 8), np.float32), layer._w, layer._z, 4, 8, 4)   # a host array as X
    with pytest.raises(gpu.AccelError):
        gpu.dense_xw(layer._z, layer._w, layer._z, 4, 8, 4, ldx=7)           # stride below K
    with pytest.raises(gpu.AccelError):
        gpu.dense_xw_numpy(np.zeros((4, 8), np.float32), np.zeros((7, 4), np.float32))
    Y = layer.forward_numpy(np.zeros((g.n_cols, 8), np.float32))             # zero features: act(bias) = 0
    assert Y.shape == (g.n_rows, 4) and not Y.any()
    layer.close(); layer.close(); op.close()
