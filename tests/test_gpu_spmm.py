"""Parity of the HIP SpMM with the CPU oracle.

Acceptance: max |Y - R| / max(S, tiny) <= 1e-5 with R = A X in fp64 and
S = |A| |X| (the summation order differs from scipy's, so the error is scaled by
the size of the terms, not of the result).  All calls go through the C ABI.
"""
import numpy as np
import pytest

import helpers
from oracle import c_oracle, partition_oracle as po, spmm_oracle as so

pytestmark = pytest.mark.gpu

TOL = 1e-5
ALL_N = [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 13, 16, 17, 30, 32, 33, 48, 50, 60, 64, 99, 100, 127, 128, 130, 200, 256,
         257, 260, 261, 300, 512, 515]


@pytest.fixture(scope="module", params=["workgroup units", "wavefront units"])
def mixed(gpu, request):
    """A small matrix with every degree regime, once with a workgroup per unit (what the
    library chooses for a matrix of this size) and once with a wavefront per unit (what
    it chooses for large ones)."""
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=7, n_long=8, zeros=11), seed=7)
    team = 2 if request.param == "workgroup units" else 1
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team)
    assert op.info.plan_team == (team == 2)
    yield g, op
    op.close()


@pytest.mark.parametrize("N", ALL_N)
def test_every_column_count(gpu, mixed, N):
    """Every vector width / group width, column tails, N beyond one pass (N > 256),
    and the N upstream's lane mapping gets wrong (130, 200)."""
    g, op = mixed
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    Y = op.matmul(X)                                   # output buffer is pre-filled with NaN
    assert np.isfinite(Y).all(), "some row of Y was not written"
    assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL
    d = np.diff(g.indptr)
    assert np.array_equal(Y[d == 0], np.zeros(((d == 0).sum(), N), np.float32))   # beta = 0


@pytest.mark.parametrize("N", [4, 5, 17, 64, 99, 259])
def test_operands_at_any_4_byte_alignment(gpu, mixed, N):
    """X and Y that start 4, 8 or 12 bytes past a 16-byte boundary (and rows that do so
    because N is odd) are read and written with 16-byte accesses at those addresses; the
    words just before and just behind Y must stay untouched."""
    g, op = mixed
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    pad = 8                                               # floats of canary on either side of Y
    for off in (1, 2, 3):                                 # floats past the aligned start
        hx = np.zeros(X.size + 4, np.float32)
        hx[off:off + X.size] = X.reshape(-1)
        dX = gpu.DeviceBuffer.from_numpy(hx)
        dY = gpu.DeviceBuffer((g.n_rows * N + 2 * pad + 4) * 4)
        dY.fill_u32(0x7FC00000)
        op.run(dX.address + 4 * off, dY.address + 4 * (pad + off), N)
        op.synchronize()
        raw = dY.to_numpy(np.float32, (g.n_rows * N + 2 * pad + 4,))
        Y = raw[pad + off:pad + off + g.n_rows * N].reshape(g.n_rows, N)
        assert np.isnan(raw[:pad + off]).all() and np.isnan(raw[pad + off + g.n_rows * N:]).all()
        assert np.isfinite(Y).all()
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL
        dX.close()
        dY.close()


@pytest.mark.parametrize("N,ld", [(127, 128), (50, 64), (64, 80), (17, 32), (3, 8), (130, 131), (300, 320)])
def test_rows_with_a_stride(gpu, mixed, N, ld):
    """accel_run_strided: rows of X and Y are ld floats apart; the padding columns of X are
    never read (they hold NaN) and those of Y never written."""
    g, op = mixed
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    Xp = np.full((g.n_cols, ld), np.nan, np.float32)
    Xp[:, :N] = X
    dX = gpu.DeviceBuffer.from_numpy(Xp.reshape(-1)[: (g.n_cols - 1) * ld + N])   # no padding behind the last row
    dY = gpu.DeviceBuffer(((g.n_rows - 1) * ld + N) * 4)
    dY.fill_u32(0x7FC00000)
    op.run_strided(dX, dY, N, ld)
    op.synchronize()
    flat = dY.to_numpy(np.float32, ((g.n_rows - 1) * ld + N,))
    Yp = np.full((g.n_rows, ld), np.nan, np.float32)
    Yp.reshape(-1)[: flat.size] = flat
    assert np.isfinite(Yp[:, :N]).all()
    assert np.isnan(Yp[:-1, N:]).all(), "padding columns of Y were written"
    assert so.check(np.ascontiguousarray(Yp[:, :N]), g.indptr, g.indices, g.values, X) <= TOL
    with pytest.raises(gpu.AccelError):
        op.run_strided(dX, dY, N, N - 1)
    dX.close()
    dY.close()


@pytest.mark.parametrize("N,ld,relu", [(50, 64, True), (127, 128, False), (64, 0, True), (20, 32, True), (130, 160, True)])
def test_every_option_of_a_run_at_once(gpu, mixed, N, ld, relu):
    """accel_run_ex: rows with a stride and the fused bias / ReLU in one call; with the other
    fields at zero it is accel_run / accel_run_strided / accel_run_epilogue, bit for bit."""
    g, op = mixed
    step = ld or N
    rng = np.random.default_rng(N + step)
    X = rng.uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    bias = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    Xp = np.full((g.n_cols, step), np.nan, np.float32)
    Xp[:, :N] = X
    dX = gpu.DeviceBuffer.from_numpy(Xp.reshape(-1)[: (g.n_cols - 1) * step + N])
    dB = gpu.DeviceBuffer.from_numpy(bias)
    n_out = (g.n_rows - 1) * step + N

    def result(call):
        dY = gpu.DeviceBuffer(n_out * 4)
        dY.fill_u32(0x7FC00000)
        call(dY)
        op.synchronize()
        Yp = np.full((g.n_rows, step), np.nan, np.float32)
        Yp.reshape(-1)[:n_out] = dY.to_numpy(np.float32, (n_out,))
        dY.close()
        assert np.isnan(Yp[:-1, N:]).all(), "padding columns of Y were written"
        return np.ascontiguousarray(Yp[:, :N])

    Y = result(lambda dY: op.run_ex(dX, dY, N, ld=ld, bias=dB, relu=relu))
    R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
    R = R + bias.astype(np.float64)
    if relu:
        R = np.maximum(R, 0.0)
    assert np.isfinite(Y).all()
    assert np.max(np.abs(Y - R) / np.maximum(S + np.abs(bias), 1e-30)) <= TOL
    if relu:
        assert (Y >= 0).all()
    # the plain product through the same entry point = the dedicated entry points
    plain = result(lambda dY: op.run_ex(dX, dY, N, ld=ld))
    same = result(lambda dY: op.run_strided(dX, dY, N, step)) if ld else result(lambda dY: op.run(dX, dY, N))
    assert np.array_equal(plain.view(np.uint32), same.view(np.uint32))
    if not ld:
        fused = result(lambda dY: op.run_epilogue(dX, dY, N, bias=dB, relu=relu))
        assert np.array_equal(Y.view(np.uint32), fused.view(np.uint32))
    with pytest.raises(gpu.AccelError) as e:
        op.run_ex(dX, gpu.DeviceBuffer(16), N, ld=ld)          # Y too small
    assert e.value.status == gpu._lib.ERR_ARG
    L = gpu._lib.lib()
    assert L.accel_run_ex(op._h, None) == gpu._lib.ERR_ARG
    a = gpu._lib.RunArgs()
    a.X, a.N, a.ld, a.flags = dX.address, N, step, 8
    assert L.accel_run_ex(op._h, a) == gpu._lib.ERR_ARG        # unknown flag (checked before Y)
    dX.close()
    dB.close()


@pytest.mark.parametrize("N", [17, 33, 50, 99, 127])
def test_column_counts_of_upstreams_sweep_on_cfg2(gpu, N):
    """Upstream sweeps dim 16..128 in steps of 1 (main.cu:12): three quarters of those are
    not multiples of 4.  cfg2 is large enough for wavefront units and split rows."""
    g = gpu.synthetic.cfg2()
    X = gpu.synthetic.dense_operand("cfg2", g.n_cols, N)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    assert op.info.plan_team == 0 and op.info.n_split_rows > 0
    Y = op.matmul(X)
    R, S = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
    assert so.scaled_error(Y, R, S) <= TOL
    op.close()


@pytest.mark.parametrize("N,panel", [(64, 32), (128, 32), (128, 64), (96, 32), (48, 16), (256, 128),
                                     (100, 64), (100, 32), (72, 20), (8, 4)])    # the last panel narrower
def test_forced_column_panels(gpu, mixed, N, panel):
    """A run cut into column panels computes the same product (a narrower panel gives a row
    more lane groups, so the order of the additions may differ)."""
    g, op = mixed
    X = np.random.default_rng(N + panel).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    op.set_panel(N)                                       # one pass
    Y1 = op.matmul(X)
    op.set_panel(panel)
    Yp = op.matmul(X)
    op.set_panel(0)
    assert np.isfinite(Yp).all()
    assert so.check(Yp, g.indptr, g.indices, g.values, X) <= TOL
    assert np.max(np.abs(Yp - Y1)) <= 1e-5 * np.abs(Y1).max()


def test_workload_cfg1(gpu):
    g = gpu.synthetic.cfg1()
    X = gpu.synthetic.dense_operand("cfg1", g.n_cols, 32)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    Y = op.matmul(X)
    assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL
    Ys = so.spmm_scipy32(g.indptr, g.indices, g.values, X)
    assert np.max(np.abs(Y - Ys)) / np.max(np.abs(Ys)) <= TOL
    assert so.upstream_mean_abs_error(Y, Ys) < 1e-3     # upstream's own, looser bar (main.cu:41)
    op.close()


@pytest.mark.parametrize("N", [16, 32, 64, 128])
def test_workload_cfg2(gpu, N):
    g = gpu.synthetic.cfg2()
    X = gpu.synthetic.dense_operand("cfg2", g.n_cols, N)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    Y = op.matmul(X)
    R, S = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
    assert so.scaled_error(Y, R, S) <= TOL
    op.close()


def test_hub_rows_and_wide_X(gpu):
    """Shape of cfg5: rows spanning several 384-non-zero segments, a majority of
    degree-1 rows, N = 256, X ~ N(0,1), val ~ U(0,1]."""
    g = gpu.synthetic.hub_graph_small()
    X = gpu.synthetic.dense_operand(g.name, g.n_cols, 256)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    assert op.info.n_long_rows >= 4
    Y = op.matmul(X)
    assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL
    op.close()


def test_one_very_long_row(gpu):
    # 100k non-zeros in one row: 261 segments reduced through the scratch buffer
    deg = np.array([1, 100_000, 0, 2, 384, 385], dtype=np.int64)
    g = helpers.graph_from_degrees(deg, n_cols=120_000, seed=9)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    for N in (4, 64, 100):
        X = np.random.default_rng(N).standard_normal((g.n_cols, N)).astype(np.float32)
        Y = op.matmul(X)
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL
    op.close()


def test_closed_forms(gpu):
    deg = helpers.degree_mix(seed=4, n_long=5)
    g = helpers.graph_from_degrees(deg, seed=4, value_mode="ones")
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    Y = op.matmul(np.ones((g.n_cols, 8), np.float32))
    assert np.array_equal(Y, np.repeat(deg[:, None], 8, 1).astype(np.float32))   # ones -> row degree, exact
    op.close()
    n = 777                                                                     # identity -> X, exact
    X = np.random.default_rng(0).standard_normal((n, 20)).astype(np.float32)
    eye = gpu.AccelSpMM(np.arange(n + 1, dtype=np.int32), np.arange(n, dtype=np.int32),
                        np.ones(n, np.float32), n).preprocess()
    assert np.array_equal(eye.matmul(X), X)
    eye.close()


def test_row_order_follows_the_callers_csr(gpu):
    """Rows of Y are in the caller's order; the same matrix given already
    degree-sorted (as upstream's *.new_* files are) gives the permuted rows."""
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=5, n_long=4), seed=5)
    X = np.random.default_rng(5).uniform(-1, 1, (g.n_cols, 48)).astype(np.float32)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    Y = op.matmul(X)
    perm = po.degree_sort(g.indptr)
    sip, six, sval = po.permute_csr(g.indptr, g.indices, g.values, perm)
    ops = gpu.AccelSpMM(sip, six, sval, g.n_cols).preprocess()
    assert ops.info.already_sorted == 1
    assert np.array_equal(ops.matmul(X), Y[perm])        # same arithmetic, same bits
    op.close()
    ops.close()


def test_deterministic_and_overwrites(gpu, mixed):
    g, op = mixed
    X = np.random.default_rng(1).uniform(-1, 1, (g.n_cols, 64)).astype(np.float32)
    dX = gpu.DeviceBuffer.from_numpy(X)
    dY = gpu.DeviceBuffer(g.n_rows * 64 * 4)
    outs = []
    for fill in (0x7FC00000, 0x3F800000, 0):            # NaN, 1.0, 0.0 left in Y before the run
        dY.fill_u32(fill)
        op.run(dX, dY, 64)
        op.run(dX, dY, 64)                               # twice: upstream would accumulate
        op.synchronize()
        outs.append(dY.to_numpy(np.float32, (g.n_rows, 64)))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    assert so.check(outs[0], g.indptr, g.indices, g.values, X) <= TOL
    dX.close()
    dY.close()


def test_linearity_and_column_slicing(gpu):
    g = gpu.synthetic.cfg2()
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    rng = np.random.default_rng(2)
    X1 = rng.uniform(-1, 1, (g.n_cols, 128)).astype(np.float32)
    X2 = rng.uniform(-1, 1, (g.n_cols, 128)).astype(np.float32)
    Y1, Y2, Y12 = op.matmul(X1), op.matmul(X2), op.matmul(X1 + X2)
    scale = np.abs(Y1).max() + np.abs(Y2).max()
    assert np.max(np.abs(Y12 - (Y1 + Y2))) <= 1e-5 * scale
    # column j of the N=128 result is column j of the N=16 result on the same columns
    Y16 = op.matmul(np.ascontiguousarray(X1[:, :16]))
    assert np.max(np.abs(Y16 - Y1[:, :16])) <= 1e-5 * np.abs(Y1).max()
    op.close()


def test_operator_mirror_do_test(gpu, tmp_path):
    """SpmmAccel follows SPMM_ACCEL: construct on device pointers of a
    degree-sorted CSR, do_test(False, dim) computes, do_test(True, dim) returns
    seconds; a matching .block4 file is accepted, a stale one refused."""
    g0 = gpu.synthetic.cfg1()
    perm = po.degree_sort(g0.indptr)
    sip, six, sval = po.permute_csr(g0.indptr, g0.indices, g0.values, perm)
    dim_max = 64
    X = gpu.synthetic.dense_operand("cfg1", g0.n_cols, dim_max)
    bufs = [gpu.DeviceBuffer.from_numpy(a) for a in (sip, six, sval, X)]
    vout = gpu.DeviceBuffer(g0.n_rows * dim_max * 4)
    meta = tmp_path / "block_level_meta"
    meta.mkdir()
    gpu.block_level_partition.write_block4(meta / "cfg1.block4", po.partition_closed_form(sip))
    acc = gpu.SpmmAccel("cfg1", bufs[0], bufs[1], bufs[2], bufs[3], vout, g0.n_rows, g0.nnz, dim_max,
                        meta_dir=meta)
    for dim in (16, 33, 64):                              # leading dimension = current dim
        assert acc.do_test(False, dim) == 0.0
        Y = vout.to_numpy(np.float32, (g0.n_rows, dim))
        Xd = X.reshape(-1)[: g0.n_cols * dim].reshape(g0.n_cols, dim)
        assert so.check(Y, sip, six, sval, Xd) <= TOL
    t = acc.do_test(True, 64)
    assert 0 < t < 1.0
    # the array of values rewritten in place between two calls (upstream's kernel reads it on
    # every launch, spmm_accel.cu:75): the next call computes with the new values
    v2 = (sval * np.float32(-0.5)).astype(np.float32)
    gpu._lib.check(gpu._lib.lib().accel_memcpy_h2d(bufs[2].address, v2.ctypes.data, v2.nbytes))
    assert acc.do_test(False, 16) == 0.0
    Xd = X.reshape(-1)[: g0.n_cols * 16].reshape(g0.n_cols, 16)
    assert so.check(vout.to_numpy(np.float32, (g0.n_rows, 16)), sip, six, v2, Xd) <= TOL
    b = po.partition_closed_form(sip).copy()
    b[0, 3] += 1
    gpu.block_level_partition.write_block4(meta / "stale.block4", b)
    stale = gpu.SpmmAccel("stale", bufs[0], bufs[1], bufs[2], bufs[3], vout, g0.n_rows, g0.nnz, dim_max,
                          meta_dir=meta)
    with pytest.raises(gpu.AccelError) as e:
        stale.do_test(False, 16)
    assert e.value.status == gpu._lib.ERR_META
    for bfr in bufs + [vout]:
        bfr.close()


def test_timing_entry_point(gpu, mixed):
    g, op = mixed
    X = np.random.default_rng(3).uniform(-1, 1, (g.n_cols, 64)).astype(np.float32)
    dX = gpu.DeviceBuffer.from_numpy(X)
    dY = gpu.DeviceBuffer(g.n_rows * 64 * 4)
    tot, main = op.time(dX, dY, 64, warmup=2, iters=5)
    assert tot.shape == (5,) and np.all(tot > 0) and np.all(main > 0) and np.all(main <= tot * 1.001)
    assert so.check(dY.to_numpy(np.float32, (g.n_rows, 64)), g.indptr, g.indices, g.values, X) <= TOL
    dX.close()
    dY.close()


def test_timing_entry_point_with_every_option(gpu, mixed):
    """accel_time_ex: the same protocol on rows with a stride, bias and ReLU; the output it
    leaves is the product."""
    g, op = mixed
    N, ld = 50, 64
    rng = np.random.default_rng(5)
    X = rng.uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    Xp = np.zeros((g.n_cols, ld), np.float32); Xp[:, :N] = X
    dX, dB = gpu.DeviceBuffer.from_numpy(Xp), gpu.DeviceBuffer.from_numpy(bias)
    dY = gpu.DeviceBuffer(g.n_rows * ld * 4)
    dY.fill_u32(0x7FC00000)
    tot, main = op.time_ex(dX, dY, N, ld=ld, bias=dB, relu=True, warmup=1, iters=4)
    assert tot.shape == (4,) and np.all(tot > 0) and np.all(main > 0) and np.all(main <= tot * 1.001)
    Y = dY.to_numpy(np.float32, (g.n_rows, ld))
    R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
    want = np.maximum(R + bias.astype(np.float64), 0.0)
    assert np.max(np.abs(Y[:, :N] - want) / np.maximum(S + np.abs(bias), 1e-30)) <= TOL
    assert np.isnan(Y[:, N:]).all()
    L = gpu._lib
    a = L.RunArgs()
    a.X, a.Y, a.N, a.ld = dX.address, dY.address, N, N - 1
    assert L.lib().accel_time_ex(op._h, a, 1, 1, None, None) == L.ERR_ARG      # stride below N
    assert L.lib().accel_time_ex(op._h, None, 1, 1, None, None) == L.ERR_ARG
    for b in (dX, dB, dY):
        b.close()


def test_medium_power_law_graph(gpu):
    """A 300k-row, ~15M-edge graph generated like cfg4 (gamma 2.1)."""
    g = gpu.synthetic.cfg4(n=300_000, n_edges=15_000_000, max_degree=17_000)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    perm, sip, six, sval, b4 = helpers.expected_preprocess(g.indptr, g.indices, g.values)
    assert np.array_equal(op.perm(), perm) and op.block4().tobytes() == po.block4_to_bytes(b4)
    for N in (64, 100):
        X = gpu.synthetic.dense_operand("cfg4", g.n_cols, N)
        Y = op.matmul(X)
        R, S = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
        assert so.scaled_error(Y, R, S) <= TOL
    op.close()


FULL_SIZE = {"cfg3": (233_000, 110_000_000), "cfg4": (2_450_000, 120_000_000), "cfg5": (1_000_000, 25_000_000)}
_full = {}


def full_size_case(gpu, name):
    """The workload at benchmark size with its operator, its row sums and the oracle's
    preprocessing; one workload is kept at a time (cfg4 alone is 1.5 GB of CSR)."""
    if name not in _full:
        for old in list(_full):
            _full.pop(old)["op"].close()
        g = getattr(gpu.synthetic, name)()
        rows, min_nnz = FULL_SIZE[name]
        assert g.n_rows == rows and g.nnz > min_nnz
        op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
        assert op.info.plan_team == 0 and op.info.plan_unit_nz == 384
        v64 = g.values.astype(np.float64)
        filled = np.flatnonzero(np.diff(g.indptr) > 0)   # reduceat wants strictly increasing starts
        row_sum, row_abs = np.zeros(g.n_rows), np.zeros(g.n_rows)
        row_sum[filled] = np.add.reduceat(v64, g.indptr[filled].astype(np.int64))
        row_abs[filled] = np.add.reduceat(np.abs(v64), g.indptr[filled].astype(np.int64))
        _full[name] = dict(g=g, op=op, row_sum=row_sum, row_abs=row_abs, v64=v64)
    return _full[name]


@pytest.mark.parametrize("name", ["cfg3", "cfg4", "cfg5"])
def test_metadata_of_large_workloads_at_full_size(gpu, name):
    """Degree sort, sorted indptr and block4 of the benchmark workloads at benchmark size,
    bit for bit against the oracle (stable argsort + the vectorised closed form of the walk)."""
    c = full_size_case(gpu, name)
    g, op = c["g"], c["op"]
    perm = po.degree_sort(g.indptr)
    assert np.array_equal(op.perm(), perm)
    sip = np.zeros(g.n_rows + 1, dtype=np.int64)
    np.cumsum(np.diff(g.indptr)[perm], out=sip[1:])
    got_ip, _, _ = op.sorted_csr()
    assert np.array_equal(got_ip, sip.astype(np.int32))
    assert op.block4().tobytes() == po.block4_to_bytes(po.partition_closed_form(sip.astype(np.int32)))
    assert op.info.n_blocks == op.block4().shape[0]


@pytest.mark.parametrize("name,N", [("cfg3", 32), ("cfg3", 64), ("cfg3", 128), ("cfg4", 16), ("cfg4", 64),
                                    ("cfg4", 100), ("cfg5", 256)])
def test_large_workloads_at_full_size(gpu, name, N):
    """Every (workload, N) pair of the benchmark at benchmark size (cfg4 at N = 64 is the
    headline: 2.45 M rows, ~125 M non-zeros).  Every row of Y against the fp64 oracle, plus
    properties that cost O(nnz) on the host: X = 1 gives the row sums of A; the column sums
    of Y equal (1^T A) X; A (X1 + X2) = A X1 + A X2."""
    import os
    c = full_size_case(gpu, name)
    g, op, row_sum, row_abs, v64 = c["g"], c["op"], c["row_sum"], c["row_abs"], c["v64"]
    tiny = 1e-300
    ones = gpu.DeviceBuffer.from_numpy(np.ones((g.n_cols, N), np.float32))
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    op.run(ones, dY, N)
    Y1 = dY.to_numpy(np.float32, (g.n_rows, N))
    assert np.max(np.abs(Y1 - row_sum[:, None]) / np.maximum(row_abs[:, None], tiny)) <= TOL
    ones.close()
    dY.close()
    del Y1
    X1 = gpu.synthetic.dense_operand(name, g.n_cols, N)
    Ya = op.matmul(X1)
    assert np.isfinite(Ya).all()
    # all rows against A X in fp64, a slab of rows at a time
    threads = min(16, os.cpu_count() or 1)
    worst = 0.0
    slab = max(1, (64 << 20) // N)                        # 512 MB of R and S at a time
    for r0 in range(0, g.n_rows, slab):
        r1 = min(g.n_rows, r0 + slab)
        R, S = c_oracle.spmm_csr_f64(g.indptr[r0:r1 + 1], g.indices, g.values, X1, threads=threads)
        worst = max(worst, so.scaled_error(Ya[r0:r1], R, S))
        del R, S
    assert worst <= TOL
    col_w = np.bincount(g.indices, weights=v64, minlength=g.n_cols)
    col_a = np.bincount(g.indices, weights=np.abs(v64), minlength=g.n_cols)
    check_sum = Ya.sum(axis=0, dtype=np.float64)
    bound = col_a @ np.abs(X1).astype(np.float64)
    assert np.max(np.abs(check_sum - col_w @ X1.astype(np.float64)) / np.maximum(bound, tiny)) <= TOL
    if N == 64 or name == "cfg5":                         # linearity once per workload
        X2 = np.random.default_rng(5).uniform(-1, 1, X1.shape).astype(np.float32)
        Yb = op.matmul(X2)
        Yc = op.matmul(X1 + X2)
        # |A| (|X1| + |X2|) <= |A| 1 (max|X1| + max|X2|)
        Sabs = row_abs[:, None] * float(np.abs(X1).max() + np.abs(X2).max())
        assert np.max(np.abs(Yc - (Ya + Yb)) / np.maximum(Sabs, tiny)) <= 4 * TOL


def test_release_full_size_cases():
    for old in list(_full):
        _full.pop(old)["op"].close()


@pytest.mark.parametrize("N", [16, 64, 100, 3])
def test_fused_bias_and_relu(gpu, mixed, N):
    """Y = relu(A X + b) in the store; rows of degree 0 become relu(b)."""
    g, op = mixed
    rng = np.random.default_rng(N)
    X = rng.uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    b = rng.uniform(-0.5, 0.5, N).astype(np.float32)
    dX, db = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(b)
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
    for bias, relu in ((db, True), (db, False), (None, True), (None, False)):
        dY.fill_u32(0x7FC00000)
        op.run_epilogue(dX, dY, N, bias=bias, relu=relu)
        op.synchronize()
        Y = dY.to_numpy(np.float32, (g.n_rows, N)).astype(np.float64)
        ref = R + (b.astype(np.float64) if bias is not None else 0.0)
        scale = S + (np.abs(b) if bias is not None else 0.0)
        if relu:
            ref = np.maximum(ref, 0.0)
        assert np.isfinite(Y).all()
        assert np.max(np.abs(Y - ref) / np.maximum(scale, np.finfo(np.float32).tiny)) <= TOL
        if relu:
            assert Y.min() >= 0.0
    with pytest.raises(gpu.AccelError) as e:
        gpu._lib.check(gpu.lib().accel_run_epilogue(op._h, gpu._lib.ptr(dX), gpu._lib.ptr(dY), N, None, 8, None))
    assert e.value.status == gpu._lib.ERR_ARG
    for buf in (dX, db, dY):
        buf.close()


@pytest.mark.parametrize("n_cols,team", [(5_000_000, 2), (5_000_000, 1), (4_194_300, 1)])
def test_operands_beyond_4_gib(gpu, n_cols, team):
    """X and Y larger than 4 GiB: row offsets need 64-bit arithmetic (both kernels), and an X
    just below 4 GiB, the largest that is addressed with 32-bit byte offsets.  The
    matrix references rows of X at both ends of a 5.1 (4.3) GB buffer and writes rows
    of Y at both ends of a 4.4 GB buffer; only the touched rows travel to the host."""
    import ctypes as C
    N, n_rows = 256, 4_300_000
    assert (n_cols * N * 4 > 2 ** 32) == (n_cols == 5_000_000)
    rng = np.random.default_rng(0)
    cols = np.unique(np.concatenate([[0, 1, n_cols - 1, n_cols - 2, min(4_194_304, n_cols - 3), 4_194_203],
                                     rng.integers(0, n_cols, 500)])).astype(np.int32)
    live_rows = np.unique(np.concatenate([[0, 7, n_rows - 1, n_rows - 2, 4_194_304, 4_194_305],
                                          rng.integers(0, n_rows, 60)]))
    deg = np.zeros(n_rows, dtype=np.int64)
    deg[live_rows] = rng.integers(1, 40, live_rows.size)
    deg[live_rows[3]] = 450                                   # one long row as well
    indptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    nnz = int(indptr[-1])
    idx = np.concatenate([np.sort(rng.choice(cols, d, replace=False)) for d in deg[live_rows]]).astype(np.int32)
    val = rng.uniform(-1, 1, nnz).astype(np.float32)
    Xrows = rng.uniform(-1, 1, (cols.size, N)).astype(np.float32)

    lib = gpu.lib()
    dX = gpu.DeviceBuffer(n_cols * N * 4)
    dY = gpu.DeviceBuffer(n_rows * N * 4)
    dX.fill_u32(0)
    dY.fill_u32(0x7FC00000)
    for c, row in zip(cols, Xrows):                            # only the referenced rows of X are non-zero
        gpu._lib.check(lib.accel_memcpy_h2d(C.c_void_p(dX.address + int(c) * N * 4), C.c_void_p(row.ctypes.data), N * 4))
    op = gpu.AccelSpMM(indptr.astype(np.int32), idx, val, n_cols).preprocess(plan_team=team)
    op.run(dX, dY, N)
    op.synchronize()

    def y_row(r):
        out = np.empty(N, dtype=np.float32)
        gpu._lib.check(lib.accel_memcpy_d2h(C.c_void_p(out.ctypes.data), C.c_void_p(dY.address + int(r) * N * 4), N * 4))
        return out

    pos = {int(c): i for i, c in enumerate(cols)}
    for r in live_rows:
        a, b = indptr[r], indptr[r + 1]
        xs = Xrows[[pos[int(c)] for c in idx[a:b]]].astype(np.float64)
        ref = (val[a:b].astype(np.float64)[:, None] * xs).sum(0)
        scale = (np.abs(val[a:b]).astype(np.float64)[:, None] * np.abs(xs)).sum(0)
        assert np.max(np.abs(y_row(r) - ref) / np.maximum(scale, 1e-30)) <= TOL, r
    live = set(live_rows.tolist())
    for r in (1, 2, 4_194_303, 4_194_306, n_rows - 3, n_rows // 2):     # zero-degree rows at both ends
        if r not in live:
            assert np.array_equal(y_row(r), np.zeros(N, np.float32)), r
    op.close(); dX.close(); dY.close()


def test_random_shapes(gpu):
    """Sixty seeded random matrices: random row counts, degree mixes (empty rows,
    every slice-table regime, rows of several thousand non-zeros) and column
    counts 1..320, rectangular as well as square; alternately with a workgroup and
    with a wavefront per unit."""
    rng = np.random.default_rng(2024)
    pool = np.array([0, 0, 1, 1, 2, 3, 7, 12, 31, 32, 33, 64, 65, 96, 97, 128, 129, 191, 192, 200, 383, 384,
                     385, 500, 768, 769, 1153, 3000])
    for case in range(60):
        n_rows = int(rng.integers(1, 260))
        deg = rng.choice(pool, size=n_rows, p=None)
        if case % 3 == 0:
            deg = np.minimum(deg, 40)                         # short rows only
        n_cols = int(max(deg.max() + 1, rng.integers(1, 5000)))
        N = int(rng.integers(1, 321))
        g = gpu.synthetic.random_csr(n_rows, n_cols, deg, seed=case)
        X = rng.uniform(-1, 1, (n_cols, N)).astype(np.float32)
        op = gpu.AccelSpMM(g.indptr, g.indices, g.values, n_cols).preprocess(plan_team=1 + case % 2)
        Y = op.matmul(X)
        assert np.isfinite(Y).all(), (case, n_rows, N)
        err = so.check(Y, g.indptr, g.indices, g.values, X)
        assert err <= TOL, (case, n_rows, n_cols, N, err)
        op.close()


def test_very_wide_operand(gpu):
    """N beyond 8192 columns: many column passes per unit, and the zero-fill of empty rows
    changes from several rows per workgroup to one."""
    deg = np.array([0, 3, 0, 40, 500, 1, 0, 200, 12, 0, 385], dtype=np.int64)
    g = helpers.graph_from_degrees(deg, n_cols=600, seed=12)
    for team in (1, 2):
        op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team)
        for N in (8188, 8192, 8200, 9001):
            X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
            Y = op.matmul(X)
            assert np.all(Y[deg == 0] == 0.0)
            assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL, (team, N)
        op.close()


def test_column_panels(gpu):
    """Wide operands on a matrix large enough to be computed in 64-column panels
    (N = 128, 256) next to widths that are not (N = 100, 192 is, 130 is not)."""
    g = gpu.synthetic.cfg4(n=200_000, n_edges=4_500_000, max_degree=9_000)
    assert g.nnz >= 4_000_000 and g.nnz >= 16 * g.n_rows
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    for N in (128, 256, 192, 100, 130):
        X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
        Y = op.matmul(X)
        assert np.isfinite(Y).all()
        R, S = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
        assert so.scaled_error(Y, R, S) <= TOL, N
    # fused epilogue across panels
    N = 128
    X = np.random.default_rng(1).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    b = np.random.default_rng(2).uniform(-0.5, 0.5, N).astype(np.float32)
    dX, db, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(b), gpu.DeviceBuffer(g.n_rows * N * 4)
    op.run_epilogue(dX, dY, N, bias=db, relu=True)
    op.synchronize()
    R, S = c_oracle.spmm_csr_f64(g.indptr, g.indices, g.values, X)
    ref = np.maximum(R + b.astype(np.float64), 0.0)
    Y = dY.to_numpy(np.float32, (g.n_rows, N)).astype(np.float64)
    assert np.max(np.abs(Y - ref) / np.maximum(S + np.abs(b), 1e-30)) <= TOL
    for buf in (dX, db, dY):
        buf.close()
    op.close()


def test_non_finite_inputs_stay_in_their_rows(gpu, mixed):
    """Inf/NaN in a row of X reach exactly the rows of Y that reference it (masked
    lanes and padding never multiply a stray row of X by zero)."""
    g, op = mixed
    N = 48
    rng = np.random.default_rng(5)
    X = rng.uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    bad_cols = np.unique(g.indices[rng.integers(0, g.nnz, 6)])
    X[bad_cols[0::2], 3] = np.inf
    X[bad_cols[1::2], 7] = np.nan
    X[0, :] = np.nan                       # row 0 of X is where a careless clamp would read
    Y = op.matmul(X)
    with np.errstate(invalid="ignore", over="ignore"):
        ref = so.spmm_scipy32(g.indptr, g.indices, g.values, X)
    assert np.array_equal(np.isnan(Y), np.isnan(ref))
    assert np.array_equal(np.isinf(Y), np.isinf(ref))
    fin = np.isfinite(ref)
    assert np.max(np.abs(Y[fin] - ref[fin])) <= 1e-4
