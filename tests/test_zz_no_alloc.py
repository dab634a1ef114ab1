"""accel_run_static: the entry point that allocates nothing.

It must give the same bits as accel_run (same kernels, the partial sums of split
rows in the library's static device array instead of the handle's buffer), on two
calls in a row of which the second is smaller, and it must refuse a matrix whose
partial sums do not fit the array.  All calls go through the C ABI.
"""
import numpy as np
import pytest

import helpers
from oracle import spmm_oracle as so

pytestmark = pytest.mark.gpu

TOL = 1e-5


def both_ways(gpu, op, g, N, seed):
    X = np.random.default_rng(seed).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    dX = gpu.DeviceBuffer.from_numpy(X)
    dY = gpu.DeviceBuffer(max(g.n_rows * N * 4, 4))
    try:
        dY.fill_u32(0x7FC00000)
        op.run(dX, dY, N)
        op.synchronize()
        Y_run = dY.to_numpy(np.float32, (g.n_rows, N))
        dY.fill_u32(0x7FC00000)
        op.run_static(dX, dY, N)
        op.synchronize()
        Y_static = dY.to_numpy(np.float32, (g.n_rows, N))
    finally:
        dX.close()
        dY.close()
    return X, Y_run, Y_static


def test_same_bits_as_accel_run_twice_second_call_smaller(gpu):
    # wavefront units, so that every row above 192 non-zeros goes through partial sums
    big = helpers.graph_from_degrees(helpers.degree_mix(seed=3, n_long=40, zeros=7), seed=3)
    small = helpers.graph_from_degrees(helpers.degree_mix(seed=4, n_long=5, zeros=2), seed=4)
    op_big = gpu.AccelSpMM(big.indptr, big.indices, big.values, big.n_cols).preprocess(plan_team=1)
    op_small = gpu.AccelSpMM(small.indptr, small.indices, small.values, small.n_cols).preprocess(plan_team=1)
    try:
        assert op_big.info.n_split_rows > op_small.info.n_split_rows > 0
        for op, g, N, seed in ((op_big, big, 96, 11), (op_small, small, 20, 12)):
            X, Y_run, Y_static = both_ways(gpu, op, g, N, seed)
            assert np.isfinite(Y_static).all(), "some row of Y was not written"
            assert np.array_equal(Y_run.view(np.uint32), Y_static.view(np.uint32))
            assert so.check(Y_static, g.indptr, g.indices, g.values, X) <= TOL
    finally:
        op_big.close()
        op_small.close()


def test_first_call_on_a_fresh_handle_allocates_nothing(gpu):
    """The property the entry point exists for: on a handle that has never run (so that no
    partial-sum buffer exists yet) accel_run_static leaves the free device memory where it
    was, while the first accel_run afterwards allocates the handle's buffer."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so.7")
    for name in ("hipMemGetInfo", "hipDeviceSynchronize"):
        getattr(hip, name).restype = C.c_int

    def free_bytes():
        assert hip.hipDeviceSynchronize() == 0
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    # 6,000 split rows of 8 column groups each: 48,000 pieces, 24.6 MB of partial sums at N = 128
    deg = np.concatenate([np.random.default_rng(9).integers(0, 60, 2000), np.full(6000, 400)])
    g = helpers.graph_from_degrees(deg, n_cols=6000, seed=9)
    N = 128
    slack = 2 << 20        # the runtime's own pools move in chunks of this size, in either direction
    X = np.random.default_rng(15).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    dX = gpu.DeviceBuffer.from_numpy(X)
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1)
    try:
        assert op.info.n_split_rows == 6000
        dY.fill_u32(0x7FC00000)
        free_bytes()
        before = free_bytes()
        op.run_static(dX, dY, N)                          # the handle's first run of any kind
        after = free_bytes()
        assert before - after <= slack, f"accel_run_static took {before - after} bytes of device memory"
        Y_static = dY.to_numpy(np.float32, (g.n_rows, N))
        assert so.check(Y_static, g.indptr, g.indices, g.values, X) <= TOL
        op.run_static(dX, dY, 16)                         # another N: still nothing
        assert before - free_bytes() <= slack
        dY.fill_u32(0x7FC00000)
        now = free_bytes()
        op.run(dX, dY, N)                                 # accel_run does allocate its buffer (24.6 MB)
        assert now - free_bytes() >= 6000 * 8 * N * 4 - slack
        assert np.array_equal(dY.to_numpy(np.float32, (g.n_rows, N)).view(np.uint32), Y_static.view(np.uint32))
    finally:
        dX.close()
        dY.close()
        op.close()


def test_workgroup_units_and_no_split_rows(gpu):
    """Small matrices (a workgroup per unit) and matrices without split rows use no
    scratch at all; the entry point must still give accel_run's result."""
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=5, n_long=6, zeros=3), seed=5)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    try:
        X, Y_run, Y_static = both_ways(gpu, op, g, 64, 13)
        assert np.array_equal(Y_run.view(np.uint32), Y_static.view(np.uint32))
        assert so.check(Y_static, g.indptr, g.indices, g.values, X) <= TOL
    finally:
        op.close()
    deg = np.random.default_rng(6).integers(0, 150, 3000)
    g = helpers.graph_from_degrees(deg, n_cols=4000, seed=6)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1, plan_unit=384)
    try:
        assert op.info.n_split_rows == 0
        X, Y_run, Y_static = both_ways(gpu, op, g, 33, 14)
        assert np.array_equal(Y_run.view(np.uint32), Y_static.view(np.uint32))
    finally:
        op.close()


def test_too_large_for_the_static_scratch_is_refused(gpu):
    """6,000 rows of 400 non-zeros are cut into at least 8 pieces each: at N = 192 their
    partial sums need more than the 32 MiB the array holds."""
    deg = np.full(6000, 400)
    g = helpers.graph_from_degrees(deg, n_cols=5000, seed=8)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1)
    N = 192
    X = np.ones((g.n_cols, N), dtype=np.float32)
    dX = gpu.DeviceBuffer.from_numpy(X)
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    try:
        assert op.info.n_split_rows == 6000
        with pytest.raises(gpu.AccelError) as e:
            op.run_static(dX, dY, N)
        assert e.value.status == gpu._lib.ERR_ARG
        assert "static scratch" in e.value.message
        op.run_static(dX, dY, 16)                  # the same matrix fits at a small N
        op.run(dX, dY, N)                          # and accel_run takes it at any N
        op.synchronize()
    finally:
        dX.close()
        dY.close()
        op.close()
