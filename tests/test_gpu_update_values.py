"""accel_update_values: new values on an unchanged structure.

Upstream's kernel reads the caller's value array on every launch (spmm_accel.cu:75), so
rewriting the array is all a caller does there.  Here the kernels read a degree-sorted
copy; after accel_update_values a run must give what a fresh operator on the new values
gives (same bits: the structure, the plan and the order of summation are unchanged), and
the metadata must not move.
"""
import numpy as np
import pytest

import helpers
from oracle import spmm_oracle as so

pytestmark = pytest.mark.gpu

TOL = 1e-5


def graph(seed, n_long=12):
    return helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=n_long, zeros=6), seed=seed)


def new_values(g, seed):
    return np.random.default_rng(seed).uniform(-2, 2, g.values.size).astype(np.float32)


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("N", [64, 21])
def test_updated_values_give_the_bits_of_a_fresh_operator(gpu, team, N):
    g = graph(31)
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team)
    assert a.info.n_split_rows > 0 and a.info.already_sorted == 0
    before = (a.block4(), a.perm(), a.plan(), a.sorted_csr()[1])
    assert so.check(a.matmul(X), g.indptr, g.indices, g.values, X) <= TOL
    for seed in (1, 2):                                   # twice: the copy is refreshed in place
        v = new_values(g, seed)
        a.update_values(v)
        Ya = a.matmul(X)
        assert so.check(Ya, g.indptr, g.indices, v, X) <= TOL
        b = gpu.AccelSpMM(g.indptr, g.indices, v, g.n_cols).preprocess(plan_team=team)
        assert np.array_equal(Ya.view(np.uint32), b.matmul(X).view(np.uint32))
        assert np.array_equal(a.sorted_csr()[2], b.sorted_csr()[2])
        b.close()
    for u, w in zip(before, (a.block4(), a.perm(), a.plan(), a.sorted_csr()[1])):
        assert np.array_equal(u, w)                       # nothing but the values moved
    a.close()


def test_sorted_input_without_split_rows(gpu):
    """The operator has no copy of its own here: the values live in the uploaded CSR."""
    deg = np.sort(np.random.default_rng(3).integers(0, 150, 2000))
    g = helpers.graph_from_degrees(deg, n_cols=3000, seed=3)
    X = np.random.default_rng(4).uniform(-1, 1, (g.n_cols, 20)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1, plan_unit=384)
    assert a.info.already_sorted == 1 and a.info.n_split_rows == 0
    v = new_values(g, 5)
    a.update_values(v)
    assert so.check(a.matmul(X), g.indptr, g.indices, v, X) <= TOL
    a.close()


def test_sorted_input_with_split_rows(gpu):
    deg = np.sort(np.concatenate([np.random.default_rng(6).integers(0, 150, 1500), [700, 900, 5000]]))
    g = helpers.graph_from_degrees(deg, n_cols=6000, seed=6)
    X = np.random.default_rng(7).uniform(-1, 1, (g.n_cols, 32)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    assert a.info.already_sorted == 1 and a.info.n_split_rows > 0
    v = new_values(g, 8)
    a.update_values(v)
    assert so.check(a.matmul(X), g.indptr, g.indices, v, X) <= TOL
    a.close()


def test_after_a_loaded_state(gpu, tmp_path):
    g = graph(32)
    X = np.random.default_rng(9).uniform(-1, 1, (g.n_cols, 48)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    v = new_values(g, 10)
    a.update_values(v)
    Ya = a.matmul(X)
    a.close()
    # the state holds no values: it serves a handle created on the new ones, and one updated afterwards
    b = gpu.AccelSpMM(g.indptr, g.indices, v, g.n_cols).load_state(path)
    assert np.array_equal(Ya.view(np.uint32), b.matmul(X).view(np.uint32))
    w = new_values(g, 11)
    b.update_values(w)
    assert so.check(b.matmul(X), g.indptr, g.indices, w, X) <= TOL
    b.close()


def test_preprocessing_again_after_an_update_keeps_the_new_values(gpu, tmp_path):
    """A handle that uploaded its CSR updates only its sorted copy; its copy of the caller's
    order is brought back from there when the handle is preprocessed (or loads a state) again."""
    g = graph(35)
    N = 24
    X = np.random.default_rng(15).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    a.save_state(tmp_path / "g.accelstate")
    v = new_values(g, 16)
    dV = gpu.DeviceBuffer.from_numpy(v)
    a.update_values_async(dV)
    dV.close()                                            # the handle does not borrow it
    want = a.matmul(X)
    assert so.check(want, g.indptr, g.indices, v, X) <= TOL
    a.preprocess(plan_unit=64)                            # other plan, same (new) values
    assert so.check(a.matmul(X), g.indptr, g.indices, v, X) <= TOL
    w = new_values(g, 17)
    dW = gpu.DeviceBuffer.from_numpy(w)
    a.update_values_async(dW)
    a.update_values_async(dW)
    a.load_state(tmp_path / "g.accelstate")               # the saved order, the newest values
    got = a.matmul(X)
    assert so.check(got, g.indptr, g.indices, w, X) <= TOL
    b = gpu.AccelSpMM(g.indptr, g.indices, w, g.n_cols).preprocess()
    assert np.array_equal(got.view(np.uint32), b.matmul(X).view(np.uint32))
    a.update_values(v)                                    # a host array goes into the handle's copy directly
    a.preprocess()
    assert np.array_equal(a.matmul(X).view(np.uint32), want.view(np.uint32))
    dW.close()
    a.close()
    b.close()


def test_borrowed_device_csr(gpu):
    """A handle on the caller's device arrays: the same array rewritten in place, then another one."""
    g = graph(33)
    N = 40
    X = np.random.default_rng(12).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    d_ip = gpu.DeviceBuffer.from_numpy(g.indptr.astype(np.int32))
    d_ix = gpu.DeviceBuffer.from_numpy(g.indices.astype(np.int32))
    d_v = gpu.DeviceBuffer.from_numpy(g.values.astype(np.float32))
    a = gpu.AccelSpMM(d_ip, d_ix, d_v, g.n_cols, device=True, n_rows=g.n_rows, nnz=g.indices.size).preprocess()
    assert so.check(a.matmul(X), g.indptr, g.indices, g.values, X) <= TOL
    v = new_values(g, 13)
    gpu._lib.check(gpu._lib.lib().accel_memcpy_h2d(d_v.address, v.ctypes.data, v.nbytes))
    a.update_values(d_v)                                  # same array, new contents
    assert so.check(a.matmul(X), g.indptr, g.indices, v, X) <= TOL
    w = new_values(g, 14)
    d_w = gpu.DeviceBuffer.from_numpy(w)
    a.update_values(d_w)                                  # another array: borrowed from now on
    assert so.check(a.matmul(X), g.indptr, g.indices, w, X) <= TOL
    with pytest.raises(gpu.AccelError) as e:              # a host array cannot be borrowed
        a.update_values(v)
    assert e.value.status == gpu._lib.ERR_ARG
    assert so.check(a.matmul(X), g.indptr, g.indices, w, X) <= TOL
    a.close()
    for d in (d_ip, d_ix, d_v, d_w):
        d.close()


def test_refusals(gpu):
    g = graph(34)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)
    with pytest.raises(gpu.AccelError) as e:              # before preprocess
        a.update_values(g.values)
    assert e.value.status == gpu._lib.ERR_STATE
    a.preprocess()
    with pytest.raises(gpu.AccelError) as e:              # wrong length
        a.update_values(g.values[:-1])
    assert e.value.status == gpu._lib.ERR_ARG
    small = gpu.DeviceBuffer(16)
    with pytest.raises(gpu.AccelError) as e:              # device array too small
        a.update_values(small)
    assert e.value.status == gpu._lib.ERR_ARG
    L = gpu._lib.lib()
    assert L.accel_update_values(a._h, None, gpu._lib.PTR_HOST) == gpu._lib.ERR_ARG
    assert L.accel_update_values(a._h, small.address, 7) == gpu._lib.ERR_ARG
    # a raw device address that is too small is caught by the library itself
    assert L.accel_update_values(a._h, small.address, gpu._lib.PTR_DEVICE) == gpu._lib.ERR_ARG
    small.close()
    a.close()


def test_empty_matrix(gpu):
    a = gpu.AccelSpMM(np.zeros(4, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 5).preprocess()
    a.update_values(np.zeros(0, np.float32))
    assert np.array_equal(a.matmul(np.ones((5, 8), np.float32)), np.zeros((3, 8), np.float32))
    a.close()
