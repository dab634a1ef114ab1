"""Saved preprocessing state: accel_save_state / accel_load_state.

A state saved for a CSR and loaded into a new handle on the same CSR must give the
same metadata and the same bits of Y as preprocessing again; a state of another CSR,
a damaged or a truncated file must be refused and leave the handle un-preprocessed.
"""
import numpy as np
import pytest

import helpers
from oracle import partition_oracle as po, spmm_oracle as so

pytestmark = pytest.mark.gpu

TOL = 1e-5


def graph(seed, n_long=12):
    return helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=n_long, zeros=6), seed=seed)


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("N", [64, 33])
def test_loaded_state_gives_the_same_bits(gpu, tmp_path, team, N):
    g = graph(21)
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team)
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    Ya = a.matmul(X)
    b = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).load_state(path)
    try:
        for f in ("rows", "cols", "nnz", "n_blocks", "n_long_blocks", "n_long_rows", "n_zero_rows",
                  "max_degree", "already_sorted", "n_plan_units", "n_split_rows", "plan_unit_nz",
                  "plan_groups", "plan_split_nz", "plan_team"):
            assert getattr(a.info, f) == getattr(b.info, f), f
        assert np.array_equal(a.block4(), b.block4())
        assert np.array_equal(a.perm(), b.perm())
        assert np.array_equal(a.plan(), b.plan())
        for u, v in zip(a.sorted_csr(), b.sorted_csr()):
            assert np.array_equal(u, v)
        Yb = b.matmul(X)
        assert np.array_equal(Ya.view(np.uint32), Yb.view(np.uint32))
        assert so.check(Yb, g.indptr, g.indices, g.values, X) <= TOL
        # the metadata in the state is upstream's partition of the sorted rows
        perm = po.degree_sort(g.indptr)
        sip, _, _ = po.permute_csr(g.indptr, g.indices, g.values, perm)
        assert np.array_equal(b.block4(), po.partition_closed_form(sip))
    finally:
        a.close()
        b.close()


def test_state_of_an_already_sorted_csr_without_split_rows(gpu, tmp_path):
    """No permutation and no private copy of the non-zeros: the handle aliases the caller's arrays."""
    deg = np.sort(np.random.default_rng(3).integers(0, 150, 2000))
    g = helpers.graph_from_degrees(deg, n_cols=3000, seed=3)
    X = np.random.default_rng(4).uniform(-1, 1, (g.n_cols, 20)).astype(np.float32)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1, plan_unit=384)
    assert a.info.already_sorted == 1 and a.info.n_split_rows == 0
    a.save_state(tmp_path / "s.accelstate")
    b = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).load_state(tmp_path / "s.accelstate")
    assert np.array_equal(a.matmul(X).view(np.uint32), b.matmul(X).view(np.uint32))
    a.close()
    b.close()


def test_state_of_another_csr_is_refused(gpu, tmp_path):
    g = graph(22)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    a.close()
    # same shape and row degrees, one column index changed
    idx2 = g.indices.copy()
    row = int(np.argmax(np.diff(g.indptr)))
    p = int(g.indptr[row])
    free = np.setdiff1d(np.arange(g.n_cols), idx2[g.indptr[row]:g.indptr[row + 1]])
    idx2[p] = free[0]
    b = gpu.AccelSpMM(g.indptr, idx2, g.values, g.n_cols)
    with pytest.raises(gpu.AccelError) as e:
        b.load_state(path)
    assert e.value.status == gpu._lib.ERR_META and "different CSR" in e.value.message
    # the handle is left un-preprocessed and still usable
    dX = gpu.DeviceBuffer(g.n_cols * 4 * 4)
    dY = gpu.DeviceBuffer(g.n_rows * 4 * 4)
    with pytest.raises(gpu.AccelError) as e:
        b.run(dX, dY, 4)
    assert e.value.status == gpu._lib.ERR_STATE
    b.preprocess()
    X = np.ones((g.n_cols, 4), np.float32)
    assert so.check(b.matmul(X), g.indptr, idx2, g.values, X) <= TOL
    b.close()
    # other dimensions
    g3 = graph(23, n_long=3)
    c = gpu.AccelSpMM(g3.indptr, g3.indices, g3.values, g3.n_cols)
    with pytest.raises(gpu.AccelError) as e:
        c.load_state(path)
    assert e.value.status == gpu._lib.ERR_META
    c.close()
    dX.close()
    dY.close()


def test_damaged_truncated_and_missing_files(gpu, tmp_path):
    g = graph(24)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    a.close()
    raw = bytearray(path.read_bytes())
    b = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)

    def refused(data, status):
        bad = tmp_path / "bad.accelstate"
        bad.write_bytes(bytes(data))
        with pytest.raises(gpu.AccelError) as e:
            b.load_state(bad)
        assert e.value.status == status, e.value

    flipped = bytearray(raw)
    flipped[len(raw) // 2] ^= 0x40                       # one bit in a stored array
    refused(flipped, gpu._lib.ERR_META)
    flipped = bytearray(raw)
    flipped[40] ^= 0x01                                  # one bit in the header
    refused(flipped, gpu._lib.ERR_META)
    refused(raw[: len(raw) - 100], gpu._lib.ERR_IO)      # truncated payload
    refused(raw[:50], gpu._lib.ERR_IO)                   # truncated header
    refused(raw + b"\0" * 8, gpu._lib.ERR_IO)            # longer than its header says
    refused(b"not a state file" * 40, gpu._lib.ERR_META)
    with pytest.raises(gpu.AccelError) as e:
        b.load_state(tmp_path / "nothing_here.accelstate")
    assert e.value.status == gpu._lib.ERR_IO
    b.load_state(path)                                   # the intact file still loads afterwards
    X = np.ones((g.n_cols, 8), np.float32)
    assert so.check(b.matmul(X), g.indptr, g.indices, g.values, X) <= TOL
    b.close()


def test_operator_mirror_uses_the_saved_state(gpu, tmp_path):
    """SpmmAccel loads <meta_dir>/<graph>.accelstate instead of preprocessing, as
    upstream's operator loads its metadata file (spmm_accel.cu:122)."""
    g0 = gpu.synthetic.cfg1()
    perm = po.degree_sort(g0.indptr)
    sip, six, sval = po.permute_csr(g0.indptr, g0.indices, g0.values, perm)
    X = gpu.synthetic.dense_operand("cfg1", g0.n_cols, 32)
    bufs = [gpu.DeviceBuffer.from_numpy(a) for a in (sip, six, sval, X)]
    vout = gpu.DeviceBuffer(g0.n_rows * 32 * 4)
    meta = tmp_path / "block_level_meta"
    meta.mkdir()
    outs = []
    for expect_loaded in (False, True):
        acc = gpu.SpmmAccel("cfg1", bufs[0], bufs[1], bufs[2], bufs[3], vout, g0.n_rows, g0.nnz, 32, meta_dir=meta)
        acc.save_state = True
        vout.fill_u32(0x7FC00000)
        assert acc.do_test(False, 32) == 0.0
        assert acc.state_loaded == expect_loaded
        outs.append(vout.to_numpy(np.float32, (g0.n_rows, 32)))
        acc.op.close()
    assert (meta / "cfg1.accelstate").exists()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    assert so.check(outs[1], sip, six, sval, X) <= TOL
    for b in bufs + [vout]:
        b.close()
