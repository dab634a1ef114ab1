"""Saved preprocessing state: accel_save_state / accel_load_state.

The state holds the degree-sort order and the plan options; everything else is rebuilt on
load.  A state saved for a CSR and loaded into a new handle on the same CSR must give the
same metadata and the same bits of Y as preprocessing again; a state whose order is not
the degree order of the handle's CSR, a damaged or a truncated file must be refused and
leave the handle un-preprocessed.
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
    assert path.stat().st_size <= 4 * g.n_rows + 128      # the permutation and a small header
    Ya = a.matmul(X)
    b = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).load_state(path)
    try:
        for f in ("rows", "cols", "nnz", "n_blocks", "n_long_blocks", "n_long_rows", "n_zero_rows",
                  "max_degree", "already_sorted", "n_plan_units", "n_split_rows", "plan_unit_nz",
                  "plan_groups", "plan_split_nz", "plan_team", "plan_queues"):
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
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_groups=16)
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    a.close()
    # same shape, two rows of different degree exchanged: the saved order is not this CSR's
    deg = np.diff(g.indptr)
    i, j = int(np.argmax(deg)), int(np.argmin(deg))
    deg2 = deg.copy()
    deg2[i], deg2[j] = deg[j], deg[i]
    g2 = helpers.graph_from_degrees(deg2, n_cols=g.n_cols, seed=5)
    assert g2.indices.size == g.indices.size
    b = gpu.AccelSpMM(g2.indptr, g2.indices, g2.values, g2.n_cols)
    with pytest.raises(gpu.AccelError) as e:
        b.load_state(path)
    assert e.value.status == gpu._lib.ERR_META and "degree order" in e.value.message
    # the handle is left un-preprocessed, with its own options, and still usable
    dX = gpu.DeviceBuffer(g.n_cols * 4 * 4)
    dY = gpu.DeviceBuffer(g.n_rows * 4 * 4)
    with pytest.raises(gpu.AccelError) as e:
        b.run(dX, dY, 4)
    assert e.value.status == gpu._lib.ERR_STATE
    b.preprocess()
    assert b.info.plan_groups == 0                        # not the 16 of the refused state
    X = np.ones((g.n_cols, 4), np.float32)
    assert so.check(b.matmul(X), g2.indptr, g2.indices, g2.values, X) <= TOL
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


def test_state_serves_any_csr_with_the_same_row_degrees(gpu, tmp_path):
    """The stored order depends on the row degrees only and nothing else in the file is
    used to index memory: a CSR with the same degrees and other columns and values loads
    the state and computes its own product, bit for bit what a fresh preprocessing gives."""
    g = graph(25)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    a.close()
    g2 = helpers.graph_from_degrees(np.diff(g.indptr), n_cols=g.n_cols, seed=99)
    assert np.array_equal(g2.indptr, g.indptr) and not np.array_equal(g2.indices, g.indices)
    X = np.random.default_rng(1).uniform(-1, 1, (g.n_cols, 24)).astype(np.float32)
    b = gpu.AccelSpMM(g2.indptr, g2.indices, g2.values, g2.n_cols).load_state(path)
    c = gpu.AccelSpMM(g2.indptr, g2.indices, g2.values, g2.n_cols).preprocess()
    Yb = b.matmul(X)
    assert so.check(Yb, g2.indptr, g2.indices, g2.values, X) <= TOL
    assert np.array_equal(Yb.view(np.uint32), c.matmul(X).view(np.uint32))
    assert np.array_equal(b.plan(), c.plan())
    b.close()
    c.close()


def test_an_order_that_is_not_the_sort_is_refused(gpu, tmp_path):
    """Every way a stored permutation can be wrong is caught by the check on the GPU: an entry
    out of range, a row twice, two rows of equal degree exchanged (not the stable order), two
    rows of different degree exchanged."""
    import struct
    g = graph(26)
    a = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    path = tmp_path / "g.accelstate"
    a.save_state(path)
    perm = a.perm()
    a.close()
    raw = path.read_bytes()
    head = len(raw) - 4 * g.n_rows
    assert np.array_equal(np.frombuffer(raw[head:], "<i4"), perm)
    deg = np.diff(g.indptr)[perm]
    same = int(np.flatnonzero(deg[1:] == deg[:-1])[0])      # sorted rows same, same + 1 have equal degree
    diff = int(np.flatnonzero(deg[1:] != deg[:-1])[0])
    b = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)
    cases = {}
    p = perm.copy(); p[7] = g.n_rows; cases["out of range"] = p
    p = perm.copy(); p[7] = -1; cases["negative"] = p
    p = perm.copy(); p[9] = p[8]; cases["a row twice"] = p
    p = perm.copy(); p[same], p[same + 1] = perm[same + 1], perm[same]; cases["ties out of order"] = p
    p = perm.copy(); p[diff], p[diff + 1] = perm[diff + 1], perm[diff]; cases["degrees out of order"] = p
    for what, p in cases.items():
        bad = tmp_path / "bad.accelstate"
        bad.write_bytes(raw[:head] + p.astype("<i4").tobytes())
        with pytest.raises(gpu.AccelError) as e:
            b.load_state(bad)
        assert e.value.status == gpu._lib.ERR_META, what
    b.load_state(path)
    X = np.ones((g.n_cols, 8), np.float32)
    assert so.check(b.matmul(X), g.indptr, g.indices, g.values, X) <= TOL
    b.close()


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

    for at in (len(raw) // 2, len(raw) - 1, 200):
        flipped = bytearray(raw)
        flipped[at] ^= 0x40                              # one bit in the stored order
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
    """With save_state on, SpmmAccel loads <meta_dir>/<graph>.accelstate instead of sorting,
    as upstream's operator loads its metadata file (spmm_accel.cu:122); without it the file
    is not looked at."""
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
    acc = gpu.SpmmAccel("cfg1", bufs[0], bufs[1], bufs[2], bufs[3], vout, g0.n_rows, g0.nnz, 32, meta_dir=meta)
    acc.do_test(False, 32)
    assert not acc.state_loaded                          # the cache is opt-in
    acc.op.close()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    assert so.check(outs[1], sip, six, sval, X) <= TOL
    for b in bufs + [vout]:
        b.close()
