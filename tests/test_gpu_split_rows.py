"""Where the partial sums of split rows meet: in the gather kernel itself (the wavefront, or
workgroup, that stores a row's last piece adds the row up; one launch, as upstream's run is,
spmm_accel.cu:104-108) or in a second kernel.  Both must give the product within the
tolerance; each must give the same bits on every run, whichever piece happens to finish
last, because the slots are added in a fixed order."""
import numpy as np
import pytest

import helpers
from oracle import spmm_oracle as so

pytestmark = pytest.mark.gpu

TOL = 1e-5


def graph_with_split_rows(seed, n_long=30):
    return helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=n_long, zeros=5), seed=seed)


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("N", [1, 4, 16, 33, 64, 100, 128, 256, 300])
def test_both_ways_of_adding_split_rows_up(gpu, team, N):
    g = graph_with_split_rows(51)
    X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    Ys = {}
    for mode in (1, 2):
        op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team, plan_reduce=mode)
        assert op.info.n_split_rows > 0
        Y = op.matmul(X)
        assert np.isfinite(Y).all(), f"mode {mode}: some row of Y was not written"
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= TOL, f"mode {mode}"
        Ys[mode] = Y
        op.close()
    # rows that are not split do not depend on the mode at all
    whole = np.diff(g.indptr) <= 48
    assert np.array_equal(Ys[1][whole].view(np.uint32), Ys[2][whole].view(np.uint32))


@pytest.mark.parametrize("workload,N", [("cfg2", 16), ("cfg2", 64), ("hub", 256), ("hub", 64), ("long", 100)])
def test_one_launch_gives_the_same_bits_every_time(gpu, workload, N):
    """Many launches back to back, the partial sums and the per-row counters reused by each:
    every launch must leave the bits of the first (a piece counted in before its sums have
    arrived, or a counter not back at zero, would show up here), and they must be right."""
    if workload == "cfg2":
        g = gpu.synthetic.cfg2()
    elif workload == "hub":
        g = gpu.synthetic.hub_graph_small()
    else:
        g = helpers.graph_from_degrees(np.array([1, 100_000, 0, 2, 384, 385, 40_000, 700]), n_cols=120_000, seed=9)
    X = gpu.synthetic.dense_operand(g.name if workload != "long" else "long", g.n_cols, N)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_reduce=1)
    assert op.info.n_split_rows > 0
    dX = gpu.DeviceBuffer.from_numpy(X)
    dY = gpu.DeviceBuffer(g.n_rows * N * 4)
    dY.fill_u32(0x7FC00000)
    op.run(dX, dY, N)
    op.synchronize()
    first = dY.to_numpy(np.float32, (g.n_rows, N))
    assert so.check(first, g.indptr, g.indices, g.values, X) <= TOL
    for rep in range(40):
        dY.fill_u32(0x7FC00000)
        for _ in range(5):                                # queued back to back, no wait in between
            op.run(dX, dY, N)
        op.synchronize()
        assert np.array_equal(dY.to_numpy(np.float32, (g.n_rows, N)).view(np.uint32), first.view(np.uint32)), rep
    # the second kernel, for comparison (it groups the slots of the longest rows differently,
    # so the bits may differ there; both are within the tolerance)
    ref = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_reduce=2)
    dY.fill_u32(0x7FC00000)
    ref.run(dX, dY, N)
    ref.synchronize()
    assert so.check(dY.to_numpy(np.float32, (g.n_rows, N)), g.indptr, g.indices, g.values, X) <= TOL
    dX.close(); dY.close(); op.close(); ref.close()


def test_epilogue_strides_and_panels_in_one_launch(gpu):
    g = graph_with_split_rows(52, n_long=12)
    rng = np.random.default_rng(3)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1, plan_reduce=1)
    for N, ld, panel in ((50, 64, 0), (128, 0, 64), (96, 128, 32), (17, 0, 0)):
        step = ld or N
        X = rng.uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
        bias = rng.uniform(-1, 1, N).astype(np.float32)
        Xp = np.zeros((g.n_cols, step), np.float32); Xp[:, :N] = X
        dX, dB = gpu.DeviceBuffer.from_numpy(Xp), gpu.DeviceBuffer.from_numpy(bias)
        dY = gpu.DeviceBuffer(g.n_rows * step * 4)
        dY.fill_u32(0x7FC00000)
        op.set_panel(panel)
        op.run_ex(dX, dY, N, ld=ld, bias=dB, relu=True)
        op.synchronize()
        Y = dY.to_numpy(np.float32, (g.n_rows, step))
        R, S = so.spmm_fp64(g.indptr, g.indices, g.values, X)
        want = np.maximum(R + bias.astype(np.float64), 0.0)
        assert np.max(np.abs(Y[:, :N] - want) / np.maximum(S + np.abs(bias), 1e-30)) <= TOL, (N, ld, panel)
        if step > N:
            assert np.isnan(Y[:, N:]).all()               # the padding is never written
        for b in (dX, dB, dY):
            b.close()
    op.close()


def test_the_library_chooses_by_the_number_of_pieces(gpu):
    """Up to 16,384 pieces the gather kernel adds the rows up itself (a second launch would
    cost more); beyond, a second kernel does."""
    g = graph_with_split_rows(54, n_long=4)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1)
    assert 0 < op.info.n_plan_pieces <= 16384 and op.info.plan_reduce == 1
    assert op.info.n_plan_pieces == int((op.plan()[:, 0] > 384).sum())
    op.close()
    many = helpers.graph_from_degrees(np.full(2100, 400), n_cols=3000, seed=1)     # 8 pieces per row
    op = gpu.AccelSpMM(many.indptr, many.indices, many.values, many.n_cols).preprocess(plan_team=1)
    assert op.info.n_plan_pieces == 2100 * 8 and op.info.plan_reduce == 2
    X = np.ones((many.n_cols, 8), np.float32)
    assert so.check(op.matmul(X), many.indptr, many.indices, many.values, X) <= TOL
    op.close()
    op = gpu.AccelSpMM(many.indptr, many.indices, many.values, many.n_cols).preprocess(plan_team=1, plan_reduce=1)
    assert op.info.plan_reduce == 1
    assert so.check(op.matmul(X), many.indptr, many.indices, many.values, X) <= TOL
    op.close()


def test_setter_refuses_unknown_modes(gpu):
    g = graph_with_split_rows(53, n_long=2)
    with pytest.raises(gpu.AccelError) as e:
        gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_reduce=3)
    assert e.value.status == gpu._lib.ERR_ARG
