"""GPU preprocessing (degree sort, permuted CSR, block4 partition) is bit-exact
with the CPU oracle and with the reference's 16 golden .block4 files."""
import ctypes as C

import numpy as np
import pytest

import block4_codec
import helpers
from oracle import partition_oracle as po

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", block4_codec.names())
def test_gpu_partition_reproduces_golden(gpu, name):
    golden = block4_codec.load(name)
    indptr = po.indptr_from_degrees(po.degrees_from_block4(golden))
    got = gpu.block_level_partition.partition(indptr, backend="gpu")
    assert got.tobytes() == golden.tobytes()


@pytest.mark.parametrize("seed", range(6))
def test_gpu_partition_on_unsorted_rows(gpu, seed):
    """The walk also defines a result for rows that are not sorted (runs of equal
    degree, zero-degree rows anywhere); the kernels follow it."""
    rng = np.random.default_rng(seed)
    deg = np.repeat(rng.choice([0, 0, 1, 2, 5, 32, 33, 64, 96, 97, 129, 191, 192, 384, 385, 768, 5000],
                               size=700), rng.integers(1, 30, size=700))
    indptr = po.indptr_from_degrees(deg)
    got = gpu.block_level_partition.partition(indptr, backend="gpu")
    assert np.array_equal(got, po.partition_closed_form(indptr))
    assert np.array_equal(got, gpu.block_level_partition.partition(indptr, backend="host"))


def test_stage_on_gpu_writes_golden_file(gpu, tmp_path):
    graphs = tmp_path / "graphs"
    graphs.mkdir()
    for name in ("pubmed", "collab"):
        golden = block4_codec.load(name)
        (graphs / f"{name}.config").write_text("")
        po.indptr_from_degrees(po.degrees_from_block4(golden)).astype("<i4").tofile(graphs / f"{name}.new_indptr")
    done = gpu.block_level_partition.run_stage(graphs, tmp_path / "meta", verbose=False)
    assert set(done) == {"pubmed", "collab"}
    for name in done:
        assert (tmp_path / "meta" / f"{name}.block4").read_bytes() == block4_codec.load(name).tobytes()


def check_preprocess(gpu, g, plan_unit=None, plan_groups=None, plan_split=None, plan_team=None):
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_unit, plan_groups, plan_split,
                                                                         plan_team)
    if plan_team is not None:
        assert op.info.plan_team == (plan_team == 2)
    else:
        assert op.info.plan_team == (g.nnz < 512 * 1024)          # workgroup units for small matrices
    if plan_split is not None:
        # a wavefront never takes more than one unit; a workgroup takes whole rows up to the threshold
        assert op.info.plan_split_nz == (plan_split if op.info.plan_team else min(plan_split, op.info.plan_unit_nz))
    if plan_unit is not None:
        assert op.info.plan_unit_nz == plan_unit
    assert op.info.plan_groups == (plan_groups or 0)
    perm, sip, six, sval, b4 = helpers.expected_preprocess(g.indptr, g.indices, g.values,
                                                           op.info.plan_split_nz, op.info.plan_groups)
    assert np.array_equal(op.perm(), perm)
    ip, ix, v = op.sorted_csr()
    assert np.array_equal(ip, sip) and np.array_equal(ix, six) and np.array_equal(v, sval)
    assert op.block4().tobytes() == po.block4_to_bytes(b4)
    d = np.diff(g.indptr)
    info = op.info
    assert (info.rows, info.cols, info.nnz) == (g.n_rows, g.n_cols, g.nnz)
    assert info.n_blocks == len(b4)
    assert info.n_zero_rows == int((d == 0).sum()) and info.n_long_rows == int((d > 384).sum())
    assert info.n_long_blocks == int(np.sum(-(-d[d > 384] // 384)))
    assert info.max_degree == int(d.max(initial=0))
    assert info.n_split_rows == int((d > info.plan_split_nz).sum())
    op.check_block4(b4)
    return op


@pytest.mark.parametrize("seed", range(4))
def test_preprocess_mixed_degrees(gpu, seed):
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=7, zeros=9), seed=seed)
    op = check_preprocess(gpu, g)
    assert op.info.already_sorted == 0
    op.close()


def test_preprocess_workloads(gpu):
    for g in (gpu.synthetic.cfg1(), gpu.synthetic.cfg2(), gpu.synthetic.hub_graph_small()):
        check_preprocess(gpu, g).close()


def test_preprocess_needs_three_radix_passes(gpu):
    # a degree above 65535 exercises the third 8-bit pass of the sort
    deg = np.array([3, 70_000, 0, 3, 1, 300, 70_000, 2, 65_536, 1], dtype=np.int64)
    g = helpers.graph_from_degrees(deg, n_cols=80_000, seed=5)
    check_preprocess(gpu, g).close()


@pytest.mark.parametrize("n_long", [0, 4])
def test_already_sorted_input(gpu, n_long):
    """Input in upstream's *.new_* order: the sort is skipped, perm is the
    identity, and only rows with more than 384 non-zeros are regrouped."""
    g0 = helpers.graph_from_degrees(helpers.degree_mix(seed=2, n_long=n_long), seed=2)
    perm = po.degree_sort(g0.indptr)
    sip, six, sval = po.permute_csr(g0.indptr, g0.indices, g0.values, perm)
    op = gpu.AccelSpMM(sip, six, sval, g0.n_cols).preprocess()
    assert op.info.already_sorted == 1 and op.info.n_long_rows == n_long
    assert np.array_equal(op.perm(), np.arange(g0.n_rows))
    assert np.array_equal(op.block4(), po.partition_closed_form(sip))
    ip, ix, v = op.sorted_csr()
    gix, gval = po.group_long_rows(sip, six, sval, op.info.plan_split_nz, op.info.plan_groups)
    assert np.array_equal(ip, sip) and np.array_equal(ix, gix) and np.array_equal(v, gval)
    op.close()


def test_edge_shapes(gpu):
    empty = gpu.AccelSpMM(np.zeros(1, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 5).preprocess()
    assert empty.info.n_blocks == 0 and empty.block4().shape == (0, 4)
    assert empty.matmul(np.ones((5, 3), np.float32)).shape == (0, 3)
    empty.close()
    allzero = gpu.AccelSpMM(np.zeros(8, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 5).preprocess()
    assert allzero.info.n_blocks == 0 and allzero.info.n_zero_rows == 7
    assert np.array_equal(allzero.matmul(np.ones((5, 3), np.float32)), np.zeros((7, 3), np.float32))
    allzero.close()
    one = gpu.AccelSpMM(np.array([0, 2], np.int32), np.array([1, 3], np.int32),
                        np.array([2.0, -1.0], np.float32), 4).preprocess()
    assert one.block4().tolist() == [[2, 0, 0, (2 << 16) + 1]]
    X = np.arange(8, dtype=np.float32).reshape(4, 2)
    assert np.array_equal(one.matmul(X), (2 * X[1] - X[3])[None, :])
    one.close()


def test_bad_csr_is_rejected(gpu):
    lib = gpu._lib
    ok = helpers.graph_from_degrees([2, 3, 1], n_cols=6)
    cases = {
        "decreasing": (np.array([0, 3, 2, 6], np.int32), ok.indices, ok.values),
        "nonzero start": (np.array([1, 2, 5, 6], np.int32), ok.indices, ok.values),
        "wrong end": (np.array([0, 2, 4, 5], np.int32), ok.indices, ok.values),
        "column too large": (ok.indptr, np.array([0, 1, 2, 3, 6, 0], np.int32), ok.values),
        "negative column": (ok.indptr, np.array([0, 1, -1, 3, 4, 0], np.int32), ok.values),
    }
    for what, (ip, ix, v) in cases.items():
        op = gpu.AccelSpMM(ip, ix, v, 6)
        with pytest.raises(gpu.AccelError) as e:
            op.preprocess()
        assert e.value.status == lib.ERR_CSR, what
        with pytest.raises(gpu.AccelError) as e:      # and the handle stays unusable
            op.run(0, 0, 4)
        assert e.value.status == lib.ERR_STATE, what
        op.close()


def test_borrowed_csr_must_be_device_memory(gpu):
    """A CSR passed as device memory is read by kernels: host arrays, and device arrays
    smaller than the stated sizes, are refused before anything is launched."""
    import ctypes as C
    lib, E = gpu.lib(), gpu._lib
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=2, n_long=2), seed=2)
    host = [np.ascontiguousarray(a) for a in (g.indptr, g.indices, g.values)]
    dev = [gpu.DeviceBuffer.from_numpy(a) for a in host]
    h = C.c_void_p()

    def create(ip, ix, v, rows=g.n_rows, nnz=g.nnz):
        return lib.accel_create(C.c_void_p(ip), C.c_void_p(ix), C.c_void_p(v), rows, g.n_cols, nnz, E.PTR_DEVICE,
                                C.byref(h))
    addr = [d.address for d in dev]
    for k in range(3):                                     # each array in turn as a host address
        mixed = list(addr)
        mixed[k] = host[k].ctypes.data
        assert create(*mixed) == E.ERR_ARG and not h.value
        assert "not memory the GPU can access" in E.last_error()
    assert create(*addr, rows=g.n_rows + 1) == E.ERR_ARG   # indptr too small for one more row
    assert create(*addr, nnz=g.nnz + 1) == E.ERR_ARG       # idx and val too small
    assert "needs" in E.last_error()
    assert create(*addr) == 0 and h.value
    E.check(lib.accel_preprocess(h))
    # the arrays are asked about again when the handle is preprocessed: freed since, refused
    dev[1].close()
    small = gpu.DeviceBuffer(16)
    rc = lib.accel_preprocess(h)
    assert rc in (0, E.ERR_ARG)                            # 0 only if the address is still mapped and large enough
    if rc == E.ERR_ARG:
        assert "idx" in E.last_error()
    lib.accel_destroy(h)
    small.close()
    for d in (dev[0], dev[2]):
        d.close()


def test_stale_metadata_is_rejected(gpu):
    g = helpers.graph_from_degrees(np.sort(helpers.degree_mix(seed=1)), seed=1)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    b4 = op.block4()
    op.check_block4(b4)
    bad = b4.copy()
    bad[3, 2] += 1
    for wrong in (bad, b4[:-1]):
        with pytest.raises(gpu.AccelError) as e:
            op.check_block4(wrong)
        assert e.value.status == gpu._lib.ERR_META
    op.close()


def test_call_order_and_arguments(gpu):
    g = helpers.graph_from_degrees([2, 3, 1], n_cols=6)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, 6)
    with pytest.raises(gpu.AccelError) as e:
        op.run(0, 0, 4)
    assert e.value.status == gpu._lib.ERR_STATE
    op.preprocess()
    buf = gpu.DeviceBuffer(1024)
    for N in (0, -3):
        with pytest.raises(gpu.AccelError) as e:
            op.run(buf, buf, N)
        assert e.value.status == gpu._lib.ERR_ARG
    with pytest.raises(gpu.AccelError) as e:
        op.run(None, buf, 4)
    assert e.value.status == gpu._lib.ERR_ARG
    buf.close()
    op.close()


def check_plan(op, n_cols):
    """The launch plan covers every non-zero exactly once; units of whole rows stay
    inside one block4 entry and hold at most plan_unit non-zeros (or one row); pieces of
    split rows hold at most plan_unit non-zeros (the split threshold, if that is larger)
    of one column group and are queued on the die that owns that group.  With one queue
    (plan_queues == 1) the same order holds for the list as a whole."""
    unit, split, nq = op.info.plan_unit_nz, op.info.plan_split_nz, op.info.plan_queues
    assert nq in (1, 8)
    piece = max(unit, split)
    plan = op.plan().astype(np.int64)
    b4 = op.block4().astype(np.int64)
    sip, six, _ = op.sorted_csr()
    deg = np.diff(sip)
    assert plan.shape[0] % (4 * nq) == 0 and plan.shape[0] == op.info.n_plan_units   # queues x 4 wavefronts
    live = plan[plan[:, 3] != 0]
    short = live[live[:, 0] <= 384]
    long_ = live[live[:, 0] > 384]
    covered = np.zeros(six.size, dtype=np.int32)
    for x, y, z, w in long_:
        covered[z:z + w] += 1
        assert 0 < w <= piece and sip[y] <= z and z + w <= sip[y + 1] and deg[y] > split
    entry_of_row = {}
    for d, r, loc, info in b4[b4[:, 0] <= 384]:
        for q in range(info & 0xFFFF):
            entry_of_row[r + q] = (d, r, loc, info >> 16)
    for d, r, loc, info in short:
        n = info & 0xFFFF
        covered[loc:loc + d * n] += 1
        assert d <= split and (n * d <= unit or n == 1)
        ed, er, eloc, ew = entry_of_row[r]                       # same block4 entry, same fields
        assert ed == d and loc == sip[r] and (info >> 16) == ew
        assert entry_of_row[r + n - 1][1] == er
    if unit == 384:
        assert sorted(map(tuple, short)) == sorted(map(tuple, b4[b4[:, 0] <= split]))   # entries verbatim
    assert np.all(covered == 1)
    # queue of unit e is (e // 4) % 8 (one queue: 0)
    queue = (np.arange(plan.shape[0]) // 4) % nq
    # the plan orders by the caller's row id in bands: the id's top 16 bits
    shift = 0
    while (max(deg.size, 1) - 1) >> shift >= 65536:
        shift += 1
    n_split = int((deg > split).sum())
    last = {}
    for e in np.flatnonzero((plan[:, 3] != 0) & (plan[:, 0] > 384)):
        x, y, z, w = plan[e]
        groups = po.row_groups(int(deg[y]), op.info.plan_groups)
        fine = po.column_group(six[z:z + w], groups)
        assert np.all(fine == fine[0]) and fine[0] % nq == queue[e]  # one group, on its die
        # a die takes the rows with the most groups first and its groups in turn; inside a group
        # the rows follow the caller's row ids (8-group rows) or come largest first (longer rows)
        key = (-groups, int(fine[0]),
               int(op.perm()[y]) >> shift if groups == 8 else (deg.size - 1 - int(y)) >> shift)
        assert deg.size - n_split <= y
        assert key >= last.get(queue[e], (-65, 0, -1))
        last[queue[e]] = key
    # partial-sum slots: 0 .. n-1, each once, contiguous per row in row order
    slots = long_[:, 0] - 385
    assert sorted(slots.tolist()) == list(range(len(long_)))
    order = np.argsort(slots)
    assert np.all(np.diff(long_[order, 1]) >= 0)
    # whole-row units: behind the pieces in every queue, the eight queues taking consecutive
    # shares of the order of the caller's row ids (of each unit's first row); inside a queue
    # they keep that order, except that the last 2,048 light units of the share (all of them
    # if there are fewer) are held back to the very end
    perm = op.perm()
    light_nz = max(24, unit // 4)
    keys = []
    for q in range(nq):
        mine = plan[queue == q]
        mine = mine[mine[:, 3] != 0]
        is_short = mine[:, 0] <= 384
        n_pieces = int((~is_short).sum())
        assert not is_short[:n_pieces].any() and is_short[n_pieces:].all()
        mine = mine[n_pieces:]
        k = perm[mine[:, 1]] >> shift
        light = mine[:, 0] * (mine[:, 3] & 0xFFFF) <= light_nz
        n_tail = min(2048, int(light.sum()))
        in_line = len(k) - n_tail
        assert light[in_line:].all()
        assert np.all(np.diff(k[:in_line]) >= 0) and np.all(np.diff(k[in_line:]) >= 0)
        if shift == 0:
            assert np.all(np.diff(k[:in_line]) > 0) and np.all(np.diff(k[in_line:]) > 0)
        if n_tail and light[:in_line].any():             # held back: the light units with the highest ids
            assert k[in_line:].min() >= k[:in_line][light[:in_line]].max()
        keys.append(k)
    for q in range(nq - 1):                             # queue q's rows all precede queue q + 1's
        later = np.concatenate(keys[q + 1:])
        if keys[q].size and later.size:
            assert keys[q].max() <= later.min()
    # ... and the shares level the load: cost = non-zeros + rows + 8 per unit, + 8 per piece
    load = np.zeros(nq)
    for e in np.flatnonzero(plan[:, 3] != 0):
        x, y, z, w = plan[e]
        load[queue[e]] += (w + 9) if x > 384 else (x + 1) * (w & 0xFFFF) + 8
    heaviest_unit = 384 + 64 + 8
    short_load = np.array([sum((d + 1) * (i & 0xFFFF) + 8 for d, r, l, i in plan[queue == q] if 0 < d <= 384 and i)
                           for q in range(nq)])
    with_short = short_load > 0
    if with_short.sum() > 1:
        # queues that received whole-row units end up within a few units of each other
        assert load[with_short].max() - load[with_short].min() <= 8 * heaviest_unit + 0.02 * load.max()
        # and none of them is lighter than a queue that holds pieces only
        assert load[~with_short].min(initial=np.inf) >= load[with_short].min() - 8 * heaviest_unit


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("seed,n_long", [(0, 0), (1, 3), (2, 9)])
def test_launch_plan(gpu, seed, n_long, team):
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=n_long), seed=seed)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team)
    assert (op.info.plan_unit_nz, op.info.plan_split_nz) == ((48, 384) if team == 2 else (48, 48))
    assert op.info.plan_queues == 8                      # the whole GPU: one queue per die
    check_plan(op, g.n_cols)
    op.close()


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("seed,n_long", [(3, 0), (4, 9)])
def test_launch_plan_in_one_queue(gpu, seed, n_long, team):
    """The layout for a device that is not the whole GPU (a partition, where "workgroup i
    runs on die i % 8" does not hold), forced here: the same units in plain order, column
    group after column group, and the same product."""
    from oracle import spmm_oracle as so
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=n_long, zeros=5), seed=seed)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team, plan_queues=1)
    assert op.info.plan_queues == 1
    check_plan(op, g.n_cols)
    ref = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=team)
    assert np.array_equal(op.block4(), ref.block4()) and np.array_equal(op.perm(), ref.perm())
    assert sorted(map(tuple, op.plan()[op.plan()[:, 3] != 0])) == sorted(map(tuple, ref.plan()[ref.plan()[:, 3] != 0]))
    for N in (16, 64, 100):
        X = np.random.default_rng(N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
        Y = op.matmul(X)
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL
        assert np.array_equal(Y.view(np.uint32), ref.matmul(X).view(np.uint32))   # same units, same sums
    with pytest.raises(gpu.AccelError) as e:
        gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_queues=4)
    assert e.value.status == gpu._lib.ERR_ARG
    op.close()
    ref.close()


def test_launch_plan_row_bands(gpu):
    """More than 65,536 rows: the plan orders by bands of row ids (the id's top 16 bits)."""
    rng = np.random.default_rng(21)
    deg = rng.integers(0, 9, 140_000)
    deg[rng.integers(0, deg.size, 40)] = rng.integers(200, 3000, 40)
    g = helpers.graph_from_degrees(deg, n_cols=5000, seed=21)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=1)
    check_plan(op, g.n_cols)
    X = rng.uniform(-1, 1, (g.n_cols, 8)).astype(np.float32)
    from oracle import spmm_oracle as so
    assert so.check(op.matmul(X), g.indptr, g.indices, g.values, X) <= so.TOL
    op.close()


def test_near_diagonal_matrices_keep_mid_rows_whole(gpu):
    """The split threshold is 192 for a large matrix, unless most of its non-zeros lie near the
    diagonal: then rows of up to 384 non-zeros stay whole (sampled on the GPU)."""
    from oracle import spmm_oracle as so
    rng = np.random.default_rng(33)
    n, d = 60_000, 10
    deg = np.full(n, d)
    deg[rng.integers(0, n, 300)] = rng.integers(200, 380, 300)
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int32)
    rows_of = np.repeat(np.arange(n), deg)
    values = rng.uniform(-1, 1, rows_of.size).astype(np.float32)
    X = rng.uniform(-1, 1, (n, 16)).astype(np.float32)
    for kind, want in (("band", 384), ("uniform", 192)):
        if kind == "band":
            cols = np.clip(rows_of + rng.integers(-600, 601, rows_of.size), 0, n - 1)
        else:
            cols = rng.integers(0, n, rows_of.size)
        op = gpu.AccelSpMM(indptr, cols.astype(np.int32), values, n).preprocess()
        assert op.info.nnz >= 512 * 1024 and op.info.plan_team == 0
        assert op.info.plan_split_nz == want, kind
        assert op.info.n_split_rows == int((deg > want).sum())
        assert so.check(op.matmul(X), indptr, cols.astype(np.int32), values, X) <= so.TOL
        op.close()
    # an explicit threshold is never overridden
    op = gpu.AccelSpMM(indptr, cols.astype(np.int32), values, n).preprocess(plan_split=100)
    assert op.info.plan_split_nz == 100
    op.close()


def test_launch_plan_hub_graph(gpu):
    g = gpu.synthetic.hub_graph_small()
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    check_plan(op, g.n_cols)
    op.close()


@pytest.mark.parametrize("groups", [8, 16, 32, 64])
def test_plan_column_groups(gpu, groups):
    from oracle import spmm_oracle as so
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=8, n_long=12), n_cols=9000, seed=8)
    assert po.row_groups(385) == 8 and po.row_groups(1535) == 8 and po.row_groups(1536) == 16
    assert po.row_groups(3072) == 32 and po.row_groups(6144) == 64 and po.row_groups(10 ** 6) == 64
    op = check_preprocess(gpu, g, plan_groups=groups)
    check_plan(op, g.n_cols)
    X = np.random.default_rng(groups).uniform(-1, 1, (g.n_cols, 48)).astype(np.float32)
    Y = op.matmul(X)
    assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL
    op.close()
    with pytest.raises(gpu.AccelError) as e:
        gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_groups=12)
    assert e.value.status == gpu._lib.ERR_ARG


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("unit", [16, 50, 96, 200, 384])
def test_plan_unit_sizes(gpu, unit, team):
    """Smaller units change the plan and which rows are stored grouped, never the
    block4 metadata or the product; with a wavefront or a workgroup per unit."""
    from oracle import spmm_oracle as so
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=6, n_long=5), seed=6)
    op = check_preprocess(gpu, g, plan_unit=unit, plan_team=team)
    check_plan(op, g.n_cols)
    for N in (64, 10):
        X = np.random.default_rng(unit + N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
        Y = op.matmul(X)
        assert np.isfinite(Y).all()
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL
    op.close()
    with pytest.raises(gpu.AccelError) as e:
        gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_unit=1000)
    assert e.value.status == gpu._lib.ERR_ARG
    with pytest.raises(gpu.AccelError) as e:
        gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess(plan_team=3)
    assert e.value.status == gpu._lib.ERR_ARG


def test_plan_groups_follow_row_length(gpu):
    """Automatic rule: rows of 385..1535 non-zeros use 8 column groups, longer rows
    16, 32 or 64; the plan serves the rows with the most groups first."""
    from oracle import spmm_oracle as so
    deg = np.array([5, 400, 1500, 1600, 3100, 6200, 12500, 20000, 1, 0, 64, 3000], dtype=np.int64)
    g = helpers.graph_from_degrees(deg, n_cols=30_000, seed=3)
    op = check_preprocess(gpu, g)
    assert op.info.plan_groups == 0
    check_plan(op, g.n_cols)
    X = np.random.default_rng(3).standard_normal((g.n_cols, 32)).astype(np.float32)
    assert so.check(op.matmul(X), g.indptr, g.indices, g.values, X) <= so.TOL
    op.close()


@pytest.mark.parametrize("team", [1, 2])
@pytest.mark.parametrize("unit,split", [(384, 100), (384, 200), (128, 40), (96, 384)])
def test_plan_split_threshold(gpu, unit, split, team):
    from oracle import spmm_oracle as so
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=9, n_long=6), seed=9)
    op = check_preprocess(gpu, g, plan_unit=unit, plan_split=split, plan_team=team)
    check_plan(op, g.n_cols)
    X = np.random.default_rng(split).uniform(-1, 1, (g.n_cols, 40)).astype(np.float32)
    assert so.check(op.matmul(X), g.indptr, g.indices, g.values, X) <= so.TOL
    op.close()


@pytest.mark.parametrize("seed", range(16))
def test_plan_options_in_combination(gpu, seed):
    """Unit size, split threshold, column groups and who works on a unit, drawn together:
    the metadata never moves, the plan stays a cover of the non-zeros, the product holds."""
    from oracle import spmm_oracle as so
    rng = np.random.default_rng(1000 + seed)
    unit = int(rng.choice([16, 24, 48, 77, 128, 250, 384]))
    split = int(rng.choice([16, 40, 96, 192, 300, 384]))
    groups = int(rng.choice([0, 8, 16, 32, 64]))
    team = int(rng.choice([1, 2]))
    deg = helpers.degree_mix(seed=seed, n_long=int(rng.integers(0, 8)), zeros=int(rng.integers(0, 9)))
    if seed % 4 == 3:
        deg = np.concatenate([deg, [int(rng.integers(5000, 30000))]])      # one hub row
    g = helpers.graph_from_degrees(deg, seed=seed)
    op = check_preprocess(gpu, g, plan_unit=unit, plan_split=split, plan_groups=groups or None, plan_team=team)
    check_plan(op, g.n_cols)
    for N in (int(rng.choice([1, 7, 20])), int(rng.choice([64, 100, 130]))):
        X = np.random.default_rng(seed + N).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
        Y = op.matmul(X)
        assert np.isfinite(Y).all()
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL, (unit, split, groups, team, N)
    op.close()


def test_device_plumbing(gpu):
    import ctypes as C
    a = np.arange(100_003, dtype=np.uint32)
    src, dst = gpu.DeviceBuffer.from_numpy(a), gpu.DeviceBuffer(a.nbytes)
    dst.fill_u32(0xDEADBEEF)
    assert np.all(dst.to_numpy(np.uint32, a.shape) == 0xDEADBEEF)
    gpu._lib.check(gpu.lib().accel_dev_copy_u32(C.c_void_p(dst.address), C.c_void_p(src.address), a.size, None))
    gpu._lib.check(gpu.lib().accel_stream_sync(None))
    assert np.array_equal(dst.to_numpy(np.uint32, a.shape), a)
    with pytest.raises(ValueError):
        dst.to_numpy(np.uint32, (a.size + 1,))
    # the two kernels behind these calls get the same protection as the operator's: no launch on
    # a host address or past the end of an allocation
    E, L = gpu._lib, gpu.lib()
    assert L.accel_dev_fill_u32(C.c_void_p(a.ctypes.data), 0, a.size, None) == E.ERR_ARG
    assert L.accel_dev_fill_u32(C.c_void_p(dst.address), 0, a.size + 1, None) == E.ERR_ARG
    assert L.accel_dev_copy_u32(C.c_void_p(dst.address), C.c_void_p(a.ctypes.data), a.size, None) == E.ERR_ARG
    assert L.accel_dev_copy_u32(C.c_void_p(dst.address + 8), C.c_void_p(src.address), a.size, None) == E.ERR_ARG
    assert np.array_equal(dst.to_numpy(np.uint32, a.shape), a)
    src.close()
    dst.close()
    dst.close()                                  # closing twice is harmless
