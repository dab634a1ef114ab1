"""accel_run on caller-owned HIP streams and inside a captured HIP graph: the run
path launches kernels only (no synchronisation, no allocation once the scratch
buffer for that N exists), so it can be replayed from a graph."""
import ctypes as C

import numpy as np
import pytest

import helpers
from oracle import spmm_oracle as so

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip(gpu):
    gpu.lib()                                    # the HIP runtime the library itself uses
    h = C.CDLL("libamdhip64.so.7")
    for name in ("hipStreamCreate", "hipStreamDestroy", "hipStreamSynchronize", "hipStreamBeginCapture",
                 "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch", "hipGraphExecDestroy",
                 "hipGraphDestroy", "hipMemGetInfo", "hipDeviceSynchronize"):
        getattr(h, name).restype = C.c_int
    return h


def ok(rc):
    assert rc == 0, f"HIP call failed with {rc}"


def make_case(gpu, seed, N):
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=seed, n_long=6, zeros=7), seed=seed)
    X = np.random.default_rng(seed).uniform(-1, 1, (g.n_cols, N)).astype(np.float32)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    return g, X, op


def test_two_streams_two_handles(gpu, hip):
    s1, s2 = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s1)))
    ok(hip.hipStreamCreate(C.byref(s2)))
    cases = [make_case(gpu, 31, 64), make_case(gpu, 32, 100)]
    bufs = []
    for (g, X, op), s in zip(cases, (s1, s2)):
        dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * X.shape[1] * 4)
        dY.fill_u32(0x7FC00000)
        bufs.append((dX, dY))
    gpu._lib.check(gpu.lib().accel_stream_sync(None))
    for _ in range(3):                                    # interleaved launches on both streams
        for (g, X, op), (dX, dY), s in zip(cases, bufs, (s1, s2)):
            op.run(dX, dY, X.shape[1], stream=s.value)
    ok(hip.hipStreamSynchronize(s1))
    ok(hip.hipStreamSynchronize(s2))
    for (g, X, op), (dX, dY) in zip(cases, bufs):
        Y = dY.to_numpy(np.float32, (g.n_rows, X.shape[1]))
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL
        dX.close(); dY.close(); op.close()
    ok(hip.hipStreamDestroy(s1))
    ok(hip.hipStreamDestroy(s2))


def test_two_host_threads_two_handles(gpu):
    """Distinct handles are independent: two host threads create, preprocess, run and
    check their own operator at the same time; errors are reported per thread."""
    import threading
    results, errors = {}, {}

    def worker(tag, seed, N):
        try:
            for rep in range(3):
                g, X, op = make_case(gpu, seed + rep, N)
                Y = op.matmul(X)
                results[(tag, rep)] = so.check(Y, g.indptr, g.indices, g.values, X)
                op.close()
            # an error on this thread must not show up as the other thread's message
            with pytest.raises(gpu.AccelError) as e:
                gpu.AccelSpMM(np.array([0, 2, 1], np.int32), np.zeros(1, np.int32), np.zeros(1, np.float32), 4)\
                    .preprocess()
            errors[tag] = str(e.value)
        except BaseException as exc:                      # surfaced by the assertions below
            errors[tag] = f"worker failed: {exc!r}"

    threads = [threading.Thread(target=worker, args=("a", 40, 64)),
               threading.Thread(target=worker, args=("b", 50, 24))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
        assert not t.is_alive()
    assert len(results) == 6 and all(v <= so.TOL for v in results.values()), (results, errors)
    assert all("indptr" in errors[t] for t in ("a", "b")), errors


def test_graph_capture_and_replay(gpu, hip):
    g, X, op = make_case(gpu, 33, 64)
    N = 64
    dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * N * 4)
    op.run(dX, dY, N)                                     # eager warm-up: allocates the scratch for this N
    op.synchronize()
    eager = dY.to_numpy(np.float32, (g.n_rows, N))
    s = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s)))
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(s, 0))                   # hipStreamCaptureModeGlobal
    op.run(dX, dY, N, stream=s.value)
    ok(hip.hipStreamEndCapture(s, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0))
    for rep in range(4):
        dY.fill_u32(0x7FC00000)                           # eager work between replays
        op.synchronize()
        ok(hip.hipGraphLaunch(gexec, s))
        ok(hip.hipStreamSynchronize(s))
        Y = dY.to_numpy(np.float32, (g.n_rows, N))
        assert np.array_equal(Y, eager), f"replay {rep} differs from the eager result"
    ok(hip.hipGraphExecDestroy(gexec))
    ok(hip.hipGraphDestroy(graph))
    ok(hip.hipStreamDestroy(s))
    dX.close(); dY.close(); op.close()


def test_captured_graph_sees_updated_values(gpu, hip):
    """accel_update_values rewrites the sorted copy in place: a graph captured before the
    update computes with the new values when it is replayed."""
    g, X, op = make_case(gpu, 35, 48)
    N = 48
    assert op.info.n_split_rows > 0
    dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * N * 4)
    op.run(dX, dY, N)
    op.synchronize()
    s = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s)))
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(s, 0))
    op.run(dX, dY, N, stream=s.value)
    ok(hip.hipStreamEndCapture(s, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0))
    for seed in (1, 2, 3):
        v = np.random.default_rng(seed).uniform(-1, 1, g.values.size).astype(np.float32)
        op.update_values(v)
        dY.fill_u32(0x7FC00000)
        op.synchronize()
        ok(hip.hipGraphLaunch(gexec, s))
        ok(hip.hipStreamSynchronize(s))
        Y = dY.to_numpy(np.float32, (g.n_rows, N))
        assert so.check(Y, g.indptr, g.indices, v, X) <= so.TOL, f"replay after update {seed}"
        op.run(dX, dY, N)
        op.synchronize()
        assert np.array_equal(Y, dY.to_numpy(np.float32, (g.n_rows, N)))   # eager run: same bits
    ok(hip.hipGraphExecDestroy(gexec))
    ok(hip.hipGraphDestroy(graph))
    ok(hip.hipStreamDestroy(s))
    dX.close(); dY.close(); op.close()


def test_second_stream_waits_for_the_first_on_the_device(gpu, hip):
    """The partial-sum buffer of a handle is shared by its runs: a run on another stream
    than the previous one is ordered behind it on the device (no error, no host wait), so
    runs queued on two streams give what they give one after the other."""
    g = gpu.synthetic.cfg2()
    N = 128
    X = gpu.synthetic.dense_operand("cfg2", g.n_cols, N)
    X2 = np.ascontiguousarray(-2.0 * X)
    op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    assert op.info.n_split_rows > 0
    dX, dX2 = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer.from_numpy(X2)
    dY, dY2 = gpu.DeviceBuffer(g.n_rows * N * 4), gpu.DeviceBuffer(g.n_rows * N * 4)
    op.run(dX, dY, N)
    op.run(dX2, dY2, N)
    op.synchronize()
    want, want2 = dY.to_numpy(np.float32, (g.n_rows, N)), dY2.to_numpy(np.float32, (g.n_rows, N))
    assert so.check(want, g.indptr, g.indices, g.values, X) <= so.TOL
    s1, s2 = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s1)))
    ok(hip.hipStreamCreate(C.byref(s2)))
    for rep in range(3):
        dY.fill_u32(0x7FC00000)
        dY2.fill_u32(0x7FC00000)
        op.synchronize()
        for _ in range(100):                              # some 15 ms of queued work on s1
            op.run(dX, dY, N, stream=s1.value)
        op.run(dX2, dY2, N, stream=s2.value)              # queued at once; waits on the device
        for _ in range(20):                               # and back and forth, never waiting on the host
            op.run(dX, dY, N, stream=s1.value)
            op.run(dX2, dY2, N, stream=s2.value)
        ok(hip.hipStreamSynchronize(s1))
        ok(hip.hipStreamSynchronize(s2))
        assert np.array_equal(dY.to_numpy(np.float32, (g.n_rows, N)), want), f"round {rep}, stream 1"
        assert np.array_equal(dY2.to_numpy(np.float32, (g.n_rows, N)), want2), f"round {rep}, stream 2"
    # a stream that is gone does not break the next run (the handle waits for the device instead)
    op.run(dX, dY, N, stream=s1.value)
    ok(hip.hipStreamSynchronize(s1))
    ok(hip.hipStreamDestroy(s1))
    op.run(dX2, dY2, N, stream=s2.value)
    ok(hip.hipStreamSynchronize(s2))
    assert np.array_equal(dY2.to_numpy(np.float32, (g.n_rows, N)), want2)
    ok(hip.hipStreamDestroy(s2))
    for b in (dX, dX2, dY, dY2):
        b.close()
    op.close()


def test_value_update_is_ordered_on_the_device(gpu, hip):
    """accel_update_values_async queues one kernel and returns: an update and the run behind
    it need no host wait, on one stream or on two, and give the bits of a fresh operator on
    the new values; runs queued before the update compute with the old ones."""
    g = gpu.synthetic.cfg2()
    N = 64
    X = gpu.synthetic.dense_operand("cfg2", g.n_cols, N)
    v0 = np.ascontiguousarray(g.values, dtype=np.float32)
    v1 = np.random.default_rng(1).uniform(-2, 2, v0.size).astype(np.float32)
    v2 = np.random.default_rng(2).uniform(-2, 2, v0.size).astype(np.float32)

    def fresh(v):
        o = gpu.AccelSpMM(g.indptr, g.indices, v, g.n_cols).preprocess()
        Y = o.matmul(X)
        o.close()
        return Y

    want0, want1, want2 = fresh(v0), fresh(v1), fresh(v2)
    assert so.check(want1, g.indptr, g.indices, v1, X) <= so.TOL
    op = gpu.AccelSpMM(g.indptr, g.indices, v0, g.n_cols).preprocess()
    dX = gpu.DeviceBuffer.from_numpy(X)
    dYa, dYb, dYc = (gpu.DeviceBuffer(g.n_rows * N * 4) for _ in range(3))
    dV1, dV2 = gpu.DeviceBuffer.from_numpy(v1), gpu.DeviceBuffer.from_numpy(v2)
    s1, s2 = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s1)))
    ok(hip.hipStreamCreate(C.byref(s2)))
    op.update_values_async(dV1, stream=s1.value)          # the first update builds the position map
    op.update_values(v0)                                  # back to the old values (host array, waits)
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    ok(hip.hipDeviceSynchronize())
    ok(hip.hipMemGetInfo(C.byref(free0), C.byref(total)))
    for rep in range(3):
        for d in (dYa, dYb, dYc):
            d.fill_u32(0x7FC00000)
        op.synchronize()
        for _ in range(50):                               # old values, in flight on s1
            op.run(dX, dYa, N, stream=s1.value)
        op.update_values_async(dV1, stream=s2.value)      # waits for them on the device
        op.run(dX, dYb, N, stream=s2.value)               # same stream as the update
        op.update_values_async(dV2, stream=s2.value)
        op.run(dX, dYc, N, stream=s1.value)               # another stream than the update
        ok(hip.hipStreamSynchronize(s1))
        ok(hip.hipStreamSynchronize(s2))
        assert np.array_equal(dYa.to_numpy(np.float32, (g.n_rows, N)), want0), f"round {rep}: runs before the update"
        assert np.array_equal(dYb.to_numpy(np.float32, (g.n_rows, N)), want1), f"round {rep}: update + run, one stream"
        assert np.array_equal(dYc.to_numpy(np.float32, (g.n_rows, N)), want2), f"round {rep}: update + run, two streams"
        op.update_values(v0)
    ok(hip.hipDeviceSynchronize())
    ok(hip.hipMemGetInfo(C.byref(free1), C.byref(total)))
    # later updates allocate nothing: the map is 9.6 MB; the runtime's own pools (events, staging for
    # the host array above) may grow by a 2 MiB chunk
    assert free0.value - free1.value < (4 << 20)
    ok(hip.hipStreamDestroy(s1))
    ok(hip.hipStreamDestroy(s2))
    for b in (dX, dYa, dYb, dYc, dV1, dV2):
        b.close()
    op.close()


def test_captured_update_and_run_follow_the_values(gpu, hip):
    """A graph that holds a value update and the run behind it: every replay reads the value
    array as it is then, so rewriting the array in place between replays is all a caller does
    (upstream's kernel reads val on every launch, spmm_accel.cu:75)."""
    g, X, op = make_case(gpu, 36, 48)
    N = 48
    assert op.info.n_split_rows > 0
    dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * N * 4)
    dV = gpu.DeviceBuffer.from_numpy(np.ascontiguousarray(g.values, dtype=np.float32))
    s = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s)))
    # a first update inside a capture is refused: it would have to allocate the position map
    fresh = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
    graph = C.c_void_p()
    ok(hip.hipStreamBeginCapture(s, 0))
    with pytest.raises(gpu.AccelError) as e:
        fresh.update_values_async(dV, stream=s.value)
    assert e.value.status == gpu._lib.ERR_STATE and "before the capture" in e.value.message
    hip.hipStreamEndCapture(s, C.byref(graph))
    if graph.value:
        hip.hipGraphDestroy(graph)
    fresh.close()
    op.update_values_async(dV)                            # outside: builds the map
    op.run(dX, dY, N)                                     # and the partial-sum buffer
    op.synchronize()
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(s, 0))
    op.update_values_async(dV, stream=s.value)
    op.run(dX, dY, N, stream=s.value)
    ok(hip.hipStreamEndCapture(s, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0))
    for seed in (1, 2, 3, 4):
        v = np.random.default_rng(seed).uniform(-1, 1, g.values.size).astype(np.float32)
        gpu._lib.check(gpu.lib().accel_memcpy_h2d(dV.address, v.ctypes.data, v.nbytes))   # in place
        dY.fill_u32(0x7FC00000)
        op.synchronize()
        ok(hip.hipGraphLaunch(gexec, s))
        ok(hip.hipStreamSynchronize(s))
        Y = dY.to_numpy(np.float32, (g.n_rows, N))
        assert so.check(Y, g.indptr, g.indices, v, X) <= so.TOL, f"replay {seed}"
        ref = gpu.AccelSpMM(g.indptr, g.indices, v, g.n_cols).preprocess()
        assert np.array_equal(Y.view(np.uint32), ref.matmul(X).view(np.uint32)), f"replay {seed}: bits"
        ref.close()
    ok(hip.hipGraphExecDestroy(gexec))
    ok(hip.hipGraphDestroy(graph))
    ok(hip.hipStreamDestroy(s))
    for b in (dX, dY, dV):
        b.close()
    op.close()


def test_reserve_before_capture(gpu, hip):
    """A captured run must not grow the partial-sum buffer: without accel_reserve a first
    run with a larger N inside a capture is refused; with it, the graph replays and later
    eager runs with smaller N leave the graph valid."""
    g, X, op = make_case(gpu, 34, 96)
    N = 96
    dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * N * 4)
    X16 = np.ascontiguousarray(X[:, :16])
    dX16, dY16 = gpu.DeviceBuffer.from_numpy(X16), gpu.DeviceBuffer(g.n_rows * 16 * 4)
    op.run(dX16, dY16, 16)                                # the buffer now fits N = 16 only
    op.synchronize()
    s = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(s)))
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(s, 0))
    with pytest.raises(gpu.AccelError) as e:
        op.run(dX, dY, N, stream=s.value)
    assert e.value.status == gpu._lib.ERR_STATE and "accel_reserve" in e.value.message
    hip.hipStreamEndCapture(s, C.byref(graph))            # nothing was recorded; end the capture
    if graph.value:
        hip.hipGraphDestroy(graph)
    op.reserve(N)
    graph = C.c_void_p()
    ok(hip.hipStreamBeginCapture(s, 0))
    op.run(dX, dY, N, stream=s.value)
    ok(hip.hipStreamEndCapture(s, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0))
    for rep in range(3):
        dY.fill_u32(0x7FC00000)
        op.run(dX16, dY16, 16)                            # eager runs with a smaller N in between
        op.synchronize()
        ok(hip.hipGraphLaunch(gexec, s))
        ok(hip.hipStreamSynchronize(s))
        Y = dY.to_numpy(np.float32, (g.n_rows, N))
        assert so.check(Y, g.indptr, g.indices, g.values, X) <= so.TOL, f"replay {rep}"
    ok(hip.hipGraphExecDestroy(gexec))
    ok(hip.hipGraphDestroy(graph))
    ok(hip.hipStreamDestroy(s))
    for b in (dX, dY, dX16, dY16):
        b.close()
    op.close()


def test_operands_the_gpu_cannot_use_are_refused(gpu):
    """A host address or an allocation that is too small comes back as ACCEL_ERR_ARG from the
    C ABI (given as raw addresses, so that the host-side checks of the binding do not see them)."""
    g, X, op = make_case(gpu, 35, 32)
    N = 32
    dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * N * 4)
    host_y = np.zeros((g.n_rows, N), np.float32)
    small = gpu.DeviceBuffer(g.n_rows * N * 4 - 64)
    for args in ((X.ctypes.data, dY.address), (dX.address, host_y.ctypes.data), (dX.address, small.address),
                 (dX.address + 64, dY.address)):
        with pytest.raises(gpu.AccelError) as e:
            op.run(args[0], args[1], N)
        assert e.value.status == gpu._lib.ERR_ARG, e.value
    with pytest.raises(gpu.AccelError):                   # the binding's own check
        op.run(X, dY, N)
    with pytest.raises(gpu.AccelError):
        op.run(dX, small, N)
    op.run(dX, dY, N)                                     # good operands still run
    op.synchronize()
    assert so.check(dY.to_numpy(np.float32, (g.n_rows, N)), g.indptr, g.indices, g.values, X) <= so.TOL
    for b in (dX, dY, small):
        b.close()
    op.close()


def test_a_recycled_address_is_checked_again(gpu):
    """The operand check asks the runtime on every call: after a buffer that passed has been
    freed and a smaller allocation has taken its address, the same call is refused (a check
    remembered from the first call would let the kernel run past the new allocation)."""
    g, X, op = make_case(gpu, 37, 64)
    N = 64
    dX = gpu.DeviceBuffer.from_numpy(X)
    need = g.n_rows * N * 4
    dY = gpu.DeviceBuffer(need)
    op.run(dX, dY, N)                                     # passes, with this address and size
    op.synchronize()
    addr = dY.address
    dY.close()
    small, others = None, []
    for size in (need - 4096, need // 2, need // 4, need // 16):   # allocators hand freed addresses out again
        for _ in range(16):
            b = gpu.DeviceBuffer(size)
            if b.address == addr:
                small = b
                break
            others.append(b)
        if small is not None:
            break
    for b in others:
        b.close()
    if small is None:
        dX.close(); op.close()
        pytest.skip("the allocator did not hand the freed address out again")
    with pytest.raises(gpu.AccelError) as e:
        op.run(dX, addr, N)
    assert e.value.status == gpu._lib.ERR_ARG and "allocation holds" in e.value.message
    small.close()
    dX.close()
    op.close()


def test_torch_tensors_as_operands(gpu):
    """torch tensors (data_ptr, torch's current stream) straight into the C ABI, in a
    process that imports torch first so that one HIP runtime serves both."""
    import importlib.util
    import subprocess
    import sys
    from pathlib import Path
    if importlib.util.find_spec("torch") is None:
        pytest.skip("torch is not installed")
    case = Path(__file__).resolve().parent / "cases" / "torch_interop.py"
    r = subprocess.run([sys.executable, str(case)], capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "RESULT" in r.stdout


def test_no_device_memory_leak(gpu, hip):
    """Create / preprocess / run / destroy in a loop leaves the free device memory
    where it was (every buffer the handle owns is released)."""
    hip.hipMemGetInfo.restype = C.c_int
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    g = helpers.graph_from_degrees(helpers.degree_mix(seed=40, n_long=6), seed=40)
    X = np.random.default_rng(0).uniform(-1, 1, (g.n_cols, 64)).astype(np.float32)

    def cycle():
        op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()
        op.matmul(X)
        op.preprocess(plan_unit=64)                      # re-preprocessing replaces the products
        op.matmul(X)
        op.close()

    cycle()                                              # first use may grow runtime-internal pools
    gpu._lib.check(gpu.lib().accel_stream_sync(None))
    ok(hip.hipMemGetInfo(C.byref(free0), C.byref(total)))
    for _ in range(20):
        cycle()
    gpu._lib.check(gpu.lib().accel_stream_sync(None))
    ok(hip.hipMemGetInfo(C.byref(free1), C.byref(total)))
    assert free0.value - free1.value < (8 << 20), f"free memory fell by {free0.value - free1.value} bytes"


def test_handles_give_their_memory_back(gpu, hip, tmp_path):
    """Create, preprocess (or load a state), run every way, update the values, destroy,
    many times over: the free device memory must come back to where it was."""
    g = gpu.synthetic.cfg2()                               # 2.4 M non-zeros: some 50 MB per handle
    N = 64
    X = gpu.synthetic.dense_operand("cfg2", g.n_cols, N)
    dX, dY = gpu.DeviceBuffer.from_numpy(X), gpu.DeviceBuffer(g.n_rows * N * 4)
    state = tmp_path / "cfg2.accelstate"

    def free_bytes():
        ok(hip.hipDeviceSynchronize())
        free, total = C.c_size_t(), C.c_size_t()
        ok(hip.hipMemGetInfo(C.byref(free), C.byref(total)))
        return free.value

    def cycle(i):
        op = gpu.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)
        if i % 3 == 2:
            op.load_state(state)
        else:
            op.preprocess()
        if i == 0:
            op.save_state(state)
        op.run(dX, dY, N)
        op.reserve(128)
        op.run_static(dX, dY, 16)
        op.run_ex(dX, dY, 32, ld=64, relu=True)
        op.update_values(g.values)
        if i % 4 == 1:
            op.preprocess()                                # a second time on the same handle
        op.synchronize()
        op.close()

    cycle(0)                                               # whatever the first use of the library keeps
    before = free_bytes()
    for i in range(1, 25):
        cycle(i)
    after = free_bytes()
    assert before - after < 8 << 20, f"{(before - after) / 1e6:.1f} MB not returned after 24 handles"
    dX.close(); dY.close()
