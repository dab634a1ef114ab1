#!/usr/bin/env python3
"""Benchmark of the SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4] [--N 64]

A step is one Y = A X over the whole synthetic graph, inputs resident in HBM.
Prints ONE JSON line: GFLOP/s = 2 * nnz * N / t, the HBM-roofline figures of the
gather kernel (algorithmic bytes = nnz*(4+4) + M*N*4 + rows*N*4 per launch,
launch duration from HIP events recorded on the launch stream during the timed
steps), and scipy's CSR @ dense timed on this host's cores on a bounded row
sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0


KERNEL_SOURCES = ("spmm.hip", "preprocess.hip", "internal.h")


def kernel_source_hash():
    """First 16 hex digits of the SHA-256 over the sources that decide what the gather kernel
    does and in which order (kernels, launch plan, shared constants)."""
    import hashlib
    h = hashlib.sha256()
    base = os.path.join(os.path.dirname(os.path.abspath(__file__)), "iccad-accel-gcn_amd", "csrc")
    for name in KERNEL_SOURCES:
        with open(os.path.join(base, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def recorded_traffic(workload, N):
    """HBM bytes per launch from the committed rocprofv3 counter runs (the counters cannot be
    read from inside a timing run).  Every entry records the hash of the kernel sources it was
    taken with: an entry taken with other sources is reported as stale, not as this run's."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "spmm_gather_traffic.json")
    try:
        with open(path) as f:
            entry = json.load(f).get(f"{workload}/N{N}")
    except OSError:
        return None, "no profile file"
    if not entry:
        return None, "this workload was not profiled"
    now = kernel_source_hash()
    if entry.get("source_sha16") != now:
        return None, (f"profiles/spmm_gather_traffic.json holds {entry.get('traffic_bytes')} bytes for this "
                      f"workload, taken with kernel sources {entry.get('source_sha16', 'of unknown hash')}; "
                      f"the sources now hash to {now}")
    return entry, None


def probe_rates(N):
    """What the pure-gather probe kernel sustains on this GPU for rows of N floats, in GB/s of
    gathered rows: every gather an L2 hit / every gather an L2 miss into an operand of several
    hundred MB (committed with the counter runs; the probe is `bench.py --gather-probe`)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "spmm_gather_traffic.json")
    try:
        with open(path) as f:
            table = json.load(f).get("_probe_rates_GBps")
    except OSError:
        return None
    if not table:
        return None
    key = "N16" if N <= 16 else "N32" if N <= 32 else "N64"
    return table.get(key)


def ceilings(alg_bytes, delivered_bytes, l2_hit_rate, rates):
    """Bounds on the roofline fraction of a launch that gathers one row of X per non-zero:
    delivered_bytes (nnz * N * 4) must pass through the vector-memory path whatever the
    schedule.  all_hits: every gather served by an L2 at the probe's hit rate; at_hit_rate: the
    launch's own measured L2 hit rate, hits and misses at the probe's two rates."""
    if not rates:
        return None, None
    t_hits = delivered_bytes / (rates["l2_hit"] * 1e9)
    all_hits = alg_bytes / t_hits / 1e9 / HBM_PEAK_GBS
    if l2_hit_rate is None:
        return all_hits, None
    t = delivered_bytes * (l2_hit_rate / (rates["l2_hit"] * 1e9) + (1.0 - l2_hit_rate) / (rates["l2_miss"] * 1e9))
    return all_hits, alg_bytes / t / 1e9 / HBM_PEAK_GBS


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_baseline(g, X, N, budget_s=10.0):
    """scipy csr @ X (fp32, one thread) on the first rows of the CSR that fit the
    time budget; the checker only, never the measured path."""
    from oracle import spmm_oracle as so

    rows = g.n_rows

    def run(n_rows):
        ip = g.indptr[: n_rows + 1]
        nz = int(ip[-1])
        A = so.csr(ip, g.indices[:nz], g.values[:nz], g.n_cols)
        t0 = time.perf_counter()
        Y = A @ X
        return time.perf_counter() - t0, nz, Y

    probe_rows = max(1, min(rows, rows // 50))
    t_probe, nz_probe, _ = run(probe_rows)
    rate = nz_probe / max(t_probe, 1e-9)                       # non-zeros per second
    want_nz = min(g.nnz, int(rate * budget_s))
    n_rows = int(np.searchsorted(g.indptr, want_nz, side="right")) - 1
    n_rows = max(probe_rows, min(rows, n_rows))
    t, nz, Y = run(n_rows)
    return {"value": 2.0 * nz * N / t / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "host_cores": os.cpu_count(), "seconds": round(t, 3),
            "sample": f"scipy.sparse csr_matrix @ dense, fp32, first {n_rows} of {rows} rows "
                      f"({nz} of {g.nnz} non-zeros), N={N}, 1 thread"}, n_rows, Y


def load_workload(syn, spec, cache_dir):
    """The workload's CSR, generated once per machine: the arrays are kept under
    ``cache_dir`` so that repeated runs (profiler passes) skip the generator."""
    import hashlib
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "iccad-accel-gcn_amd", "synthetic.py"), "rb") as f:
        tag = hashlib.sha256(f.read() + spec.encode()).hexdigest()[:16]
    path = os.path.join(cache_dir, f"{spec.replace(':', '-')}-{tag}.npz") if cache_dir else None
    if path and os.path.exists(path):
        try:
            z = np.load(path)
            return syn.Graph(spec, z["indptr"], z["indices"], z["values"], int(z["n_rows"]), int(z["n_cols"])), True
        except Exception:
            pass                                           # unreadable cache entry: generate again
    g = syn.workload(spec)
    if path:
        try:
            os.makedirs(cache_dir, exist_ok=True)
            tmp = path + f".{os.getpid()}.tmp.npz"
            np.savez(tmp, indptr=g.indptr, indices=g.indices, values=g.values, n_rows=g.n_rows, n_cols=g.n_cols)
            os.replace(tmp, path)
        except OSError:
            pass
    return g, False


def rocsparse_baseline(pkg, op, g, dX, N, iters=10):
    """Vendor-library CSR SpMM on the same resident operands (comparison only, as
    upstream compares with cuSPARSE; never part of `value`)."""
    import ctypes as C
    path = os.path.join(os.path.dirname(str(pkg._lib.LIB_PATH)), "libaccelgcn_baselines.so")
    L = C.CDLL(path)
    L.baseline_last_error.restype = C.c_char_p
    bufs = [pkg.DeviceBuffer.from_numpy(a) for a in (g.indptr, g.indices, g.values)]
    dY = pkg.DeviceBuffer(g.n_rows * N * 4)
    out = {}
    for name, alg in (("default", 0), ("row_split", 4), ("nnz_split", 5), ("merge_path", 9)):
        ms = (C.c_float * iters)()
        pre = C.c_float(0)
        rc = L.baseline_rocsparse_spmm(C.c_void_p(bufs[0].address), C.c_void_p(bufs[1].address),
                                       C.c_void_p(bufs[2].address), C.c_int64(g.n_rows), C.c_int64(g.n_cols),
                                       C.c_int64(g.nnz), C.c_void_p(dX.address), C.c_void_p(dY.address),
                                       C.c_int32(N), alg, 3, iters, ms, C.byref(pre))
        if rc != 0:
            out[name] = {"error": L.baseline_last_error().decode()}
            continue
        out[name] = {"ms": round(float(np.median(list(ms))), 5), "preprocess_ms": round(pre.value, 3)}
    Yr = dY.to_numpy(np.float32, (g.n_rows, N))
    for b in bufs + [dY]:
        b.close()
    return out, Yr


def neighbor_partition_baseline(pkg, g, dX, N, iters=10):
    """Neighbour-partition SpMM (the scheme of upstream's second comparison kernel,
    spmm_gnna.cu) on the same resident operands; comparison only."""
    import ctypes as C
    path = os.path.join(os.path.dirname(str(pkg._lib.LIB_PATH)), "libaccelgcn_baselines.so")
    L = C.CDLL(path)
    L.baseline_neighbor_partition_last_error.restype = C.c_char_p
    bufs = [pkg.DeviceBuffer.from_numpy(a) for a in (g.indices, g.values)]
    dY = pkg.DeviceBuffer(g.n_rows * N * 4)
    ms = (C.c_float * iters)()
    pre, n_parts = C.c_float(0), C.c_int64(0)
    indptr = np.ascontiguousarray(g.indptr, dtype=np.int32)
    rc = L.baseline_neighbor_partition_spmm(
        indptr.ctypes.data_as(C.c_void_p), C.c_void_p(bufs[0].address), C.c_void_p(bufs[1].address),
        C.c_int64(g.n_rows), C.c_int64(g.nnz), C.c_void_p(dX.address), C.c_void_p(dY.address),
        C.c_int32(N), 0, 3, iters, ms, C.byref(pre), C.byref(n_parts))
    if rc != 0:
        out, Yn = {"error": L.baseline_neighbor_partition_last_error().decode()}, None
    else:
        out = {"ms": round(float(np.median(list(ms))), 5), "preprocess_ms": round(pre.value, 3),
               "parts": n_parts.value, "part_size": max(1, g.nnz // max(g.n_rows, 1))}
        Yn = dY.to_numpy(np.float32, (g.n_rows, N))
    for b in bufs + [dY]:
        b.close()
    return out, Yn


def gcn_layer_timing(pkg, op, g, N, K, steps, compare_rocblas=False):
    """Z = F W (accel_dense_xw) alone, then the layer Y = relu(A (F W) + b): both on the host
    clock over `steps` launches queued back to back; a sample of rows of Z is checked against
    an fp64 product.  The dense product alone is warmed up for 80 launches: a burst of
    matrix-core work makes the GPU lower its clocks for the first 20 ms or so (launches of
    0.44 ms grow to 0.63 ms and come back down over some forty launches); inside the layer,
    next to the sparse product, the same kernel takes 0.41 ms from the start."""
    rng = np.random.default_rng(5)
    rows = g.n_cols
    F = rng.uniform(-1, 1, (rows, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    dF, dW, dZ = pkg.DeviceBuffer.from_numpy(F), pkg.DeviceBuffer.from_numpy(W), pkg.DeviceBuffer(rows * N * 4)
    dB = pkg.DeviceBuffer.from_numpy(rng.standard_normal(N).astype(np.float32))
    dY = pkg.DeviceBuffer(g.n_rows * N * 4)            # the layer's own output: the timed run's Y stays as it is

    def timed(fn, warm=10):
        for _ in range(warm):
            fn()
        op.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        op.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    dense_ms = timed(lambda: pkg.dense_xw(dF, dW, dZ, rows, K, N), warm=80)
    Z = dZ.to_numpy(np.float32, (rows, N))
    idx = np.unique(np.concatenate([np.arange(min(rows, 2048)), rng.integers(0, rows, 4096), np.arange(max(0, rows - 2048), rows)]))
    R = F[idx].astype(np.float64) @ W.astype(np.float64)
    S = np.abs(F[idx].astype(np.float64)) @ np.abs(W.astype(np.float64))
    err = float(np.max(np.abs(Z[idx] - R) / np.maximum(S, np.finfo(np.float32).tiny)))

    def one_layer():
        pkg.dense_xw(dF, dW, dZ, rows, K, N)
        op.run_epilogue(dZ, dY, N, bias=dB, relu=True)
    layer_ms = timed(one_layer)
    sparse_ms = timed(lambda: op.run_epilogue(dZ, dY, N, bias=dB, relu=True))
    dense_bytes = rows * K * 4 + rows * N * 4 + K * N * 4
    out = {"K": K, "dense_ms": round(dense_ms, 5), "layer_ms": round(layer_ms, 5),
           "sparse_with_bias_relu_ms": round(sparse_ms, 5),
           "dense_TFLOPs": round(2.0 * rows * K * N / (dense_ms * 1e-3) / 1e12, 2),
           "dense_frac_of_fp32_matrix_peak": round(2.0 * rows * K * N / (dense_ms * 1e-3) / 1e12 / 157.3, 4),
           "dense_algorithmic_bytes": dense_bytes,
           "dense_GBps": round(dense_bytes / (dense_ms * 1e-3) / 1e9, 1),
           "dense_frac_of_hbm_peak": round(dense_bytes / (dense_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "dense_scaled_error": err, "dense_rows_checked": int(idx.size), "dense_ok": bool(err <= 1e-5)}
    if compare_rocblas:
        # both sides the same way: the host clock over `steps` launches queued back to back, after 80 warm-ups
        import ctypes as C
        L = C.CDLL(os.path.join(os.path.dirname(str(pkg._lib.LIB_PATH)), "libaccelgcn_baselines.so"))
        L.baseline_rocblas_last_error.restype = C.c_char_p
        ms, queued = (C.c_float * steps)(), C.c_float(0)
        rc = L.baseline_rocblas_sgemm(C.c_void_p(dF.address), C.c_void_p(dW.address), C.c_void_p(dZ.address),
                                      C.c_int64(rows), C.c_int32(K), C.c_int32(N), 80, steps, ms, C.byref(queued))
        if rc != 0:
            out["rocblas"] = {"error": L.baseline_rocblas_last_error().decode()}
        else:
            Zr = dZ.to_numpy(np.float32, (rows, N))
            theirs = float(queued.value)
            out["rocblas"] = {"sgemm_ms": round(theirs, 5), "sgemm_ms_by_events_median": round(float(np.median(list(ms))), 5),
                              "ours_ms": out["dense_ms"],
                              "speedup": round(theirs / out["dense_ms"], 3),
                              "max_abs_diff": float(np.max(np.abs(Zr[idx] - Z[idx])))}
    for b in (dF, dW, dZ, dB, dY):
        b.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=40,
                    help="untimed steps before the timed ones; the GPU reaches its steady clocks after some "
                         "60 ms of load (about 19 steps of the default workload run 4 %% slower than all later ones)")
    ap.add_argument("--workload", default="cfg4",
                    help="cfg1..cfg5, or fixture:<name> for the degree sequence of one of the "
                         "reference's graphs (e.g. fixture:OVCAR-8H, fixture:ppa) with uniform random "
                         "columns, or local:<name>:<sigma> for the same with columns within about "
                         "sigma of the row id, or uniform:<rows>:<degree>:<cols> for rows of one "
                         "degree with uniform random columns")
    ap.add_argument("--N", type=int, default=0, help="columns of X (default: the workload's first)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the scipy baseline and the check")
    ap.add_argument("--compare-rocsparse", action="store_true",
                    help="also time rocSPARSE's CSR SpMM on the same operands (comparison only)")
    ap.add_argument("--compare-neighbor-partition", action="store_true",
                    help="also time a neighbour-partition kernel with atomics (the scheme of "
                         "upstream's spmm_gnna.cu) on the same operands (comparison only)")
    ap.add_argument("--gather-probe", type=int, default=0, metavar="ROWS",
                    help="only run the pure-gather probe: random rows of --N floats (16, 64 or 256) "
                         "from an array of ROWS rows, with --probe-stores none|plain|streaming and one "
                         "stored row per --probe-row-len gathers (what the GPU sustains for the SpMM's "
                         "access pattern when a kernel does nothing else)")
    ap.add_argument("--probe-stores", default="none", choices=["none", "plain", "streaming"])
    ap.add_argument("--probe-row-len", type=int, default=32)
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="only run the plain copy kernel over this many MiB, --steps times "
                         "(known-size reference for the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--panel", type=int, default=0, help="column-panel width (accel_set_plan_panel; 0 = the library's choice)")
    ap.add_argument("--plan-split", type=int, default=0, help="rows above this many non-zeros are split (accel_set_plan_split; 0 = the library's choice)")
    ap.add_argument("--plan-groups", type=int, default=0, help="column groups of split rows (accel_set_plan_groups; 0 = per row)")
    ap.add_argument("--plan-reduce", type=int, default=0, help="where split rows are added up (accel_set_plan_reduce; 1 = in the gather kernel, 2 = second kernel, 0 = the library's choice)")
    ap.add_argument("--ld", type=int, default=0,
                    help="also time accel_run_strided with rows of X and Y this many floats apart (>= N), "
                         "on the host clock; reported as config.strided")
    ap.add_argument("--dense-k", type=int, default=0, metavar="K",
                    help="also time the dense product of a GCN layer, Z = F W with F cols x K and W K x N "
                         "(accel_dense_xw), alone and in front of the sparse product with bias and ReLU in its "
                         "store; reported as config.gcn_layer")
    ap.add_argument("--compare-rocblas", action="store_true",
                    help="with --dense-k: also time rocBLAS SGEMM on the same dense operands (comparison only)")
    ap.add_argument("--cache-dir", default="/tmp/accelgcn_bench_cache",
                    help="where generated workloads are kept between runs ('' = do not keep them)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures one GPU only (the path has no multi-GPU part); "
                 "run it with --gpus 1 in a single process")

    import __graft_entry__ as entry
    pkg = entry.load_package()
    if pkg.device_count() < 1:
        sys.exit("bench.py: no GPU: " + pkg._lib.last_error())
    if a.gather_probe:
        import ctypes as C
        L = C.CDLL(os.path.join(os.path.dirname(str(pkg._lib.LIB_PATH)), "libaccelgcn_baselines.so"))
        L.baseline_gather_probe_last_error.restype = C.c_char_p
        N = a.N or 64
        ms, gathered, stored = C.c_float(0), C.c_double(0), C.c_double(0)
        stores = {"none": 0, "plain": 1, "streaming": 2}[a.probe_stores]
        rc = L.baseline_gather_probe(C.c_int64(a.gather_probe), C.c_int32(N), C.c_int32(256),
                                     C.c_int32(a.probe_row_len), C.c_int32(stores), C.c_int32(5),
                                     C.byref(ms), C.byref(gathered), C.byref(stored))
        if rc != 0:
            sys.exit("bench.py: gather probe: " + L.baseline_gather_probe_last_error().decode())
        print(json.dumps({"gather_probe": {"rows_of_X": a.gather_probe, "N": N, "X_MB": round(a.gather_probe * N * 4 / 1e6, 2),
                                            "stores": a.probe_stores, "gathers_per_stored_row": a.probe_row_len,
                                            "ms": round(ms.value, 4),
                                            "gathered_TB_per_s": round(gathered.value / ms.value / 1e9, 2),
                                            "stored_TB_per_s": round(stored.value / ms.value / 1e9, 3)}}), flush=True)
        return
    if a.copy_calibration:
        import ctypes as C
        words = a.copy_calibration * (1 << 20) // 4
        src, dst = pkg.DeviceBuffer(words * 4), pkg.DeviceBuffer(words * 4)
        src.fill_u32(1)
        for _ in range(a.steps):
            pkg._lib.check(pkg.lib().accel_dev_copy_u32(C.c_void_p(dst.address), C.c_void_p(src.address), words, None))
        pkg._lib.check(pkg.lib().accel_stream_sync(None))
        print(json.dumps({"copy_calibration_MiB": a.copy_calibration, "launches": a.steps,
                          "bytes_read_per_launch": words * 4, "bytes_written_per_launch": words * 4}))
        return
    syn = pkg.synthetic
    N = a.N or syn.WORKLOAD_N.get(a.workload, (64,))[0]

    t0 = time.time()
    try:
        g, cached = load_workload(syn, a.workload, a.cache_dir)
    except (ValueError, KeyError) as e:
        sys.exit(f"bench.py: {e}")
    X = syn.dense_operand(a.workload, g.n_cols, N)
    log(f"[bench] {a.workload}: rows={g.n_rows} nnz={g.nnz} N={N} "
        f"{'loaded from the cache' if cached else 'generated'} in {time.time() - t0:.1f}s")

    t0 = time.time()
    op = pkg.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)
    t_upload = time.time() - t0
    plan = {k: v for k, v in (("plan_split", a.plan_split), ("plan_groups", a.plan_groups),
                              ("plan_reduce", a.plan_reduce)) if v}
    op.preprocess(**plan)
    first_preprocess_ms = op.info.preprocess_ms      # includes loading the kernels into the GPU
    op.preprocess(**plan)                            # the same work again: what a second graph would cost
    if a.panel:
        op.set_panel(a.panel)
    info = op.info
    log(f"[bench] upload {t_upload * 1e3:.0f} ms, preprocess {info.preprocess_ms:.1f} ms: "
        f"blocks={info.n_blocks} long_rows={info.n_long_rows} long_blocks={info.n_long_blocks} "
        f"zero_rows={info.n_zero_rows} max_degree={info.max_degree}")
    # the same products from a saved state instead (accel_save_state / accel_load_state)
    import tempfile
    from_cache_ms = None
    with tempfile.TemporaryDirectory() as td:
        state = os.path.join(td, "bench.accelstate")
        op.save_state(state)
        state_mb = os.path.getsize(state) / 1e6
        op2 = pkg.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols)
        op2.load_state(state)
        op2.load_state(state)                        # second load: file in the page cache, kernels loaded
        from_cache_ms = op2.info.preprocess_ms
        op2.close()
    log(f"[bench] preprocess from a saved state ({state_mb:.1f} MB): {from_cache_ms:.1f} ms")
    # new values on the same structure, from an array already on the device: one kernel queued
    # on the stream (accel_update_values_async; the first call builds the position map)
    dV = pkg.DeviceBuffer.from_numpy(np.ascontiguousarray(g.values, dtype=np.float32))
    op.update_values_async(dV)
    op.synchronize()
    t0 = time.perf_counter()
    for _ in range(4):
        op.update_values_async(dV)
    op.synchronize()
    update_values_ms = (time.perf_counter() - t0) * 1e3 / 4
    dV.close()
    log(f"[bench] values replaced on the same structure: {update_values_ms:.2f} ms")
    dX = pkg.DeviceBuffer.from_numpy(X)
    dY = pkg.DeviceBuffer(g.n_rows * N * 4)
    dY.fill_u32(0x7FC00000)

    # warm-up, then the timed region: K steps queued back to back, bracketed by
    # synchronisations.  Each step carries two events recorded around it (everything a call
    # launches) and two bound to the gather kernel's own start and end (its duration).
    op.time(dX, dY, N, warmup=a.warmup, iters=0)
    op.synchronize()
    t0 = time.perf_counter()
    tot_ms, main_ms = op.time(dX, dY, N, warmup=0, iters=a.steps)
    op.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / a.steps * 1e3
    # The events themselves cost a step a few microseconds, which only a launch-bound
    # workload notices (a fifth of a 30 us step): the same K steps once more without any,
    # on the host clock, for what a caller's loop of runs gets.
    op.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        op.run(dX, dY, N)
    op.synchronize()
    ms_per_step_no_events = (time.perf_counter() - t0) / a.steps * 1e3

    # secondary figure: upstream's own protocol (spmm_base.h:44-60): 4 warm-up launches,
    # then 4 launches each timed on the host clock around launch + synchronisation
    for _ in range(4):
        op.run(dX, dY, N)
    op.synchronize()
    ref_protocol = 0.0
    for _ in range(4):
        t1 = time.perf_counter()
        op.run(dX, dY, N)
        op.synchronize()
        ref_protocol += time.perf_counter() - t1
    ref_protocol_ms = ref_protocol / 4 * 1e3

    strided = None
    if a.ld:
        if a.ld < N:
            sys.exit("bench.py: --ld must be at least N")
        sX, sY = pkg.DeviceBuffer(g.n_cols * a.ld * 4), pkg.DeviceBuffer(g.n_rows * a.ld * 4)
        sX.fill_u32(0x3F000000)
        for _ in range(3):
            op.run_strided(sX, sY, N, a.ld)
        op.synchronize()
        t1 = time.perf_counter()
        for _ in range(a.steps):
            op.run_strided(sX, sY, N, a.ld)
        op.synchronize()
        strided = {"ld": a.ld, "ms_per_step": round((time.perf_counter() - t1) / a.steps * 1e3, 5)}
        s_tot, s_main = op.time_ex(sX, sY, N, ld=a.ld, warmup=0, iters=a.steps)
        strided["kernel_ms_avg"] = round(float(np.mean(s_main)), 5)
        strided["all_kernels_ms_avg"] = round(float(np.mean(s_tot)), 5)
        sX.close()
        sY.close()

    layer = gcn_layer_timing(pkg, op, g, N, a.dense_k, a.steps, a.compare_rocblas) if a.dense_k else None

    flops = 2.0 * g.nnz * N
    alg_bytes = g.nnz * 8 + g.n_cols * N * 4 + g.n_rows * N * 4
    main_avg_ms = float(np.mean(main_ms))
    achieved = alg_bytes / (main_avg_ms * 1e-3) / 1e9
    achieved_all = alg_bytes / (float(np.mean(tot_ms)) * 1e-3) / 1e9
    profiled, traffic_note = recorded_traffic(a.workload, N)
    if a.panel or a.plan_split or a.plan_groups or a.plan_reduce:
        profiled, traffic_note = None, "run with plan options: not the configuration that was profiled"
    traffic = profiled.get("traffic_bytes") if profiled else None
    l2_hit_rate = profiled.get("l2_hit_rate") if profiled else None
    delivered = g.nnz * N * 4
    rates = probe_rates(N)
    bound_all_hits, bound_at_hit_rate = ceilings(alg_bytes, delivered, l2_hit_rate, rates)
    result = {
        "metric": "SpMM GFLOP/s (2*nnz*N), fp32",
        "value": round(flops / (ms_per_step * 1e-3) / 1e9, 2),
        "unit": "GFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{a.workload}: {g.n_rows} rows, {g.nnz} non-zeros, N={N}",
                   "rows": g.n_rows, "nnz": g.nnz, "N": N, "blocks": int(info.n_blocks),
                   "preprocess_ms": round(info.preprocess_ms, 2),
                   "preprocess_first_call_ms": round(first_preprocess_ms, 2),
                   "preprocess_from_cache_ms": round(from_cache_ms, 2),
                   "update_values_ms": round(update_values_ms, 2),
                   "reference_protocol_ms": round(ref_protocol_ms, 5),
                   "ms_per_step_without_events": round(ms_per_step_no_events, 5),
                   "plan": {"split_nz": int(info.plan_split_nz), "groups": int(info.plan_groups),
                            "unit_nz": int(info.plan_unit_nz), "panel": a.panel,
                            "queues": int(info.plan_queues), "pieces": int(info.n_plan_pieces),
                            "split_rows_added_up": "in the gather kernel" if info.plan_reduce == 1 else "by a second kernel"}},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic,
                     "kernel": "spmm_gather_kernel", "kernel_ms_avg": round(main_avg_ms, 5),
                     "kernel_ms_min": round(float(np.min(main_ms)), 5),
                     "kernel_timing": "HIP events bound to the gather kernel's own start and end in each of the "
                                      "timed steps (hipExtLaunchKernel): no packet between a step's kernels",
                     "all_kernels_ms_avg": round(float(np.mean(tot_ms)), 5),
                     "all_kernels_ms_median": round(float(np.median(tot_ms)), 5),
                     "frac_all_kernels": round(achieved_all / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes": alg_bytes,
                     # what bounds the fraction for a kernel that gathers a row of X per non-zero
                     "delivered_bytes": delivered,
                     "traffic_over_algorithmic": round(traffic / alg_bytes, 2) if traffic else None,
                     "l2_hit_rate": l2_hit_rate,
                     "probe_rates_GBps": rates,
                     "frac_ceiling_all_l2_hits": round(bound_all_hits, 4) if bound_all_hits else None,
                     "frac_ceiling_at_measured_hit_rate": round(bound_at_hit_rate, 4) if bound_at_hit_rate else None,
                     "target_frac": 0.60,
                     "target_met": bool(achieved / HBM_PEAK_GBS >= 0.60),
                     "kernel_source_sha16": kernel_source_hash()},
    }
    if traffic_note:
        result["roofline"]["traffic_stale"] = traffic_note + " (traffic, l2_hit_rate and the ceiling at the measured hit rate are null for that reason)"
    if strided:
        result["config"]["strided"] = strided
    if layer:
        result["config"]["gcn_layer"] = layer

    if a.compare_rocsparse:
        rs, Yr = rocsparse_baseline(pkg, op, g, dX, N)
        # our side measured the same way: two events around each run, nothing in between
        ours, _ = op.time(dX, dY, N, warmup=3, iters=10, split=False)
        ours_ms = float(np.median(ours))
        Ymine = dY.to_numpy(np.float32, (g.n_rows, N))
        best = min((v["ms"] for v in rs.values() if "ms" in v), default=None)
        result["rocsparse"] = {"algorithms": rs, "best_ms": best, "ours_ms": round(ours_ms, 5),
                               "speedup_vs_best": round(best / ours_ms, 3) if best else None,
                               "max_abs_diff_vs_last_alg": float(np.max(np.abs(Ymine - Yr))) if Yr.size else 0.0}
    if a.compare_neighbor_partition:
        npb, Yn = neighbor_partition_baseline(pkg, g, dX, N)
        ours, _ = op.time(dX, dY, N, warmup=3, iters=10, split=False)
        ours_ms = float(np.median(ours))
        if Yn is not None:
            Ymine = dY.to_numpy(np.float32, (g.n_rows, N))
            npb["ours_ms"] = round(ours_ms, 5)
            npb["speedup"] = round(npb["ms"] / ours_ms, 3)
            npb["max_abs_diff"] = float(np.max(np.abs(Ymine - Yn))) if Yn.size else 0.0
        result["neighbor_partition"] = npb
    if not a.no_cpu:
        base, n_rows, Yc = cpu_baseline(g, X, N)
        result["cpu_baseline"] = base
        # parity of the timed output on the baseline's rows (fp64 reference, scaled error)
        from oracle import c_oracle, spmm_oracle as so
        Y = dY.to_numpy(np.float32, (g.n_rows, N))[:n_rows]
        threads = min(16, os.cpu_count() or 1)          # the checker may use the host's cores; the baseline above does not
        err, slab = 0.0, max(1, (64 << 20) // N)        # 512 MB of fp64 reference at a time
        for r0 in range(0, n_rows, slab):
            r1 = min(n_rows, r0 + slab)
            R, S = c_oracle.spmm_csr_f64(g.indptr[r0:r1 + 1], g.indices, g.values, X, threads=threads)
            err = max(err, so.scaled_error(Y[r0:r1], R, S))
            del R, S
        result["parity"] = {"rows_checked": n_rows, "scaled_error": err, "tolerance": so.TOL,
                            "ok": bool(err <= so.TOL)}
        if err > so.TOL:
            log(f"[bench] PARITY FAILURE: scaled error {err:.3e}")
    print(json.dumps(result), flush=True)
    dX.close()
    dY.close()
    op.close()
    if not a.no_cpu and not result["parity"]["ok"]:
        sys.exit(1)


if __name__ == "__main__":
    main()
