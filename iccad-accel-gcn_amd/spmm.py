"""Host-side mirror of the operator interface for Python callers.

``SpmmAccel`` follows upstream's SPMM_ACCEL (spmm_accel.h:4-20) through
SPMM_BASE (spmm_base.h:6-65): construct on (graph, ptr, idx, val, vin, vout,
num_v, num_e, dim), then ``do_test(timing, dim)`` preprocesses and runs, and
``run(dim)`` is one asynchronous launch.  ``AccelSpMM`` is the numpy-friendly
wrapper used by tests and the benchmark: init / preprocess / run.

Everything computes through the C ABI of libaccelgcn.so on the GPU.
"""
from __future__ import annotations

import ctypes as C
import time
from pathlib import Path

import numpy as np

from . import _lib
from ._lib import AccelError, DeviceBuffer, Info, check, lib, ptr


class AccelSpMM:
    """Y = A @ X for a CSR matrix A (int32 indices, fp32 values) on the GPU.

    init: ``AccelSpMM(indptr, indices, values, n_cols)`` uploads the CSR (host
    numpy arrays) or borrows it (``device=True``: objects with ``data_ptr()`` or
    raw addresses, plus explicit ``n_rows``/``nnz``).
    preprocess: ``preprocess()`` degree-sorts and partitions on the GPU.
    run: ``run(X, Y, N)`` on device buffers, or ``matmul(X)`` numpy -> numpy.
    """

    def __init__(self, indptr, indices, values, n_cols, *, device=False, n_rows=None, nnz=None):
        self._h = C.c_void_p()
        self._keep = None
        if device:
            if n_rows is None or nnz is None:
                raise ValueError("device=True needs n_rows and nnz")
            self.n_rows, self.nnz = int(n_rows), int(nnz)
            self._keep = (indptr, indices, values)
            args = (ptr(indptr), ptr(indices), ptr(values))
            flags = _lib.PTR_DEVICE
        else:
            ip = _lib.as_i32(indptr)
            ix = _lib.as_i32(indices)
            v = _lib.as_f32(values)
            if ip.ndim != 1 or ip.size < 1:
                raise AccelError(_lib.ERR_ARG, "indptr must be a 1-D array with at least one entry")
            if ix.size != v.size:
                raise AccelError(_lib.ERR_ARG, "indices and values differ in length")
            self.n_rows, self.nnz = ip.size - 1, ix.size
            self._keep = (ip, ix, v)
            args = (ptr(ip), ptr(ix), ptr(v))
            flags = _lib.PTR_HOST
        self.n_cols = int(n_cols)
        check(lib().accel_create(*args, self.n_rows, self.n_cols, self.nnz, flags, C.byref(self._h)))
        if not device:
            self._keep = None       # uploaded: host copies are no longer needed
        self._info = None

    # -- preprocess ---------------------------------------------------------
    def preprocess(self, plan_unit: int | None = None, plan_groups: int | None = None,
                   plan_split: int | None = None, plan_team: int | None = None,
                   plan_queues: int | None = None, plan_reduce: int | None = None) -> "AccelSpMM":
        """Degree sort, block4 metadata and launch plan on the GPU.  ``plan_unit``
        (16..384) overrides the automatic choice of non-zeros per unit,
        ``plan_groups`` (8, 16, 32, 64) that of column groups for split rows,
        ``plan_split`` (16..384) the row length above which rows are split,
        ``plan_team`` (1: one wavefront per unit, 2: one workgroup per unit) who
        works on a unit, ``plan_queues`` (8 or 1) the number of interleaved queues of
        the plan (default: from the shape of the device), ``plan_reduce`` (1: the gather
        kernel adds split rows up itself, 2: a second kernel does) where partial sums meet."""
        if plan_reduce is not None:
            check(lib().accel_set_plan_reduce(self._h, int(plan_reduce)))
        if plan_queues is not None:
            check(lib().accel_set_plan_queues(self._h, int(plan_queues)))
        if plan_team is not None:
            check(lib().accel_set_plan_team(self._h, int(plan_team)))
        if plan_unit is not None:
            check(lib().accel_set_plan_unit(self._h, int(plan_unit)))
        if plan_groups is not None:
            check(lib().accel_set_plan_groups(self._h, int(plan_groups)))
        if plan_split is not None:
            check(lib().accel_set_plan_split(self._h, int(plan_split)))
        check(lib().accel_preprocess(self._h))
        info = Info()
        check(lib().accel_get_info(self._h, C.byref(info)))
        self._info = info
        return self

    def save_state(self, path) -> None:
        """Write the degree-sort order and the plan options of this operator to ``path``."""
        self.info
        check(lib().accel_save_state(self._h, str(path).encode()))

    def load_state(self, path) -> "AccelSpMM":
        """Take the place of preprocess(): the preprocessing with the sort replaced by the
        order saved for the same CSR.  Raises AccelError (ERR_META) if the file belongs to
        another CSR or is damaged."""
        check(lib().accel_load_state(self._h, str(path).encode()))
        info = Info()
        check(lib().accel_get_info(self._h, C.byref(info)))
        self._info = info
        return self

    def update_values(self, values) -> "AccelSpMM":
        """New values for the same structure (see accel_update_values): a numpy array of nnz
        floats in the CSR's order, or, for device-resident values, an object with
        ``data_ptr()`` / a raw address (required when the CSR was given with ``device=True``;
        the operator then borrows that array)."""
        self.info
        if isinstance(values, np.ndarray):
            v = _lib.as_f32(values)
            if v.size != self.nnz:
                raise AccelError(_lib.ERR_ARG, f"values has {v.size} entries, the CSR has {self.nnz} non-zeros")
            check(lib().accel_update_values(self._h, ptr(v), _lib.PTR_HOST))
        else:
            check(lib().accel_update_values(self._h, _lib.dev_ptr(values, self.nnz * 4, "values"), _lib.PTR_DEVICE))
            if self._keep is not None and len(self._keep) == 3:
                self._keep = (self._keep[0], self._keep[1], values)
        return self

    def update_values_async(self, values, stream=None) -> "AccelSpMM":
        """New values for the same structure from a device array, queued on ``stream``
        without waiting (see accel_update_values_async)."""
        self.info
        check(lib().accel_update_values_async(self._h, _lib.dev_ptr(values, self.nnz * 4, "values"), ptr(stream)))
        if self._keep is not None and len(self._keep) == 3:
            self._keep = (self._keep[0], self._keep[1], values)
        return self

    def set_panel(self, columns: int) -> None:
        """Column-panel width of the following runs (0: automatic; see accel_set_plan_panel)."""
        check(lib().accel_set_plan_panel(self._h, int(columns)))

    @property
    def info(self) -> Info:
        if self._info is None:
            raise AccelError(_lib.ERR_STATE, "call preprocess() first")
        return self._info

    def block4(self) -> np.ndarray:
        out = np.empty((self.info.n_blocks, 4), dtype=np.int32)
        check(lib().accel_get_block4(self._h, ptr(out, C.c_int32), out.shape[0]))
        return out

    def plan(self) -> np.ndarray:
        """The launch plan: one (x, y, z, w) row per wavefront (see accel_get_plan)."""
        self.info
        n = C.c_int64(0)
        check(lib().accel_get_plan(self._h, None, 0, C.byref(n)))
        out = np.empty((n.value, 4), dtype=np.int32)
        check(lib().accel_get_plan(self._h, ptr(out, C.c_int32), n.value, C.byref(n)))
        return out

    def perm(self) -> np.ndarray:
        self.info
        out = np.empty(self.n_rows, dtype=np.int32)
        check(lib().accel_get_perm(self._h, ptr(out, C.c_int32), out.size))
        return out

    def sorted_csr(self):
        self.info
        ip = np.empty(self.n_rows + 1, dtype=np.int32)
        ix = np.empty(self.nnz, dtype=np.int32)
        v = np.empty(self.nnz, dtype=np.float32)
        check(lib().accel_get_sorted_csr(self._h, ptr(ip, C.c_int32), ptr(ix, C.c_int32), ptr(v, C.c_float)))
        return ip, ix, v

    def check_block4(self, block4) -> None:
        b = _lib.as_i32(block4).reshape(-1)
        if b.size % 4:
            raise AccelError(_lib.ERR_META, "metadata length is not a multiple of 4")
        check(lib().accel_check_block4(self._h, ptr(b, C.c_int32), b.size // 4))

    # -- run ----------------------------------------------------------------
    def _operands(self, X, Y, N, bias=None):
        """Device addresses of the dense operands, after the checks the host can make."""
        N = int(N)
        if N <= 0:
            raise AccelError(_lib.ERR_ARG, f"N must be positive, got {N}")
        return (_lib.dev_ptr(X, self.n_cols * N * 4, "X"), _lib.dev_ptr(Y, self.n_rows * N * 4, "Y"),
                _lib.dev_ptr(bias, N * 4, "bias"))

    def run(self, X, Y, N: int, stream=None) -> None:
        """One asynchronous launch; X, Y are device buffers."""
        x, y, _ = self._operands(X, Y, N)
        check(lib().accel_run(self._h, x, y, int(N), ptr(stream)))

    def run_strided(self, X, Y, N: int, ld: int, stream=None) -> None:
        """``run`` on operands whose rows are ``ld`` >= N floats apart (see accel_run_strided):
        rows of X padded to a multiple of 32 floats touch fewer cache lines per gather."""
        N, ld = int(N), int(ld)
        if N <= 0 or ld < N:
            raise AccelError(_lib.ERR_ARG, f"need 0 < N <= ld, got N={N}, ld={ld}")
        x = _lib.dev_ptr(X, ((self.n_cols - 1) * ld + N) * 4 if self.n_cols else 0, "X")
        y = _lib.dev_ptr(Y, ((self.n_rows - 1) * ld + N) * 4 if self.n_rows else 0, "Y")
        check(lib().accel_run_strided(self._h, x, y, N, ld, ptr(stream)))

    def reserve(self, max_N: int) -> None:
        """Allocate the partial-sum buffer for every N up to ``max_N`` now, so that no later
        run allocates (see accel_reserve)."""
        check(lib().accel_reserve(self._h, int(max_N)))

    def run_static(self, X, Y, N: int, stream=None) -> None:
        """``run`` without any device allocation: the partial sums of split rows go to
        the library's static scratch array (ACCEL_STATIC_SCRATCH_BYTES per GPU) and a
        matrix that needs more at this N is refused (see accel_run_static)."""
        x, y, _ = self._operands(X, Y, N)
        check(lib().accel_run_static(self._h, x, y, int(N), ptr(stream)))

    def run_epilogue(self, X, Y, N: int, bias=None, relu=False, stream=None) -> None:
        """Y = act(A X + bias) in one launch; bias is a device buffer of N floats or None."""
        x, y, b = self._operands(X, Y, N, bias)
        check(lib().accel_run_epilogue(self._h, x, y, int(N), b,
                                       _lib.EPILOGUE_RELU if relu else 0, ptr(stream)))

    def run_ex(self, X, Y, N: int, ld: int = 0, bias=None, relu=False, stream=None) -> None:
        """Every option of a run at once (see accel_run_ex): rows ``ld`` floats apart
        (0: packed), Y = act(A X + bias)."""
        N, ld = int(N), int(ld)
        step = ld or N
        if N <= 0 or step < N:
            raise AccelError(_lib.ERR_ARG, f"need 0 < N <= ld (or ld = 0), got N={N}, ld={ld}")
        a = _lib.RunArgs()
        x = _lib.dev_ptr(X, ((self.n_cols - 1) * step + N) * 4 if self.n_cols else 0, "X")
        y = _lib.dev_ptr(Y, ((self.n_rows - 1) * step + N) * 4 if self.n_rows else 0, "Y")
        b = _lib.dev_ptr(bias, N * 4, "bias")
        s = ptr(stream)
        a.X, a.Y, a.N, a.ld = x.value if x else None, y.value if y else None, N, ld
        a.bias, a.flags, a.stream = b.value if b else None, _lib.EPILOGUE_RELU if relu else 0, s.value if s else None
        check(lib().accel_run_ex(self._h, C.byref(a)))

    def synchronize(self, stream=None) -> None:
        check(lib().accel_stream_sync(ptr(stream)))

    def matmul(self, X: np.ndarray) -> np.ndarray:
        X = _lib.as_f32(X)
        if X.ndim != 2 or X.shape[0] != self.n_cols:
            raise AccelError(_lib.ERR_ARG, f"X must be [{self.n_cols}, N]")
        N = X.shape[1]
        dX = DeviceBuffer.from_numpy(X)
        dY = DeviceBuffer(max(self.n_rows * N * 4, 4))
        dY.fill_u32(0x7FC00000)          # NaN: any row the operator fails to write shows up
        try:
            self.run(dX, dY, N)
            self.synchronize()
            return dY.to_numpy(np.float32, (self.n_rows, N))
        finally:
            dX.close()
            dY.close()

    def time(self, X, Y, N: int, warmup: int = 4, iters: int = 20, stream=None, split: bool = True):
        """HIP-event timings in ms: (total per run, gather kernel only).  The total comes
        from two events recorded around each run, the kernel's time from two events bound to
        its own start and end (nothing is put between the kernels of a run).  With
        ``split=False`` the kernel's events are left out (the second array is then all zeros)."""
        tot = np.zeros(iters, dtype=np.float32)
        main = np.zeros(iters, dtype=np.float32)
        x, y, _ = self._operands(X, Y, N)
        check(lib().accel_time(self._h, x, y, int(N), warmup, iters,
                               ptr(tot, C.c_float), ptr(main, C.c_float) if split else None, ptr(stream)))
        return tot, main

    def time_ex(self, X, Y, N: int, ld: int = 0, bias=None, relu=False, warmup: int = 4, iters: int = 20,
                stream=None, split: bool = True):
        """``time`` on a run with every option (see accel_time_ex): rows ``ld`` floats apart
        (0: packed), Y = act(A X + bias)."""
        N, ld = int(N), int(ld)
        step = ld or N
        if N <= 0 or step < N:
            raise AccelError(_lib.ERR_ARG, f"need 0 < N <= ld (or ld = 0), got N={N}, ld={ld}")
        a = _lib.RunArgs()
        x = _lib.dev_ptr(X, ((self.n_cols - 1) * step + N) * 4 if self.n_cols else 0, "X")
        y = _lib.dev_ptr(Y, ((self.n_rows - 1) * step + N) * 4 if self.n_rows else 0, "Y")
        b = _lib.dev_ptr(bias, N * 4, "bias")
        s = ptr(stream)
        a.X, a.Y, a.N, a.ld = x.value if x else None, y.value if y else None, N, ld
        a.bias, a.flags, a.stream = b.value if b else None, _lib.EPILOGUE_RELU if relu else 0, s.value if s else None
        tot = np.zeros(iters, dtype=np.float32)
        main = np.zeros(iters, dtype=np.float32)
        check(lib().accel_time_ex(self._h, C.byref(a), warmup, iters, ptr(tot, C.c_float),
                                  ptr(main, C.c_float) if split else None))
        return tot, main

    def close(self) -> None:
        if self._h:
            lib().accel_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SpmmAccel:
    """Python mirror of SPMM_ACCEL (spmm_accel.h:4-20, spmm_base.h:9-23).

    All array arguments are device pointers (DeviceBuffer, objects with
    ``data_ptr()``, or addresses), exactly as upstream's main.cu:131 passes
    managed-memory pointers.  ``do_test`` returns mean seconds per launch over
    the 4-warm-up / 4-timed host-clock protocol (spmm_base.h:44-60), 0.0 when
    ``timing`` is false.
    """

    def __init__(self, graph, ptr_, idx, val, vin, vout, num_v, num_e, dim, meta_dir="../block_level_meta/"):
        self._graph = graph
        self.val, self.vin, self.vout = val, vin, vout
        self.num_v, self.num_e, self.dim = int(num_v), int(num_e), int(dim)
        self.meta_dir = Path(meta_dir)
        # True: use <meta_dir>/<graph>.accelstate: load it instead of sorting when it belongs
        # to this CSR, write it after preprocessing otherwise.  Off by default: on this GPU
        # the load is not faster than the preprocessing.
        self.save_state = False
        self.state_loaded = False
        self._op = AccelSpMM(ptr_, idx, val, self.num_v, device=True, n_rows=self.num_v, nnz=self.num_e)
        self._ready = False

    def _preprocess(self):
        if self._ready:
            # upstream's kernel reads val on every launch (spmm_accel.cu:75): a caller may have
            # rewritten the array since the last call; one kernel on the stream of the runs
            self._op.update_values_async(self.val)
            return
        # the saved state of an earlier run takes the place of the preprocessing, as
        # upstream's operator loads its metadata file (spmm_accel.cu:122); a state that
        # does not belong to this CSR is a stale cache entry, not an error
        state = self.meta_dir / f"{self._graph}.accelstate"
        loaded = False
        if self.save_state and state.exists():
            try:
                self._op.load_state(state)
                loaded = True
            except AccelError as e:
                if e.status not in (_lib.ERR_META, _lib.ERR_IO):
                    raise
        if not loaded:
            self._op.preprocess()
            if self.save_state and self.meta_dir.is_dir():
                self._op.save_state(state)
        self.state_loaded = loaded
        meta = self.meta_dir / f"{self._graph}.block4"
        if meta.exists():      # a stale file must not pass silently (spmm_accel.cu:122 trusts it blindly)
            self._op.check_block4(np.fromfile(meta, dtype="<i4"))
        self._ready = True

    def run(self, dim):
        self._op.run(self.vin, self.vout, dim)

    def do_test(self, timing: bool, dim: int) -> float:
        self._preprocess()
        if not timing:
            self.run(dim)
            self._op.synchronize()
            return 0.0
        times = 4
        for _ in range(times):
            self.run(dim)
        self._op.synchronize()
        total = 0.0
        for _ in range(times):
            t0 = time.perf_counter()
            self.run(dim)
            self._op.synchronize()
            total += time.perf_counter() - t0
        return total / times

    @property
    def op(self) -> AccelSpMM:
        return self._op
