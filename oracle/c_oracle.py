"""ctypes view of oracle.c (TEST INFRASTRUCTURE ONLY).  ``build()`` compiles it
with gcc; ``lib()`` loads what is built and builds only when nothing is."""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
SO = HERE / "_build" / "liboracle.so"
_lib = None


def build() -> Path:
    subprocess.run(["make", "-B", "-C", str(HERE)], check=True, capture_output=True)
    return SO


def lib():
    global _lib
    if _lib is None:
        if not SO.exists():
            build()
        L = C.CDLL(str(SO))
        i32p, f32p, f64p = (C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_double))
        L.oracle_partition_walk.restype = C.c_int64
        L.oracle_partition_walk.argtypes = [i32p, C.c_int64, i32p, C.c_int64]
        L.oracle_degree_sort.restype = C.c_int
        L.oracle_degree_sort.argtypes = [i32p, C.c_int64, i32p]
        L.oracle_spmm_csr_f32.restype = None
        L.oracle_spmm_csr_f32.argtypes = [i32p, i32p, f32p, C.c_int64, f32p, f32p, C.c_int64]
        L.oracle_spmm_csr_f64.restype = None
        L.oracle_spmm_csr_f64.argtypes = [i32p, i32p, f32p, C.c_int64, f32p, f64p, f64p, C.c_int64]
        L.oracle_spmm_block4.restype = None
        L.oracle_spmm_block4.argtypes = [i32p, C.c_int64, i32p, f32p, f32p, f32p, C.c_int64]
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def partition_walk(indptr):
    ip = _i32(indptr)
    n = ip.size - 1
    nb = lib().oracle_partition_walk(_p(ip, C.c_int32), n, None, 0)
    out = np.zeros((nb, 4), dtype=np.int32)
    lib().oracle_partition_walk(_p(ip, C.c_int32), n, _p(out, C.c_int32), nb)
    return out


def degree_sort(indptr):
    ip = _i32(indptr)
    perm = np.zeros(ip.size - 1, dtype=np.int32)
    rc = lib().oracle_degree_sort(_p(ip, C.c_int32), ip.size - 1, _p(perm, C.c_int32))
    if rc:
        raise ValueError("indptr is not monotone")
    return perm


def spmm_csr_f32(indptr, indices, values, X):
    ip, ix, v, X = _i32(indptr), _i32(indices), _f32(values), _f32(X)
    Y = np.empty((ip.size - 1, X.shape[1]), dtype=np.float32)
    lib().oracle_spmm_csr_f32(_p(ip, C.c_int32), _p(ix, C.c_int32), _p(v, C.c_float), ip.size - 1,
                              _p(X, C.c_float), _p(Y, C.c_float), X.shape[1])
    return Y


def spmm_csr_f64(indptr, indices, values, X, threads: int = 1):
    """R = A X and S = |A| |X| in fp64.  ``threads`` > 1 runs the same C routine on
    consecutive row ranges from that many host threads (ctypes releases the GIL)."""
    ip, ix, v, X = _i32(indptr), _i32(indices), _f32(values), _f32(X)
    n, N = ip.size - 1, X.shape[1]
    R = np.empty((n, N), dtype=np.float64)
    S = np.empty_like(R)
    fn = lib().oracle_spmm_csr_f64

    def rows(r0, r1):          # indptr entries stay absolute offsets into idx / val
        fn(_p(ip[r0:], C.c_int32), _p(ix, C.c_int32), _p(v, C.c_float), r1 - r0, _p(X, C.c_float),
           _p(R[r0:], C.c_double), _p(S[r0:], C.c_double), N)

    if threads <= 1 or n < 2 * threads:
        rows(0, n)
        return R, S
    import threading
    # ranges of about equal non-zeros
    cuts = np.searchsorted(ip, np.linspace(int(ip[0]), int(ip[-1]), threads + 1)[1:-1]).tolist()
    bounds = [0] + [min(max(int(c), 0), n) for c in cuts] + [n]
    ts = [threading.Thread(target=rows, args=(bounds[i], bounds[i + 1])) for i in range(threads)
          if bounds[i + 1] > bounds[i]]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    return R, S


def spmm_block4(block4, indices, values, X, n_rows):
    b4, ix, v, X = _i32(block4), _i32(indices), _f32(values), _f32(X)
    Y = np.zeros((n_rows, X.shape[1]), dtype=np.float32)
    lib().oracle_spmm_block4(_p(b4, C.c_int32), b4.size // 4, _p(ix, C.c_int32), _p(v, C.c_float),
                             _p(X, C.c_float), _p(Y, C.c_float), X.shape[1])
    return Y
