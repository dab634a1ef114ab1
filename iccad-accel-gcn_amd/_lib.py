"""ctypes binding of lib/libaccelgcn.so (the C ABI in include/accel_gcn.h).

The library is the product: if it is missing or will not load, importing the
operator fails with an error that says how to build it.  There is no Python or
CPU stand-in for any GPU entry point.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libaccelgcn.so"

OK, ERR_ARG, ERR_CSR, ERR_ALLOC, ERR_HIP, ERR_META, ERR_STATE, ERR_IO = 0, -1, -2, -3, -4, -5, -6, -7
PTR_HOST, PTR_DEVICE = 0, 1
EPILOGUE_RELU = 1
DEG_BOUND = 384
SLICES_PER_BLOCK = 12
STATIC_SCRATCH_BYTES = 32 << 20

_STATUS_NAME = {ERR_ARG: "ACCEL_ERR_ARG", ERR_CSR: "ACCEL_ERR_CSR", ERR_ALLOC: "ACCEL_ERR_ALLOC",
                ERR_HIP: "ACCEL_ERR_HIP", ERR_META: "ACCEL_ERR_META", ERR_STATE: "ACCEL_ERR_STATE",
                ERR_IO: "ACCEL_ERR_IO"}


class AccelError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"{_STATUS_NAME.get(status, status)}: {message}")
        self.status = status
        self.message = message


class Info(C.Structure):
    _fields_ = [("rows", C.c_int64), ("cols", C.c_int64), ("nnz", C.c_int64),
                ("n_blocks", C.c_int64), ("n_long_blocks", C.c_int64), ("n_long_rows", C.c_int64),
                ("n_zero_rows", C.c_int64), ("max_degree", C.c_int32), ("already_sorted", C.c_int32),
                ("preprocess_ms", C.c_double), ("n_plan_units", C.c_int64), ("n_split_rows", C.c_int64),
                ("plan_unit_nz", C.c_int32), ("plan_groups", C.c_int32),
                ("plan_split_nz", C.c_int32), ("plan_team", C.c_int32), ("plan_queues", C.c_int32),
                ("plan_reduce", C.c_int32), ("n_plan_pieces", C.c_int64)]


class RunArgs(C.Structure):
    """accel_run_args of include/accel_gcn.h."""
    _fields_ = [("X", C.c_void_p), ("Y", C.c_void_p), ("N", C.c_int32), ("ld", C.c_int32),
                ("bias", C.c_void_p), ("flags", C.c_int32), ("stream", C.c_void_p)]


i32p = C.POINTER(C.c_int32)
f32p = C.POINTER(C.c_float)
i64p = C.POINTER(C.c_int64)
vp = C.c_void_p

# name -> (restype, argtypes); every symbol include/accel_gcn.h declares
SIGNATURES = {
    "accel_last_error": (C.c_char_p, []),
    "accel_version": (C.c_int, []),
    "accel_partition_host": (C.c_int, [i32p, C.c_int64, i32p, C.c_int64, i64p]),
    "accel_degree_sort_host": (C.c_int, [i32p, C.c_int64, i32p]),
    "accel_partition_gpu": (C.c_int, [i32p, C.c_int64, i32p, C.c_int64, i64p]),
    "accel_file_count": (C.c_int, [C.c_char_p, i64p]),
    "accel_file_read": (C.c_int, [C.c_char_p, vp, C.c_int64]),
    "accel_file_write": (C.c_int, [C.c_char_p, vp, C.c_int64]),
    "accel_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "accel_dev_malloc": (C.c_int, [C.POINTER(vp), C.c_size_t]),
    "accel_dev_free": (C.c_int, [vp]),
    "accel_memcpy_h2d": (C.c_int, [vp, vp, C.c_size_t]),
    "accel_memcpy_d2h": (C.c_int, [vp, vp, C.c_size_t]),
    "accel_dev_fill_u32": (C.c_int, [vp, C.c_uint32, C.c_size_t, vp]),
    "accel_dev_copy_u32": (C.c_int, [vp, vp, C.c_size_t, vp]),
    "accel_stream_sync": (C.c_int, [vp]),
    "accel_create": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.POINTER(vp)]),
    "accel_preprocess": (C.c_int, [vp]),
    "accel_set_plan_unit": (C.c_int, [vp, C.c_int]),
    "accel_set_plan_groups": (C.c_int, [vp, C.c_int]),
    "accel_set_plan_split": (C.c_int, [vp, C.c_int]),
    "accel_set_plan_team": (C.c_int, [vp, C.c_int]),
    "accel_set_plan_panel": (C.c_int, [vp, C.c_int]),
    "accel_set_plan_queues": (C.c_int, [vp, C.c_int]),
    "accel_set_plan_reduce": (C.c_int, [vp, C.c_int]),
    "accel_save_state": (C.c_int, [vp, C.c_char_p]),
    "accel_load_state": (C.c_int, [vp, C.c_char_p]),
    "accel_update_values": (C.c_int, [vp, vp, C.c_int]),
    "accel_update_values_async": (C.c_int, [vp, vp, vp]),
    "accel_check_block4": (C.c_int, [vp, i32p, C.c_int64]),
    "accel_get_info": (C.c_int, [vp, C.POINTER(Info)]),
    "accel_get_block4": (C.c_int, [vp, i32p, C.c_int64]),
    "accel_get_plan": (C.c_int, [vp, i32p, C.c_int64, i64p]),
    "accel_get_perm": (C.c_int, [vp, i32p, C.c_int64]),
    "accel_get_sorted_csr": (C.c_int, [vp, i32p, i32p, f32p]),
    "accel_run": (C.c_int, [vp, vp, vp, C.c_int32, vp]),
    "accel_run_ex": (C.c_int, [vp, C.POINTER(RunArgs)]),
    "accel_run_strided": (C.c_int, [vp, vp, vp, C.c_int32, C.c_int32, vp]),
    "accel_reserve": (C.c_int, [vp, C.c_int32]),
    "accel_run_static": (C.c_int, [vp, vp, vp, C.c_int32, vp]),
    "accel_run_epilogue": (C.c_int, [vp, vp, vp, C.c_int32, vp, C.c_int, vp]),
    "accel_time": (C.c_int, [vp, vp, vp, C.c_int32, C.c_int, C.c_int, f32p, f32p, vp]),
    "accel_time_ex": (C.c_int, [vp, C.POINTER(RunArgs), C.c_int, C.c_int, f32p, f32p]),
    "accel_dense_xw": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32, vp]),
    "accel_destroy": (C.c_int, [vp]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, gfx950). There is no fallback implementation.")
        L = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)          # AttributeError if the ABI lost a symbol
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error() -> str:
    return (lib().accel_last_error() or b"").decode("utf-8", "replace")


def check(status: int) -> None:
    if status != OK:
        raise AccelError(status, last_error())


def as_i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def as_f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def ptr(a, ctype=None):
    """Raw address of a numpy array, DeviceBuffer, object with data_ptr(), or int."""
    if a is None:
        return None
    if isinstance(a, np.ndarray):
        return a.ctypes.data_as(C.POINTER(ctype)) if ctype else C.c_void_p(a.ctypes.data)
    if isinstance(a, DeviceBuffer):
        return C.c_void_p(a.address)
    if hasattr(a, "data_ptr"):
        return C.c_void_p(int(a.data_ptr()))
    return C.c_void_p(int(a))


def dev_ptr(a, need_bytes: int, name: str):
    """Address of a dense operand on the device.  A numpy array is host memory and is
    refused here (the kernels would fault on it); where the object tells its size, that
    size must cover ``need_bytes``.  Raw integer addresses are passed through: the
    library asks the HIP runtime about them."""
    if a is None:
        return None
    if isinstance(a, np.ndarray):
        raise AccelError(ERR_ARG, f"{name} is a numpy array (host memory); pass a DeviceBuffer, an object "
                                  "with data_ptr() on the GPU, or a device address")
    have = None
    if isinstance(a, DeviceBuffer):
        if not a.address:
            raise AccelError(ERR_ARG, f"{name} is a closed DeviceBuffer")
        have = a.nbytes
    elif hasattr(a, "data_ptr"):
        if getattr(a, "is_cuda", True) is False:
            raise AccelError(ERR_ARG, f"{name} is a host tensor; move it to the GPU first")
        if hasattr(a, "numel") and hasattr(a, "element_size"):
            have = int(a.numel()) * int(a.element_size())
    if have is not None and have < need_bytes:
        raise AccelError(ERR_ARG, f"{name} holds {have} bytes, {need_bytes} needed")
    return ptr(a)


class DeviceBuffer:
    """A hipMalloc allocation owned by Python (freed on close() or collection)."""

    def __init__(self, nbytes: int):
        p = C.c_void_p()
        check(lib().accel_dev_malloc(C.byref(p), int(nbytes)))
        self.address = p.value or 0
        self.nbytes = int(nbytes)

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        if a.nbytes:
            check(lib().accel_memcpy_h2d(C.c_void_p(buf.address), C.c_void_p(a.ctypes.data), a.nbytes))
        return buf

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        if out.nbytes > self.nbytes:
            raise ValueError("requested view is larger than the allocation")
        if out.nbytes:
            check(lib().accel_memcpy_d2h(C.c_void_p(out.ctypes.data), C.c_void_p(self.address), out.nbytes))
        return out

    def fill_u32(self, value: int = 0) -> None:
        check(lib().accel_dev_fill_u32(C.c_void_p(self.address), value, self.nbytes // 4, None))

    def data_ptr(self) -> int:
        return self.address

    def close(self) -> None:
        if self.address:
            lib().accel_dev_free(C.c_void_p(self.address))
            self.address = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def device_count() -> int:
    n = C.c_int(0)
    rc = lib().accel_device_count(C.byref(n))
    return n.value if rc == OK else 0
