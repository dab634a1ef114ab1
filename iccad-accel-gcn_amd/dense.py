"""The dense side of a GCN layer around the sparse product: Z = X W on the GPU's fp32
matrix cores (accel_dense_xw), and the layer Y = act(A (X W) + bias) as two launches.

Upstream's operator takes the dense operand as given (spmm_accel.cu:16-102 computes
A X and stops); a layer that uses it multiplies the features by its weights first.
"""
from __future__ import annotations

import numpy as np

from . import _lib
from ._lib import AccelError, DeviceBuffer, check, lib, ptr


def dense_xw(X, W, Z, rows: int, K: int, N: int, ldx: int = 0, ldz: int = 0, stream=None) -> None:
    """Z = X W on device operands (DeviceBuffer, anything with ``data_ptr()``, or a raw
    address): X ``rows x K`` with rows ``ldx`` floats apart (0: packed), W ``K x N`` packed,
    Z ``rows x N`` with rows ``ldz`` apart.  Asynchronous on ``stream``."""
    rows, K, N, ldx, ldz = int(rows), int(K), int(N), int(ldx), int(ldz)
    sx, sz = ldx or K, ldz or N
    if rows < 0 or K <= 0 or N <= 0 or sx < K or sz < N:
        raise AccelError(_lib.ERR_ARG, f"bad shape: rows={rows}, K={K}, N={N}, ldx={ldx}, ldz={ldz}")
    x = _lib.dev_ptr(X, ((rows - 1) * sx + K) * 4 if rows else 0, "X")
    w = _lib.dev_ptr(W, K * N * 4, "W")
    z = _lib.dev_ptr(Z, ((rows - 1) * sz + N) * 4 if rows else 0, "Z")
    check(lib().accel_dense_xw(x, w, z, rows, K, N, ldx, ldz, ptr(stream)))


def dense_xw_numpy(X: np.ndarray, W: np.ndarray) -> np.ndarray:
    """numpy in, numpy out: copies X and W up, Z down."""
    X, W = _lib.as_f32(X), _lib.as_f32(W)
    if X.ndim != 2 or W.ndim != 2 or X.shape[1] != W.shape[0] or W.shape[0] == 0 or W.shape[1] == 0:
        raise AccelError(_lib.ERR_ARG, f"shapes {X.shape} and {W.shape} do not multiply")
    rows, K = X.shape
    N = W.shape[1]
    dX, dW = DeviceBuffer.from_numpy(X), DeviceBuffer.from_numpy(W)
    dZ = DeviceBuffer(max(rows * N * 4, 4))
    dZ.fill_u32(0x7FC00000)               # NaN: an element the kernel fails to write shows up
    try:
        dense_xw(dX, dW, dZ, rows, K, N)
        check(lib().accel_stream_sync(None))
        return dZ.to_numpy(np.float32, (rows, N))
    finally:
        dX.close(); dW.close(); dZ.close()


class GcnLayer:
    """Y = act(A (X W) + bias): ``accel_dense_xw`` into a buffer the layer owns, then the
    sparse product with bias and ReLU in its store (``accel_run_epilogue``), both queued on
    the caller's stream.  ``op`` is a preprocessed ``AccelSpMM``; ``W`` is ``K x N`` (numpy,
    uploaded once), ``bias`` ``N`` floats or None."""

    def __init__(self, op, W: np.ndarray, bias: np.ndarray | None = None, relu: bool = True):
        W = _lib.as_f32(W)
        if W.ndim != 2 or W.size == 0:
            raise AccelError(_lib.ERR_ARG, "W must be a non-empty K x N matrix")
        self.op, self.relu = op, bool(relu)
        self.K, self.N = W.shape
        self._w = DeviceBuffer.from_numpy(W)
        self._b = None
        if bias is not None:
            b = _lib.as_f32(bias)
            if b.shape != (self.N,):
                raise AccelError(_lib.ERR_ARG, f"bias must hold {self.N} floats")
            self._b = DeviceBuffer.from_numpy(b)
        self._z = DeviceBuffer(max(op.n_cols * self.N * 4, 4))      # X W: the sparse product's dense operand

    def forward(self, X, Y, stream=None) -> None:
        """X: ``n_cols x K`` on the device, Y: ``n_rows x N`` on the device."""
        dense_xw(X, self._w, self._z, self.op.n_cols, self.K, self.N, stream=stream)
        self.op.run_epilogue(self._z, Y, self.N, bias=self._b, relu=self.relu, stream=stream)

    def forward_numpy(self, X: np.ndarray) -> np.ndarray:
        X = _lib.as_f32(X)
        if X.shape != (self.op.n_cols, self.K):
            raise AccelError(_lib.ERR_ARG, f"X must be [{self.op.n_cols}, {self.K}]")
        dX = DeviceBuffer.from_numpy(X)
        dY = DeviceBuffer(max(self.op.n_rows * self.N * 4, 4))
        dY.fill_u32(0x7FC00000)
        try:
            self.forward(dX, dY)
            check(lib().accel_stream_sync(None))
            return dY.to_numpy(np.float32, (self.op.n_rows, self.N))
        finally:
            dX.close(); dY.close()

    def close(self) -> None:
        for b in (self._w, self._b, self._z):
            if b is not None:
                b.close()
        self._w = self._b = self._z = None
