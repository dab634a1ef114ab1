"""CPU oracle for the SpMM itself.

TEST INFRASTRUCTURE ONLY (see partition_oracle.py for the rule).

The product is checked against scipy's ``csr_matrix @ dense``: upstream checks
its kernel against cuSPARSE CSR SpMM with alpha=1, beta=0 (main.cu:143-155,
spmm_cusparse.cu:6-62), which is not available here; scipy computes the same
quantity.  Because fp32 summation order differs between any two
implementations, the acceptance metric is scaled by the size of the terms:

    err = max_ij |Y_ij - R_ij| / max(S_ij, tiny),   R = A X in fp64,  S = |A| |X|

and the bound is 1e-5.  Upstream's own bar (mean |diff| < 1e-3, main.cu:18-51)
is far looser and is reported only for completeness.

Pinned by: brute-force dense products on small inputs, closed forms (all-ones
-> row degree, identity -> X), linearity, and agreement with the C restatement
(oracle.c) which is written independently of scipy.
"""
from __future__ import annotations

import numpy as np
import scipy.sparse as sp

TOL = 1e-5


def csr(indptr, indices, values, n_cols):
    n_rows = len(indptr) - 1
    return sp.csr_matrix((values, indices, indptr), shape=(n_rows, n_cols))


def spmm_scipy32(indptr, indices, values, X):
    """The named baseline: scipy CSR @ C-contiguous fp32 dense, single thread."""
    X = np.ascontiguousarray(X, dtype=np.float32)
    A = csr(indptr, indices, np.asarray(values, dtype=np.float32), X.shape[0])
    return np.asarray(A @ X, dtype=np.float32)


def spmm_fp64(indptr, indices, values, X):
    """(R, S): fp64 product and the fp64 product of absolute values."""
    X64 = np.ascontiguousarray(X, dtype=np.float64)
    v64 = np.asarray(values, dtype=np.float64)
    A = csr(indptr, indices, v64, X64.shape[0])
    Aabs = csr(indptr, indices, np.abs(v64), X64.shape[0])
    return np.asarray(A @ X64), np.asarray(Aabs @ np.abs(X64))


def scaled_error(Y, R, S):
    """max |Y - R| / max(S, tiny); rows with S == 0 must be exactly 0."""
    Y = np.asarray(Y, dtype=np.float64)
    tiny = np.finfo(np.float32).tiny
    return float(np.max(np.abs(Y - R) / np.maximum(S, tiny))) if Y.size else 0.0


def upstream_mean_abs_error(Y, Yref):
    """Upstream's acceptance figure: sum |diff| / len < 1e-3 (main.cu:18-51)."""
    Y = np.asarray(Y, dtype=np.float64)
    return float(np.abs(Y - np.asarray(Yref, dtype=np.float64)).mean()) if Y.size else 0.0


def check(Y, indptr, indices, values, X, tol=TOL):
    R, S = spmm_fp64(indptr, indices, values, X)
    return scaled_error(Y, R, S)


# --- the dense product in front of the sparse one (Z = X W) -------------------------------
# No reference counterpart (upstream's operator stops at A X, spmm_accel.cu:16-102): the
# definition is the textbook matrix product, computed here by numpy in fp64.  Pinned by a
# triple loop on small inputs, identity -> X, all-ones -> row sums, and a dropped-term
# detector (tests/test_oracle_spmm.py).
def dense_fp64(X, W):
    """(R, S): X W in fp64 and |X| |W| in fp64 (the scale of the terms)."""
    X64 = np.asarray(X, dtype=np.float64)
    W64 = np.asarray(W, dtype=np.float64)
    return X64 @ W64, np.abs(X64) @ np.abs(W64)


def check_dense(Z, X, W):
    R, S = dense_fp64(X, W)
    return scaled_error(Z, R, S)
