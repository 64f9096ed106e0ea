"""ctypes front end of oracle/oracle_kernels.c.  TEST INFRASTRUCTURE ONLY.

Loads ``oracle/liboracle.so`` (built by ``make -C oracle`` or ``__graft_entry__.build()``)
and exposes the fp64-accumulating CPU kernels on numpy arrays.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force: bool = False) -> str:
    path = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(path):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return path


def lib():
    global _LIB
    if _LIB is None:
        _LIB = C.CDLL(build())
        _LIB.orc_softmax_xent.restype = C.c_double
    return _LIB


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def csr_spmm(rowptr, col, val, h, acc64: bool = True):
    """Y = A.H on the host; fp32 storage with fp64 (default) or fp32 accumulation; fp64 in -> fp64."""
    rowptr, col = _i64(rowptr), _i64(col)
    m = rowptr.size - 1
    h = np.ascontiguousarray(h)
    d = h.shape[1]
    if h.dtype == np.float64:
        val = np.ascontiguousarray(val, dtype=np.float64)
        y = np.empty((m, d), dtype=np.float64)
        lib().orc_csr_spmm_f64(C.c_int64(m), _p(rowptr), _p(col), _p(val), _p(h), C.c_int64(d), C.c_int64(d),
                               _p(y), C.c_int64(d))
        return y
    val = np.ascontiguousarray(val, dtype=np.float32)
    h = h.astype(np.float32, copy=False)
    y = np.empty((m, d), dtype=np.float32)
    fn = lib().orc_csr_spmm_f32_acc64 if acc64 else lib().orc_csr_spmm_f32
    fn(C.c_int64(m), _p(rowptr), _p(col), _p(val), _p(h), C.c_int64(d), C.c_int64(d), _p(y), C.c_int64(d))
    return y


def gemm(a, b, ta: bool = False, tb: bool = False):
    """C = op(A).op(B), fp32 storage, fp64 accumulation."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m = a.shape[1] if ta else a.shape[0]
    k = a.shape[0] if ta else a.shape[1]
    n = b.shape[0] if tb else b.shape[1]
    c = np.empty((m, n), dtype=np.float32)
    lib().orc_gemm_f32_acc64(C.c_int(int(ta)), C.c_int(int(tb)), C.c_int64(m), C.c_int64(n), C.c_int64(k),
                             _p(a), C.c_int64(a.shape[1]), _p(b), C.c_int64(b.shape[1]), _p(c), C.c_int64(n))
    return c


def softmax_xent(logits, labels, num_nodes: int, num_classes: int, gscale: float = 1.0):
    """(loss, dlogits) of the reference's cross-entropy, fp64 math on fp32 logits."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    labels = _i64(labels)
    m, c = logits.shape
    d = np.empty((m, c), dtype=np.float32)
    loss = lib().orc_softmax_xent(C.c_int64(m), C.c_int64(c), _p(logits), C.c_int64(c), _p(labels),
                                  C.c_int64(num_nodes), C.c_int64(num_classes), C.c_double(gscale), _p(d),
                                  C.c_int64(c))
    return float(loss), d


def gcn_norm_csr(rowptr, col, val):
    rowptr, col = _i64(rowptr), _i64(col)
    val = np.ascontiguousarray(val, dtype=np.float32)
    out = np.empty_like(val)
    lib().orc_gcn_norm_csr(C.c_int64(rowptr.size - 1), _p(rowptr), _p(col), _p(val), _p(out))
    return out
