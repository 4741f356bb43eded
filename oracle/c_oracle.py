"""ctypes loader for the C restatement (oracle/spfa_oracle.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libspfa_oracle.so")
_lib = None

DEFAULT_CHUNK = 46  # columns per loop trip of the reference at d=64 on a 48 KiB-smem part

_STATUS_TO_EXC = {
    5: "The embedded dimension is too large for the amount of shared memory on your GPU.",
    6: "The local size specified is either negative or greater than/equal to (1 - Sequence Length).",
    7: "The dilation factor must be atleast 0.",
    8: "The block/window size must be a divisor of the whole tensor's size.",
    9: "The dilation factor must be less than the block/window size.",
    10: "There are either no global tokens provided or there are more than the sequence length given.",
}


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "spfa_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libspfa_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _d(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _p(a, ty):
    return a.ctypes.data_as(ctypes.POINTER(ty))


def _state(n, d, m, l, out):
    m = np.full(n, -np.inf) if m is None else _d(m).copy()
    l = np.zeros(n) if l is None else _d(l).copy()
    out = np.zeros((n, d)) if out is None else _d(out).copy()
    return m, l, out


def _check(rc):
    if rc != 0:
        raise ValueError(_STATUS_TO_EXC.get(rc, "oracle status %d" % rc))


_D = ctypes.c_double
_I64 = ctypes.c_int64


def csr(q, k, v, row_off, col_ind, m=None, l=None, out=None, use_nan=False, chunk=DEFAULT_CHUNK):
    q, k, v = _d(q), _d(k), _d(v)
    n, d = q.shape
    m, l, out = _state(n, d, m, l, out)
    ro = np.ascontiguousarray(row_off, dtype=np.int64)
    ci = np.ascontiguousarray(col_ind, dtype=np.int64)
    _check(lib().spfa_oracle_csr(_I64(n), _I64(d), _p(q, _D), _p(k, _D), _p(v, _D), _p(ro, _I64),
                                 _p(ci, _I64), _p(m, _D), _p(l, _D), _p(out, _D),
                                 ctypes.c_int(bool(use_nan)), ctypes.c_int(chunk)))
    return out, m, l


def coo(q, k, v, row_ind, col_ind, m=None, l=None, out=None, use_nan=False, chunk=DEFAULT_CHUNK):
    q, k, v = _d(q), _d(k), _d(v)
    n, d = q.shape
    m, l, out = _state(n, d, m, l, out)
    ri = np.ascontiguousarray(row_ind, dtype=np.int64)
    ci = np.ascontiguousarray(col_ind, dtype=np.int64)
    _check(lib().spfa_oracle_coo(_I64(n), _I64(d), _p(q, _D), _p(k, _D), _p(v, _D), _p(ri, _I64),
                                 _p(ci, _I64), _I64(ri.shape[0]), _p(m, _D), _p(l, _D), _p(out, _D),
                                 ctypes.c_int(bool(use_nan)), ctypes.c_int(chunk)))
    return out, m, l


def local(q, k, v, w, m=None, l=None, out=None, chunk=DEFAULT_CHUNK):
    q, k, v = _d(q), _d(k), _d(v)
    n, d = q.shape
    m, l, out = _state(n, d, m, l, out)
    _check(lib().spfa_oracle_local(_I64(n), _I64(d), _p(q, _D), _p(k, _D), _p(v, _D), _p(m, _D),
                                   _p(l, _D), _p(out, _D), _I64(w), ctypes.c_int(chunk)))
    return out, m, l


def local_1d_dilated(q, k, v, w, dil, m=None, l=None, out=None, chunk=DEFAULT_CHUNK):
    q, k, v = _d(q), _d(k), _d(v)
    n, d = q.shape
    m, l, out = _state(n, d, m, l, out)
    _check(lib().spfa_oracle_local_1d_dilated(_I64(n), _I64(d), _p(q, _D), _p(k, _D), _p(v, _D),
                                              _p(m, _D), _p(l, _D), _p(out, _D), _I64(w), _I64(dil),
                                              ctypes.c_int(chunk)))
    return out, m, l


def local_2d_dilated(q, k, v, block, dil, m=None, l=None, out=None, use_nan=False,
                     chunk=DEFAULT_CHUNK):
    q, k, v = _d(q), _d(k), _d(v)
    n, d = q.shape
    m, l, out = _state(n, d, m, l, out)
    _check(lib().spfa_oracle_local_2d_dilated(_I64(n), _I64(d), _p(q, _D), _p(k, _D), _p(v, _D),
                                              _p(m, _D), _p(l, _D), _p(out, _D), _I64(block),
                                              _I64(dil), ctypes.c_int(bool(use_nan)),
                                              ctypes.c_int(chunk)))
    return out, m, l


def global_no_local(q, k, v, globs, w, m=None, l=None, out=None, chunk=DEFAULT_CHUNK):
    q, k, v = _d(q), _d(k), _d(v)
    n, d = q.shape
    m, l, out = _state(n, d, m, l, out)
    g = np.ascontiguousarray(globs, dtype=np.int32)
    _check(lib().spfa_oracle_global_no_local(_I64(n), _I64(d), _p(q, _D), _p(k, _D), _p(v, _D),
                                             _p(m, _D), _p(l, _D), _p(out, _D),
                                             _p(g, ctypes.c_int32), _I64(g.shape[0]), _I64(w),
                                             ctypes.c_int(chunk)))
    return out, m, l
