"""ctypes front end of the C restatement (bitstack_oracle.c).

TEST INFRASTRUCTURE ONLY - see the header of bitstack_oracle.c.  Arrays are
numpy; fp16 tensors travel as uint16 bit patterns.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libbitstack_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        P = ctypes.c_void_p
        i64, i32 = ctypes.c_int64, ctypes.c_int
        L.bso_pack_sign.restype = i64
        L.bso_pack_sign.argtypes = [P, i64, P]
        L.bso_unpack_sign.restype = None
        L.bso_unpack_sign.argtypes = [P, i64, P]
        L.bso_h2f.argtypes = [P, P, i64]
        L.bso_f2h.argtypes = [P, P, i64]
        L.bso_reconstruct_w.argtypes = [P, P, P, i32, i32, i32, i32, P]
        L.bso_forward_l0.argtypes = [P, P, P, P, P, i32, i32, i32, i32, i32, P]
        L.bso_forward_f64.argtypes = [P, P, P, P, P, i32, i32, i32, i32, i32, P]
        L.bso_num_threads.restype = i32
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _h(a):
    """fp16 array -> contiguous uint16 view."""
    return np.ascontiguousarray(a, dtype=np.float16).view(np.uint16)


def pack_sign(sign):
    s = _c(sign, np.int8).reshape(-1)
    out = np.empty((s.size + 7) // 8, dtype=np.uint8)
    if lib().bso_pack_sign(_p(s), s.size, _p(out)) < 0:
        raise AssertionError("pack_sign expects +-1 entries")
    return out


def unpack_sign(packed, shape):
    p = _c(packed, np.uint8).reshape(-1)
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n, dtype=np.int8)
    lib().bso_unpack_sign(_p(p), n, _p(out))
    return out.reshape(shape)


def h2f(a):
    a = _c(a, np.uint16).reshape(-1)
    out = np.empty(a.size, dtype=np.float32)
    lib().bso_h2f(_p(a), _p(out), a.size)
    return out


def f2h(a):
    a = _c(a, np.float32).reshape(-1)
    out = np.empty(a.size, dtype=np.uint16)
    lib().bso_f2h(_p(a), _p(out), a.size)
    return out


def _dims(u, vt):
    I, M, K = u.shape
    return I, M, vt.shape[2], K


def reconstruct_w(qweight, u, vt):
    I, M, N, K = _dims(u, vt)
    q, uu, vv = _c(qweight, np.uint8), _h(u), _h(vt)
    out = np.empty((M, N), dtype=np.uint16)
    lib().bso_reconstruct_w(_p(q), _p(uu), _p(vv), I, M, N, K, _p(out))
    return out.view(np.float16)


def forward_l0(qweight, u, vt, x, bias=None):
    I, M, N, K = _dims(u, vt)
    q, uu, vv, xx = _c(qweight, np.uint8), _h(u), _h(vt), _h(x).reshape(-1, N)
    bb = None if bias is None else _h(bias)
    T = xx.shape[0]
    out = np.empty((T, M), dtype=np.uint16)
    lib().bso_forward_l0(_p(q), _p(uu), _p(vv), _p(xx), _p(bb), I, M, N, K, T, _p(out))
    return out.view(np.float16).reshape(x.shape[:-1] + (M,))


def forward_f64(qweight, u, vt, x, bias=None):
    I, M, N, K = _dims(u, vt)
    q, uu, vv, xx = _c(qweight, np.uint8), _h(u), _h(vt), _h(x).reshape(-1, N)
    bb = None if bias is None else _h(bias)
    T = xx.shape[0]
    out = np.empty((T, M), dtype=np.float64)
    lib().bso_forward_f64(_p(q), _p(uu), _p(vv), _p(xx), _p(bb), I, M, N, K, T, _p(out))
    return out.reshape(x.shape[:-1] + (M,))


def num_threads():
    return int(lib().bso_num_threads())
