"""ctypes front end of oracle/la_oracle.c (plain-C fp64 brute force).

Test infrastructure only.  ``load()`` builds the library with ``make`` when the
shared object is absent (gcc only, no GPU, < 1 s)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libla_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float64))


def naive_fwd(q, k, v, s=None):
    lib = load()
    q, k, v = _c(q), _c(k), _c(v)
    b, h, n, d = q.shape
    e = v.shape[-1]
    o = np.empty((b, h, n, e), dtype=np.float64)
    sp = None if s is None else _c(np.asarray(s).reshape(-1))
    lib.la_naive_fwd(_p(q), _p(k), _p(v), None if sp is None else _p(sp), _p(o),
                     *(ctypes.c_int64(t) for t in (b, h, n, d, e)))
    return o


def naive_bwd(q, k, v, s, do):
    lib = load()
    q, k, v, do = _c(q), _c(k), _c(v), _c(do)
    b, h, n, d = q.shape
    e = v.shape[-1]
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    sp = None if s is None else _c(np.asarray(s).reshape(-1))
    lib.la_naive_bwd(_p(q), _p(k), _p(v), None if sp is None else _p(sp), _p(do), _p(dq), _p(dk), _p(dv),
                     *(ctypes.c_int64(t) for t in (b, h, n, d, e)))
    return dq, dk, dv


def slopes(h):
    lib = load()
    out = np.empty(h, dtype=np.float64)
    lib.la_slopes(_p(out), ctypes.c_int64(h))
    return out


def srms_fwd(x, eps):
    lib = load()
    x = _c(x)
    rows, cols = x.shape
    y = np.empty_like(x)
    rstd = np.empty(rows, dtype=np.float64)
    lib.srms_fwd(_p(x), _p(y), _p(rstd), ctypes.c_int64(rows), ctypes.c_int64(cols), ctypes.c_double(eps))
    return y, rstd


def srms_bwd(x, dy, eps):
    lib = load()
    x, dy = _c(x), _c(dy)
    rows, cols = x.shape
    dx = np.empty_like(x)
    lib.srms_bwd(_p(x), _p(dy), _p(dx), ctypes.c_int64(rows), ctypes.c_int64(cols), ctypes.c_double(eps))
    return dx
