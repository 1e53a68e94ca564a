"""ctypes binding of the brute-force C oracle (``xkv_oracle.c``).  Test infrastructure only."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libxkv_oracle.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "xkv_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-fPIC", "-shared", "-o", _SO, src, "-lm"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _d(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float64))


_i = ctypes.c_int64
_f = ctypes.c_double


def split_bounds(kv_len, splits, sid):
    s, e = _i(), _i()
    lib().xo_split_bounds(_i(kv_len), _i(splits), _i(sid), ctypes.byref(s), ctypes.byref(e))
    return s.value, e.value


def rope_cs(pos, j, dim, theta):
    c, s = _f(), _f()
    lib().xo_rope_cs(_i(pos), _i(j), _i(dim), _f(theta), ctypes.byref(c), ctypes.byref(s))
    return c.value, s.value


def qab(q, A, B, rope=False, theta=0.0, pos0=0):
    q, A, B = _d(q), _d(A), _d(B)
    b, hq, d = q.shape
    _, L, r = A.shape
    hkv = B.shape[1]
    out = np.empty((b, hq, L))
    lib().xo_qab(_p(q), _p(A), _p(B), _p(out), _i(b), _i(hq), _i(hkv), _i(d), _i(L), _i(r),
                 ctypes.c_int(int(rope)), _f(theta), _i(pos0))
    return out


def decode_factorized(q, kA, kB, vA, vB, sm_scale, rope=False, theta=0.0, pos0=0):
    q, kA, kB, vA, vB = map(_d, (q, kA, kB, vA, vB))
    b, hq, d = q.shape
    _, L, rk = kA.shape
    hkv = kB.shape[1]
    rv = vA.shape[2]
    out = np.empty((b, hq, d))
    lib().xo_decode_factorized(_p(q), _p(kA), _p(kB), _p(vA), _p(vB), _p(out), _i(b), _i(hq), _i(hkv),
                               _i(d), _i(L), _i(rk), _i(rv), _f(sm_scale),
                               ctypes.c_int(int(rope)), _f(theta), _i(pos0))
    return out


def decode_plain(q, K, V, sm_scale):
    q, K, V = map(_d, (q, K, V))
    b, hq, dk = q.shape
    _, L, hkv, _ = K.shape
    dv = V.shape[-1]
    out = np.empty((b, hq, dv))
    lib().xo_decode_plain(_p(q), _p(K), _p(V), _p(out), _i(b), _i(hq), _i(hkv), _i(dk), _i(dv), _i(L),
                          _f(sm_scale))
    return out


def mla(qn, qr, ckv, kpe, sm_scale):
    qn, qr, ckv, kpe = map(_d, (qn, qr, ckv, kpe))
    b, H, c = qn.shape
    e = qr.shape[-1]
    L = ckv.shape[1]
    out = np.empty((b, H, c))
    lib().xo_mla(_p(qn), _p(qr), _p(ckv.reshape(b, L, c)), _p(kpe.reshape(b, L, e)), _p(out),
                 _i(b), _i(H), _i(c), _i(e), _i(L), _f(sm_scale))
    return out
