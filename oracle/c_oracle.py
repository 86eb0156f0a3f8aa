"""ctypes binding of the plain-C oracle (``naive_attention.c``).  Test infrastructure only."""

from __future__ import annotations

import ctypes
import pathlib
import subprocess

import numpy as np

_HERE = pathlib.Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "liboracle_attention.so"
_lib = None


def build() -> pathlib.Path:
    """Compile naive_attention.c with gcc (seconds)."""
    subprocess.run(["make", "-s", "-C", str(_HERE)], check=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(_LIB_PATH))
        dp = ctypes.POINTER(ctypes.c_double)
        lib.oracle_attention_forward.argtypes = [dp, dp, dp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                 ctypes.c_double, dp, dp]
        lib.oracle_attention_forward.restype = ctypes.c_int
        lib.oracle_attention_backward.argtypes = [dp, dp, dp, dp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                  ctypes.c_double, dp, dp, dp, dp]
        lib.oracle_attention_backward.restype = ctypes.c_int
        _lib = lib
    return _lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def forward(q, k, v, scale):
    """One (batch, head) slice: q [nq, d], k/v [nk, d] -> (o [nq, d], lse [nq]) in fp64."""
    q, k, v = (np.ascontiguousarray(np.asarray(t, dtype=np.float64)) for t in (q, k, v))
    nq, d = q.shape
    nk = k.shape[0]
    o = np.empty((nq, d), dtype=np.float64)
    lse = np.empty((nq,), dtype=np.float64)
    rc = _load().oracle_attention_forward(_ptr(q), _ptr(k), _ptr(v), nq, nk, d, float(scale), _ptr(o), _ptr(lse))
    if rc != 0:
        raise MemoryError("oracle_attention_forward failed")
    return o, lse


def backward(q, k, v, d_o, scale):
    """One slice -> (dq, dk, dv, delta) in fp64."""
    q, k, v, d_o = (np.ascontiguousarray(np.asarray(t, dtype=np.float64)) for t in (q, k, v, d_o))
    nq, d = q.shape
    nk = k.shape[0]
    dq = np.empty((nq, d), dtype=np.float64)
    dk = np.empty((nk, d), dtype=np.float64)
    dv = np.empty((nk, d), dtype=np.float64)
    delta = np.empty((nq,), dtype=np.float64)
    rc = _load().oracle_attention_backward(_ptr(q), _ptr(k), _ptr(v), _ptr(d_o), nq, nk, d, float(scale),
                                           _ptr(dq), _ptr(dk), _ptr(dv), _ptr(delta))
    if rc != 0:
        raise MemoryError("oracle_attention_backward failed")
    return dq, dk, dv, delta
