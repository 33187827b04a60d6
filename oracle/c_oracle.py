"""ctypes binding of the C restatement (``lce_oracle.c``).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblce_oracle.so")


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-B", "liblce_oracle.so"], check=True, capture_output=True)
    return _SO


def _lib():
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    d = ctypes.c_double
    p = ctypes.c_void_p
    i64 = ctypes.c_int64
    lib.lce_oracle_forward.argtypes = [p, p, p, i64, i64, i64, d, p, p, p, p, p]
    lib.lce_oracle_backward.argtypes = [p, p, p, i64, i64, i64, d, p, p, p, p]
    return lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def forward(hidden, weight, labels, temperature=1.0):
    """numpy in (fp32 [T,H], fp32 [V,H], int64 [T]) -> dict of float64 [T] arrays."""
    h = np.ascontiguousarray(hidden, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    y = np.ascontiguousarray(labels, dtype=np.int64)
    T, H = h.shape
    V = w.shape[0]
    out = {k: np.empty(T, dtype=np.float64) for k in ("logprob", "entropy", "max", "accu", "eb")}
    rc = _lib().lce_oracle_forward(_ptr(h), _ptr(w), _ptr(y), T, H, V, float(temperature),
                                   *[_ptr(out[k]) for k in ("logprob", "entropy", "max", "accu", "eb")])
    if rc != 0:
        raise ValueError("label out of range")
    return out


def backward(hidden, weight, labels, g_lp, g_ent, temperature=1.0):
    h = np.ascontiguousarray(hidden, dtype=np.float32)
    w = np.ascontiguousarray(weight, dtype=np.float32)
    y = np.ascontiguousarray(labels, dtype=np.int64)
    glp = np.ascontiguousarray(g_lp, dtype=np.float64)
    gent = None if g_ent is None else np.ascontiguousarray(g_ent, dtype=np.float64)
    T, H = h.shape
    V = w.shape[0]
    dh = np.empty((T, H), dtype=np.float64)
    dw = np.empty((V, H), dtype=np.float64)
    _lib().lce_oracle_backward(_ptr(h), _ptr(w), _ptr(y), T, H, V, float(temperature), _ptr(glp),
                               None if gent is None else _ptr(gent), _ptr(dh), _ptr(dw))
    return dh, dw
