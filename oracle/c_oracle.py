"""ctypes loader for the C oracle (``oracle/oracle.c``).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build() -> str:
    """(Re)build ``oracle/_build/liboracle.so`` with gcc via the Makefile."""
    subprocess.run(["make", "-s", "-B", "-C", _HERE], check=True)
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        lib = ctypes.CDLL(_SO)
        fp = ctypes.POINTER(ctypes.c_float)
        lib.oracle_causal_dot_product_fwd.argtypes = [fp, fp, fp, fp, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.oracle_causal_dot_product_fwd.restype = ctypes.c_int
        lib.oracle_causal_dot_product_bwd.argtypes = [fp] * 7 + [ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.oracle_causal_dot_product_bwd.restype = ctypes.c_int
        _lib = lib
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def fwd(q, k, v) -> np.ndarray:
    """O for (B, H, N, D) arrays (anything ``np.asarray`` accepts)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    o = np.empty((b, h, n, dv), dtype=np.float32)
    rc = _load().oracle_causal_dot_product_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(o), b * h, n, dqk, dv)
    if rc != 0:
        raise RuntimeError(f"oracle_causal_dot_product_fwd returned {rc}")
    return o


def bwd(q, k, v, do) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """(dQ, dK, dV) for (B, H, N, D) arrays."""
    q, k, v, do = _f32(q), _f32(k), _f32(v), _f32(do)
    b, h, n, dqk = q.shape
    dv_ = v.shape[-1]
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    rc = _load().oracle_causal_dot_product_bwd(
        _ptr(q), _ptr(k), _ptr(v), _ptr(do), _ptr(dq), _ptr(dk), _ptr(dv), b * h, n, dqk, dv_
    )
    if rc != 0:
        raise RuntimeError(f"oracle_causal_dot_product_bwd returned {rc}")
    return dq, dk, dv
