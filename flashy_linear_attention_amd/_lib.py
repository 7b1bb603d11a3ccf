"""ctypes binding of ``libfla_gfx950.so`` (C ABI declared in ``include/fla.h``).

There is no fallback: if the shared library is missing or does not export the
expected ABI, loading raises and every operator call fails.
"""

from __future__ import annotations

import ctypes
import os
import threading

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libfla_gfx950.so")
ABI_VERSION = 4

FLA_DTYPE_BF16 = 0
FLA_DTYPE_F16 = 1

_i64 = ctypes.c_int64
_ptr = ctypes.c_void_p
_strides = ctypes.POINTER(ctypes.c_int64)

# name -> argtypes, exactly as declared in include/fla.h
SIGNATURES = {
    "fla_abi_version": ([], ctypes.c_int),
    "fla_strerror": ([ctypes.c_int], ctypes.c_char_p),
    "fla_linear_attn_fwd": ([_ptr] * 4 + [_i64] * 4 + [_strides] * 4 + [ctypes.c_int, _ptr], ctypes.c_int),
    "fla_linear_attn_bwd": ([_ptr] * 7 + [_i64] * 4 + [_strides] * 7 + [ctypes.c_int, _ptr], ctypes.c_int),
    "fla_linear_attn_smallv_fwd": ([_ptr] * 4 + [_i64] * 5 + [_strides] * 4 + [ctypes.c_int, _ptr], ctypes.c_int),
    "fla_linear_attn_smallv_bwd": ([_ptr] * 7 + [_i64] * 5 + [_strides] * 7 + [ctypes.c_int, _ptr], ctypes.c_int),
    "fla_linear_attn_bwd_fused_dkdv": ([_ptr] * 7 + [_i64] * 5 + [_strides] * 7 + [ctypes.c_int, _ptr], ctypes.c_int),
    "fla_tri_xyt_z": ([_ptr] * 4 + [_i64] * 5 + [_strides] * 4 + [ctypes.c_int, ctypes.c_int, _ptr], ctypes.c_int),
    "fla_chunked_workspace_bytes": ([_i64] * 5, ctypes.c_int64),
    "fla_tri_xyt_z_chunked": ([_ptr] * 4 + [_i64] * 5 + [_strides] * 4 + [ctypes.c_int, ctypes.c_int, _ptr, _i64, _ptr],
                              ctypes.c_int),
    "fla_linear_attn_chunked_state_bytes": ([_i64] * 5, ctypes.c_int64),
    "fla_linear_attn_chunked_workspace_bytes": ([_i64] * 5, ctypes.c_int64),
    "fla_linear_attn_prefers_chunked": ([_i64] * 5, ctypes.c_int),
    "fla_linear_attn_chunked_fwd": ([_ptr] * 4 + [_i64] * 5 + [_strides] * 4
                                    + [ctypes.c_int, _ptr, ctypes.POINTER(ctypes.c_int32), _ptr, _i64, _ptr], ctypes.c_int),
    "fla_feature_attn_fwd": ([_ptr] * 6 + [_i64] * 5 + [_strides] * 6
                             + [ctypes.c_int, ctypes.c_int, _ptr, ctypes.POINTER(ctypes.c_int32), _ptr, _i64, _ptr], ctypes.c_int),
    "fla_feature_attn_bwd": ([_ptr] * 7 + [_i64] * 5 + [_strides] * 7 + [ctypes.c_int, ctypes.c_int, _ptr, _ptr, _i64, _ptr],
                             ctypes.c_int),
    "fla_feature_attn_normalised_fwd": ([_ptr] * 7 + [_i64] * 5 + [_strides] * 6
                                        + [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_int, _ptr,
                                           ctypes.POINTER(ctypes.c_int32), _ptr, _i64, _ptr],
                                        ctypes.c_int),
    "fla_feature_attn_normalised_bwd": ([_ptr] * 9 + [_i64] * 5 + [_strides] * 8
                                        + [ctypes.c_int, ctypes.c_int, ctypes.c_int, _ptr, _ptr, _i64, _ptr], ctypes.c_int),
    "fla_linear_attn_chunked_fwd_static": ([_ptr] * 4 + [_i64] * 5 + [_strides] * 4 + [ctypes.c_int, _ptr], ctypes.c_int),
    "fla_linear_attn_chunked_bwd": ([_ptr] * 7 + [_i64] * 5 + [_strides] * 7 + [ctypes.c_int, _ptr, _ptr, _i64, _ptr],
                                    ctypes.c_int),
    "fla_poly_attn_workspace_bytes": ([_i64] * 5, ctypes.c_int64),
    "fla_poly_attn_fwd": ([_ptr] * 5 + [_i64] * 5 + [_strides] * 4
                          + [ctypes.POINTER(ctypes.c_float), ctypes.c_float, ctypes.c_int, _ptr], ctypes.c_int),
    "fla_poly_attn_bwd": ([_ptr] * 9 + [_i64] * 5 + [_strides] * 8
                          + [ctypes.POINTER(ctypes.c_float), ctypes.c_int, _ptr, _i64, _ptr], ctypes.c_int),
    "fla_normalised_workspace_bytes": ([_i64] * 5 + [ctypes.c_int], ctypes.c_int64),
    "fla_linear_attn_normalised_fwd": ([_ptr] * 5 + [_i64] * 5 + [_strides] * 4
                                       + [ctypes.c_float, ctypes.c_int, ctypes.c_int, _ptr, ctypes.POINTER(ctypes.c_int32),
                                          _ptr, _i64, _ptr], ctypes.c_int),
    "fla_linear_attn_normalised_bwd": ([_ptr] * 9 + [_i64] * 5 + [_strides] * 8
                                       + [ctypes.c_int, ctypes.c_int, _ptr, _ptr, _i64, _ptr], ctypes.c_int),
}

_lock = threading.Lock()
_lib = None


class FlaError(RuntimeError):
    """A call into libfla_gfx950.so returned a negative status."""

    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


def load() -> ctypes.CDLL:
    """Load the library once; raise if it is absent or has the wrong ABI."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m flashy_linear_attention_amd.build` "
                "(there is no non-HIP fallback)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = restype
        got = lib.fla_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI version {got}, this package expects {ABI_VERSION}")
        _lib = lib
    return _lib


_STRIDES = {}


def strides_arg(t) -> ctypes.Array:
    """A tensor's 4 element strides as a C ``int64_t[4]``.  The arrays are read-only to the library
    and kept per distinct stride tuple: building one costs about as much as the rest of a call's
    argument conversion, and a caller's tensors come in a handful of layouts."""
    s = t.stride()
    a = _STRIDES.get(s)
    if a is None:
        if len(_STRIDES) > 4096:
            _STRIDES.clear()
        a = _STRIDES[s] = (ctypes.c_int64 * 4)(*s)
    return a


_SIZES = {}


def query(name: str, *args) -> int:
    """A size or plan query of the library (``fla_*_bytes``, ``fla_linear_attn_prefers_chunked``): pure
    host arithmetic on the shape, so the answer is kept per (function, arguments) -- an operator call
    makes two or three of them, each the cost of a ctypes call."""
    key = (name,) + args
    v = _SIZES.get(key)
    if v is None:
        if len(_SIZES) > 65536:
            _SIZES.clear()
        v = _SIZES[key] = getattr(load(), name)(*args)
    return v


def check(fn: str, status: int) -> None:
    if status != 0:
        raise FlaError(fn, status, load().fla_strerror(status).decode())
