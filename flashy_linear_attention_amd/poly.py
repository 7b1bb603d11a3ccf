"""Causal linear attention with a polynomial score map (an extension: the reference multiplies
materialised features, flashlinear/kernels/linear_attn_kernels_smallv_hd.py:78-86).

``PolynomialLinearAttention.apply(xq, xk, v, c0, c1, c2, normalise=False, eps=1e-5)`` returns

    tril(f(xq xk^T)) v,    f(u) = c0 + c1 u + c2 u^2

(with ``normalise`` every row divided by the sum of its masked scores plus eps)
which is ``LinearAttentionSmallVHD`` on second-order Taylor features with
``phi(x) . phi(y) = f(x . y)`` -- ``(0, 0, 1/2)`` is the reference's ``flatten(x (x) x) / sqrt 2``
(256 features from a 16-wide x), ``(1, 1, 1/2)`` the full Taylor map of exp -- but the features
are never built: a score costs one 16-wide dot product instead of a 256-wide one, forward and
backward (``fla_poly_attn_fwd/bwd``).
"""

from __future__ import annotations

import ctypes
from typing import Any, Optional, Tuple

import torch
from torch.autograd import Function

from . import _lib
from .kernels._common import device_guard, dtype_code, prepare, stream_handle


def _coef(c0: float, c1: float, c2: float):
    return (ctypes.c_float * 3)(float(c0), float(c1), float(c2))


def _check(xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor) -> None:
    assert xq.shape == xk.shape and v.shape[:3] == xq.shape[:3], "xq, xk: (B,H,N,R); v: (B,H,N,D_v)"
    assert xq.shape[-1] <= 32 and xq.shape[-1] % 8 == 0, "R must be a multiple of 8 up to 32"
    assert v.shape[-1] <= 128 and v.shape[-1] % 8 == 0, "D_v must be a multiple of 8 up to 128"


def poly_attention_fwd(
    xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, coef: Tuple[float, float, float],
    normalise: bool = False, eps: float = 1e-5,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """(out, denom).  ``normalise`` divides every output row by the sum of its masked scores plus
    eps (the normaliser of linear attention with this kernel) and returns it as ``denom``."""
    _check(xq, xk, v)
    xq, xk, v = prepare(xq, xk, v)
    b, h, n, r = xq.shape
    dv = v.shape[-1]
    out = torch.empty_like(v, memory_format=torch.contiguous_format)
    denom = torch.empty(b, h, n, dtype=torch.float32, device=xq.device) if normalise else None
    lib = _lib.load()
    with device_guard(xq.device):
        _lib.check(
            "fla_poly_attn_fwd",
            lib.fla_poly_attn_fwd(
                xq.data_ptr(), xk.data_ptr(), v.data_ptr(), out.data_ptr(),
                denom.data_ptr() if denom is not None else None, b, h, n, r, dv,
                _lib.strides_arg(xq), _lib.strides_arg(xk), _lib.strides_arg(v), _lib.strides_arg(out),
                _coef(*coef), float(eps), dtype_code(xq), stream_handle(xq.device),
            ),
        )
    return out, denom


def poly_attention_bwd(
    grad_output: torch.Tensor, xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, coef: Tuple[float, float, float],
    out: Optional[torch.Tensor] = None, denom: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dXq, dXk, dV).  For the normalised forward pass its ``out`` and ``denom``."""
    _check(xq, xk, v)
    assert (out is None) == (denom is None)
    grad_output, xq, xk, v = prepare(grad_output, xq, xk, v)
    if out is not None:
        (out,) = prepare(out)
        assert denom.dtype == torch.float32 and denom.is_contiguous() and denom.shape == xq.shape[:3]
    b, h, n, r = xq.shape
    dv = v.shape[-1]
    dxq = torch.empty_like(xq, memory_format=torch.contiguous_format)
    dxk = torch.empty_like(xk, memory_format=torch.contiguous_format)
    dvv = torch.empty_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(xq.device):
        nbytes = _lib.query("fla_poly_attn_workspace_bytes", b, h, n, r, dv)
        work = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=xq.device)
        _lib.check(
            "fla_poly_attn_bwd",
            lib.fla_poly_attn_bwd(
                grad_output.data_ptr(), xq.data_ptr(), xk.data_ptr(), v.data_ptr(),
                out.data_ptr() if out is not None else None, denom.data_ptr() if denom is not None else None,
                dxq.data_ptr(), dxk.data_ptr(), dvv.data_ptr(), b, h, n, r, dv,
                _lib.strides_arg(grad_output), _lib.strides_arg(xq), _lib.strides_arg(xk), _lib.strides_arg(v),
                _lib.strides_arg(out) if out is not None else None,
                _lib.strides_arg(dxq), _lib.strides_arg(dxk), _lib.strides_arg(dvv),
                _coef(*coef), dtype_code(xq), work.data_ptr(), nbytes, stream_handle(xq.device),
            ),
        )
    return dxq, dxk, dvv


class PolynomialLinearAttention(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, c0: float = 0.0, c1: float = 0.0,
                c2: float = 0.5, normalise: bool = False, eps: float = 1e-5) -> torch.Tensor:
        out, denom = poly_attention_fwd(xq, xk, v, (c0, c1, c2), normalise, eps)
        if normalise:
            ctx.save_for_backward(xq, xk, v, out, denom)
        else:
            ctx.save_for_backward(xq, xk, v)
        ctx.coef = (c0, c1, c2)
        ctx.normalise = normalise
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor):
        if ctx.normalise:
            xq, xk, v, out, denom = ctx.saved_tensors
        else:
            (xq, xk, v), out, denom = ctx.saved_tensors, None, None
        dxq, dxk, dv = poly_attention_bwd(grad_output, xq, xk, v, ctx.coef, out, denom)
        return dxq, dxk, dv, None, None, None, None, None
