"""Causal linear attention with the feature map inside the operator (an extension: callers of the
reference apply the map in PyTorch before ``LinearAttention.apply``, README.md:27-30 and
flashlinear/test_attn.py:36-40 of the reference):

    FeatureMapLinearAttention.apply(xq, xk, v, "elu1")   ==   LinearAttention.apply(elu(xq) + 1, elu(xk) + 1, v)

with ``"softplus"`` as the other map.  The product is evaluated chunk-wise
(``LinearAttentionChunked``'s method) and the map is applied while the kernels load xq and xk:
no pass over memory exists for the map alone.  The kernels leave phi(xq), phi(xk) behind as a
by-product; autograd keeps those instead of xq, xk, and backward returns the gradients with
respect to xq and xk themselves, the slope of phi multiplied in before the gradients are stored
(``fla_feature_attn_fwd`` / ``fla_feature_attn_bwd``).

``FeatureMapLinearAttention.apply(xq, xk, v, feature, True, eps)`` is the normalised operator on
the same features, ``LinearAttentionNormalised.apply(phi(xq), phi(xk), v, eps, True)``
(``fla_feature_attn_normalised_fwd`` / ``_bwd``); a seventh argument ``chunked=False`` selects the
quadratic product kernels there.
"""

from __future__ import annotations

import ctypes
from typing import Any, Optional, Tuple

import torch
from torch.autograd import Function

from . import _lib
from .kernels._common import device_guard, dtype_code, prepare, stream_handle

FEATURE_MAPS = {"elu1": 1, "softplus": 2}  # enum fla_feature_map


def _map_code(feature: str) -> int:
    try:
        return FEATURE_MAPS[feature]
    except KeyError:
        raise ValueError(f"feature map must be one of {sorted(FEATURE_MAPS)}, got {feature!r}") from None


def feature_attention_fwd(xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, feature: str = "elu1",
                          want_state: bool = False):
    """``(O, q, k)`` with ``O = tril(q k^T) v``, ``q = phi(xq)``, ``k = phi(xk)``.  With ``want_state``
    returns ``(O, q, k, state)``, ``state`` being the running state for :func:`feature_attention_bwd`
    (None when the shape does not allow sharing it)."""
    assert xq.shape == xk.shape and v.shape[:3] == xq.shape[:3], "xq, xk: (B,H,N,D_qk); v: (B,H,N,D_v)"
    assert xq.shape[-1] <= 256 and v.shape[-1] <= 256, "Only head_dims <= 256 are supported."
    code = _map_code(feature)
    xq, xk, v = prepare(xq, xk, v)
    b, h, n, dqk = xq.shape
    dv = v.shape[-1]
    out = torch.empty_like(v, memory_format=torch.contiguous_format)
    q = torch.empty_like(xq, memory_format=torch.contiguous_format)
    k = torch.empty_like(xk, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(xq.device):
        sbytes = _lib.query("fla_linear_attn_chunked_state_bytes", b, h, n, dqk, dv) if want_state else 0
        state = torch.empty(sbytes, dtype=torch.uint8, device=xq.device) if sbytes else None
        wbytes = _lib.query("fla_linear_attn_chunked_workspace_bytes", b, h, n, dqk, dv)
        work = torch.empty(max(wbytes, 16), dtype=torch.uint8, device=xq.device)
        valid = ctypes.c_int32(0)
        _lib.check(
            "fla_feature_attn_fwd",
            lib.fla_feature_attn_fwd(
                xq.data_ptr(), xk.data_ptr(), v.data_ptr(), out.data_ptr(), q.data_ptr(), k.data_ptr(),
                b, h, n, dqk, dv,
                _lib.strides_arg(xq), _lib.strides_arg(xk), _lib.strides_arg(v), _lib.strides_arg(out),
                _lib.strides_arg(q), _lib.strides_arg(k),
                code, dtype_code(xq), state.data_ptr() if state is not None else None, ctypes.byref(valid),
                work.data_ptr(), wbytes, stream_handle(xq.device),
            ),
        )
    if want_state:
        return out, q, k, (state if valid.value else None)
    return out, q, k


def feature_attention_bwd(grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                          feature: str = "elu1", state: Optional[torch.Tensor] = None,
                          ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dxq, dxk, dv) from the forward call's ``q = phi(xq)``, ``k = phi(xk)`` and ``state`` (or None)."""
    code = _map_code(feature)
    grad_output, xq, xk, v = prepare(grad_output, q, k, v)
    b, h, n, dqk = xq.shape
    dv = v.shape[-1]
    dxq = torch.empty_like(xq, memory_format=torch.contiguous_format)
    dxk = torch.empty_like(xk, memory_format=torch.contiguous_format)
    dvv = torch.empty_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(xq.device):
        if state is not None:
            assert state.numel() == _lib.query("fla_linear_attn_chunked_state_bytes", b, h, n, dqk, dv), "state of another shape"
        wbytes = _lib.query("fla_linear_attn_chunked_workspace_bytes", b, h, n, dqk, dv)
        work = torch.empty(max(wbytes, 16), dtype=torch.uint8, device=xq.device)
        _lib.check(
            "fla_feature_attn_bwd",
            lib.fla_feature_attn_bwd(
                grad_output.data_ptr(), xq.data_ptr(), xk.data_ptr(), v.data_ptr(),
                dxq.data_ptr(), dxk.data_ptr(), dvv.data_ptr(), b, h, n, dqk, dv,
                _lib.strides_arg(grad_output), _lib.strides_arg(xq), _lib.strides_arg(xk), _lib.strides_arg(v),
                _lib.strides_arg(dxq), _lib.strides_arg(dxk), _lib.strides_arg(dvv),
                code, dtype_code(xq), state.data_ptr() if state is not None else None, work.data_ptr(), wbytes,
                stream_handle(xq.device),
            ),
        )
    return dxq, dxk, dvv


def feature_attention_normalised_fwd(xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, feature: str = "elu1",
                                     eps: float = 1e-5, chunked: bool = True, want_state: bool = False):
    """``(out, q, k, denom)``: the normalised output, ``q = phi(xq)``, ``k = phi(xk)`` and the fp32
    normaliser (B, H, N); with ``want_state`` also what the chunk-wise forward hands to backward (or None)."""
    assert xq.shape == xk.shape and v.shape[:3] == xq.shape[:3], "xq, xk: (B,H,N,D_qk); v: (B,H,N,D_v)"
    assert xq.shape[-1] <= 256 and v.shape[-1] <= 256, "Only head_dims <= 256 are supported."
    code = _map_code(feature)
    xq, xk, v = prepare(xq, xk, v)
    b, h, n, dqk = xq.shape
    dv = v.shape[-1]
    out = torch.empty_like(v, memory_format=torch.contiguous_format)
    q = torch.empty_like(xq, memory_format=torch.contiguous_format)
    k = torch.empty_like(xk, memory_format=torch.contiguous_format)
    denom = torch.empty(b, h, n, dtype=torch.float32, device=xq.device)
    lib = _lib.load()
    with device_guard(xq.device):
        nbytes = _lib.query("fla_normalised_workspace_bytes", b, h, n, dqk, dv, int(chunked))
        work = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=xq.device)
        sbytes = _lib.query("fla_linear_attn_chunked_state_bytes", b, h, n, dqk, dv) if (want_state and chunked) else 0
        state = torch.empty(sbytes, dtype=torch.uint8, device=xq.device) if sbytes else None
        valid = ctypes.c_int32(0)
        _lib.check(
            "fla_feature_attn_normalised_fwd",
            lib.fla_feature_attn_normalised_fwd(
                xq.data_ptr(), xk.data_ptr(), v.data_ptr(), out.data_ptr(), q.data_ptr(), k.data_ptr(), denom.data_ptr(),
                b, h, n, dqk, dv,
                _lib.strides_arg(xq), _lib.strides_arg(xk), _lib.strides_arg(v), _lib.strides_arg(out),
                _lib.strides_arg(q), _lib.strides_arg(k),
                code, float(eps), dtype_code(xq), int(chunked), state.data_ptr() if state is not None else None,
                ctypes.byref(valid), work.data_ptr(), nbytes, stream_handle(xq.device),
            ),
        )
    if want_state:
        return out, q, k, denom, (state if valid.value else None)
    return out, q, k, denom


def feature_attention_normalised_bwd(grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                     out: torch.Tensor, denom: torch.Tensor, feature: str = "elu1",
                                     chunked: bool = True,
                                     state: torch.Tensor = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dxq, dxk, dv) from the forward call's ``q``, ``k``, ``out`` and ``denom`` (and ``state``, if any)."""
    code = _map_code(feature)
    grad_output, q, k, v, out = prepare(grad_output, q, k, v, out)
    assert denom.dtype == torch.float32 and denom.is_contiguous() and denom.shape == q.shape[:3]
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    dxq = torch.empty_like(q, memory_format=torch.contiguous_format)
    dxk = torch.empty_like(k, memory_format=torch.contiguous_format)
    dvv = torch.empty_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(q.device):
        nbytes = _lib.query("fla_normalised_workspace_bytes", b, h, n, dqk, dv, int(chunked))
        work = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
        _lib.check(
            "fla_feature_attn_normalised_bwd",
            lib.fla_feature_attn_normalised_bwd(
                grad_output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), denom.data_ptr(),
                dxq.data_ptr(), dxk.data_ptr(), dvv.data_ptr(), b, h, n, dqk, dv,
                _lib.strides_arg(grad_output), _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v),
                _lib.strides_arg(out), _lib.strides_arg(dxq), _lib.strides_arg(dxk), _lib.strides_arg(dvv),
                code, dtype_code(q), int(chunked), state.data_ptr() if state is not None else None, work.data_ptr(),
                nbytes, stream_handle(q.device),
            ),
        )
    return dxq, dxk, dvv


class FeatureMapLinearAttention(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, xq: torch.Tensor, xk: torch.Tensor, v: torch.Tensor, feature: str = "elu1",
                normalise: bool = False, eps: float = 1e-5, chunked: bool = True) -> torch.Tensor:
        ctx.normalise = normalise
        if normalise:
            want = bool(chunked) and any(ctx.needs_input_grad[:3])
            out, q, k, denom, state = feature_attention_normalised_fwd(xq, xk, v, feature, eps, chunked, want_state=True) \
                if want else (*feature_attention_normalised_fwd(xq, xk, v, feature, eps, chunked), None)
            ctx.feature, ctx.chunked = feature, chunked
            ctx.has_state = state is not None
            ctx.save_for_backward(*((q, k, v, out, denom) + ((state,) if state is not None else ())))
            return out
        assert chunked, "without the normaliser the feature map exists for the chunk-wise product only"
        if any(ctx.needs_input_grad[:3]):
            out, q, k, state = feature_attention_fwd(xq, xk, v, feature, want_state=True)
        else:
            (out, q, k), state = feature_attention_fwd(xq, xk, v, feature), None
        ctx.feature = feature
        ctx.has_state = state is not None
        if state is not None:
            ctx.save_for_backward(q, k, v, state)
        else:
            ctx.save_for_backward(q, k, v)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor):
        if ctx.normalise:
            q, k, v, out, denom = ctx.saved_tensors[:5]
            state = ctx.saved_tensors[5] if ctx.has_state else None
            dxq, dxk, dv = feature_attention_normalised_bwd(grad_output, q, k, v, out, denom, ctx.feature, ctx.chunked,
                                                            state)
            return dxq, dxk, dv, None, None, None, None
        if ctx.has_state:
            q, k, v, state = ctx.saved_tensors
        else:
            (q, k, v), state = ctx.saved_tensors, None
        dxq, dxk, dv = feature_attention_bwd(grad_output, q, k, v, ctx.feature, state)
        return dxq, dxk, dv, None, None, None, None
