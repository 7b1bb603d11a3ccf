"""Chunk-wise evaluation of causal linear attention (an extension: the reference has only
the quadratic kernels, flashlinear/kernels/linear_attn_kernels.py:63,166-171).

``LinearAttentionChunked.apply(q, k, v)`` computes the same ``O = tril(Q K^T) V`` and the same
gradients as ``LinearAttention`` / ``LinearAttentionSmallVHD``, but through per-chunk KV states
(``fla_tri_xyt_z_chunked``): O(N) instead of O(N^2) work, meant for long sequences.  Results
agree with the quadratic path up to rounding (the running state is rounded once to the storage
dtype before it multiplies the queries).
"""

from __future__ import annotations

import ctypes
from typing import Any, Tuple

import torch
from torch.autograd import Function

from . import _lib
from .kernels._common import device_guard, dtype_code, prepare, stream_handle


def tri_xyt_z_chunked(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, upper: bool) -> torch.Tensor:
    """``mask(X Y^T) Z`` for (B, H, N, D_c) x, y and (B, H, N, D_o) z, evaluated chunk-wise."""
    assert x.shape == y.shape and z.shape[:3] == x.shape[:3], "x, y: (B,H,N,Dc); z: (B,H,N,Do)"
    x, y, z = prepare(x, y, z)
    b, h, n, dc = x.shape
    do = z.shape[-1]
    out = torch.empty_like(z, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(x.device):
        nbytes = _lib.query("fla_chunked_workspace_bytes", b, h, n, dc, do)
        work = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        _lib.check(
            "fla_tri_xyt_z_chunked",
            lib.fla_tri_xyt_z_chunked(
                x.data_ptr(), y.data_ptr(), z.data_ptr(), out.data_ptr(), b, h, n, dc, do,
                _lib.strides_arg(x), _lib.strides_arg(y), _lib.strides_arg(z), _lib.strides_arg(out),
                int(upper), dtype_code(x), work.data_ptr(), nbytes, stream_handle(x.device),
            ),
        )
    return out


def linear_attention_chunked_fwd(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, want_state: bool = False
):
    """``O = tril(Q K^T) V`` chunk-wise.  With ``want_state`` returns ``(O, state)`` where
    ``state`` is the running KV state for :func:`linear_attention_chunked_bwd` (None when the
    shape or layout does not allow sharing it)."""
    assert q.shape == k.shape and v.shape[:3] == q.shape[:3], "q, k: (B,H,N,D_qk); v: (B,H,N,D_v)"
    assert q.shape[-1] <= 256 and v.shape[-1] <= 256, "Only head_dims <= 256 are supported."
    q, k, v = prepare(q, k, v)
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    out = torch.empty_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(q.device):
        sbytes = _lib.query("fla_linear_attn_chunked_state_bytes", b, h, n, dqk, dv) if want_state else 0
        state = torch.empty(sbytes, dtype=torch.uint8, device=q.device) if sbytes else None
        wbytes = _lib.query("fla_linear_attn_chunked_workspace_bytes", b, h, n, dqk, dv)
        work = torch.empty(max(wbytes, 16), dtype=torch.uint8, device=q.device)
        valid = ctypes.c_int32(0)
        _lib.check(
            "fla_linear_attn_chunked_fwd",
            lib.fla_linear_attn_chunked_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b, h, n, dqk, dv,
                _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v), _lib.strides_arg(out),
                dtype_code(q), state.data_ptr() if state is not None else None, ctypes.byref(valid),
                work.data_ptr(), wbytes, stream_handle(q.device),
            ),
        )
    if want_state:
        return out, (state if valid.value else None)
    return out


def linear_attention_chunked_bwd(
    grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor = None
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) chunk-wise; ``state`` is what the forward call returned (or None)."""
    grad_output, q, k, v = prepare(grad_output, q, k, v)
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    dq = torch.empty_like(q, memory_format=torch.contiguous_format)
    dk = torch.empty_like(k, memory_format=torch.contiguous_format)
    dvv = torch.empty_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(q.device):
        if state is not None:
            assert state.numel() == _lib.query("fla_linear_attn_chunked_state_bytes", b, h, n, dqk, dv), "state of another shape"
        wbytes = _lib.query("fla_linear_attn_chunked_workspace_bytes", b, h, n, dqk, dv)
        work = torch.empty(max(wbytes, 16), dtype=torch.uint8, device=q.device)
        _lib.check(
            "fla_linear_attn_chunked_bwd",
            lib.fla_linear_attn_chunked_bwd(
                grad_output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                dq.data_ptr(), dk.data_ptr(), dvv.data_ptr(), b, h, n, dqk, dv,
                _lib.strides_arg(grad_output), _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v),
                _lib.strides_arg(dq), _lib.strides_arg(dk), _lib.strides_arg(dvv),
                dtype_code(q), state.data_ptr() if state is not None else None, work.data_ptr(), wbytes,
                stream_handle(q.device),
            ),
        )
    return dq, dk, dvv


class LinearAttentionChunked(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        if any(ctx.needs_input_grad[:3]):
            out, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
        else:
            out, state = linear_attention_chunked_fwd(q, k, v), None
        ctx.has_state = state is not None
        if state is not None:
            ctx.save_for_backward(q, k, v, state)
        else:
            ctx.save_for_backward(q, k, v)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        if ctx.has_state:
            q, k, v, state = ctx.saved_tensors
        else:
            (q, k, v), state = ctx.saved_tensors, None
        return linear_attention_chunked_bwd(grad_output, q, k, v, state)
