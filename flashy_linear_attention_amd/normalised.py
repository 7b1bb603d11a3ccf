"""Normalised causal linear attention as one operator (an extension: the reference leaves the
normaliser to the caller, README.md:27-30 of the reference):

    out = LinearAttention.apply(q, k, v) / ((q * k.cumsum(-2)).sum(-1, keepdim=True) + eps)

``LinearAttentionNormalised.apply(q, k, v, eps, chunked=False)`` returns the same tensor
(``chunked=True``: the product is evaluated chunk-wise, O(N), for long sequences).  The product runs on
the kernels of ``LinearAttention``; the cumulative sum, the dot with q, eps and the division
are one fused pass in fp32 (``fla_linear_attn_normalised_fwd``), and backward adds the
normaliser's own gradient terms with two more fused passes instead of an autograd graph of
elementwise kernels (``fla_linear_attn_normalised_bwd``).
"""

from __future__ import annotations

from typing import Any, Tuple

import ctypes

import torch
from torch.autograd import Function

from . import _lib
from .kernels._common import device_guard, dtype_code, prepare, stream_handle


def _workspace(lib, b: int, h: int, n: int, dqk: int, dv: int, chunked: bool,
               device: torch.device) -> Tuple[torch.Tensor, int]:
    nbytes = _lib.query("fla_normalised_workspace_bytes", b, h, n, dqk, dv, int(chunked))
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device), nbytes


def _state_buffer(lib, b: int, h: int, n: int, dqk: int, dv: int, want: bool, device: torch.device):
    sbytes = _lib.query("fla_linear_attn_chunked_state_bytes", b, h, n, dqk, dv) if want else 0
    return torch.empty(sbytes, dtype=torch.uint8, device=device) if sbytes else None


def linear_attention_normalised_fwd(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, eps: float = 1e-5, chunked: bool = False,
    want_state: bool = False,
):
    """(out, denom): the normalised output in the dtype of q and the fp32 normaliser (B, H, N).
    ``chunked`` evaluates the product chunk-wise (O(N)) instead of with the quadratic kernels; with
    ``want_state`` the result is (out, denom, state), ``state`` being what the chunk-wise forward
    hands to :func:`linear_attention_normalised_bwd` (None when the shape has none)."""
    assert q.shape == k.shape and v.shape[:3] == q.shape[:3], "q, k: (B,H,N,D_qk); v: (B,H,N,D_v)"
    assert q.shape[-1] <= 256 and v.shape[-1] <= 256, "Only head_dims <= 256 are supported."
    q, k, v = prepare(q, k, v)
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    out = torch.empty_like(v, memory_format=torch.contiguous_format)
    denom = torch.empty(b, h, n, dtype=torch.float32, device=q.device)
    lib = _lib.load()
    with device_guard(q.device):
        work, nbytes = _workspace(lib, b, h, n, dqk, dv, chunked, q.device)
        state = _state_buffer(lib, b, h, n, dqk, dv, want_state and chunked, q.device)
        valid = ctypes.c_int32(0)
        _lib.check(
            "fla_linear_attn_normalised_fwd",
            lib.fla_linear_attn_normalised_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), denom.data_ptr(), b, h, n, dqk, dv,
                _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v), _lib.strides_arg(out),
                float(eps), dtype_code(q), int(chunked), state.data_ptr() if state is not None else None,
                ctypes.byref(valid), work.data_ptr(), nbytes, stream_handle(q.device),
            ),
        )
    if want_state:
        return out, denom, (state if valid.value else None)
    return out, denom


def linear_attention_normalised_bwd(
    grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
    denom: torch.Tensor, chunked: bool = False, state: torch.Tensor = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv) for d(out) = grad_output, given forward's ``out`` and ``denom`` (and ``state``, if
    the forward call returned one)."""
    grad_output, q, k, v, out = prepare(grad_output, q, k, v, out)
    assert denom.dtype == torch.float32 and denom.is_contiguous() and denom.shape == q.shape[:3]
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    dq = torch.empty_like(q, memory_format=torch.contiguous_format)
    dk = torch.empty_like(k, memory_format=torch.contiguous_format)
    dvv = torch.empty_like(v, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with device_guard(q.device):
        work, nbytes = _workspace(lib, b, h, n, dqk, dv, chunked, q.device)
        _lib.check(
            "fla_linear_attn_normalised_bwd",
            lib.fla_linear_attn_normalised_bwd(
                grad_output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), denom.data_ptr(),
                dq.data_ptr(), dk.data_ptr(), dvv.data_ptr(), b, h, n, dqk, dv,
                _lib.strides_arg(grad_output), _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v),
                _lib.strides_arg(out), _lib.strides_arg(dq), _lib.strides_arg(dk), _lib.strides_arg(dvv),
                dtype_code(q), int(chunked), state.data_ptr() if state is not None else None, work.data_ptr(), nbytes,
                stream_handle(q.device),
            ),
        )
    return dq, dk, dvv


class LinearAttentionNormalised(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, eps: float = 1e-5,
                chunked: bool = False) -> torch.Tensor:
        want = bool(chunked) and any(ctx.needs_input_grad[:3])
        out, denom, state = linear_attention_normalised_fwd(q, k, v, eps, chunked, want_state=True) if want else (
            *linear_attention_normalised_fwd(q, k, v, eps, chunked), None)
        ctx.has_state = state is not None
        ctx.save_for_backward(*((q, k, v, out, denom) + ((state,) if state is not None else ())))
        ctx.chunked = chunked
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor):
        q, k, v, out, denom = ctx.saved_tensors[:5]
        state = ctx.saved_tensors[5] if ctx.has_state else None
        dq, dk, dv = linear_attention_normalised_bwd(grad_output, q, k, v, out, denom, ctx.chunked, state)
        return dq, dk, dv, None, None
