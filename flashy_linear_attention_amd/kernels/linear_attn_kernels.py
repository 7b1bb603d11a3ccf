"""Launch wrappers for causal linear attention with equal head dims.

Same names, arguments and assertions as the reference's Triton launch wrappers
(flashlinear/kernels/linear_attn_kernels.py:310-384); the work is done by
``fla_linear_attn_fwd`` / ``fla_linear_attn_bwd`` in ``libfla_gfx950.so``.
Differences kept on purpose: every tensor's own strides are passed (the
reference reuses q's strides for all of them, linear_attn_kernels.py:335,378),
fp16 inputs run on fp16 MFMA (the reference hard-codes bf16,
linear_attn_kernels.py:82,98), and dQ is not pre-zeroed.
"""

from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib
from ._common import call, device_guard, dtype_code, next_power_of_2, prepare, stream_handle


def _block_sq(hd: int) -> int:
    return 64 if next_power_of_2(hd) <= 128 else 32


def linear_flash_wrapper_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """O = tril(Q K^T) V for (batch, heads, seq, head_dim) tensors."""
    batch, nh, sq, hd = q.shape
    BLOCK_SQ = _block_sq(hd)

    assert hd <= 256, "Only head_dims <= 256 are supported."
    assert sq % BLOCK_SQ == 0, f"Number of elements in sequence must be a multiple of {BLOCK_SQ}, {sq, BLOCK_SQ}"
    assert k.shape == q.shape and v.shape == q.shape, "q, k and v must have the same shape"

    q, k, v = prepare(q, k, v)
    out = torch.empty_like(q, memory_format=torch.contiguous_format)
    with device_guard(q.device):
        call(
            "fla_linear_attn_fwd",
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
            batch, nh, sq, hd,
            _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v), _lib.strides_arg(out),
            dtype_code(q), stream_handle(q.device),
        )
    return out


def linear_flash_wrapper_bwd(
    grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) of :func:`linear_flash_wrapper_fwd` for upstream gradient ``grad_output``."""
    batch, nh, sq, hd = q.shape
    BLOCK_SQ = _block_sq(hd)

    assert hd <= 256, "Only head_dims <= 256 are supported."
    assert sq % BLOCK_SQ == 0, f"Number of elements in sequence must be a multiple of {BLOCK_SQ}"
    assert k.shape == q.shape and v.shape == q.shape and grad_output.shape == q.shape, \
        "grad_output, q, k and v must have the same shape"

    grad_output, q, k, v = prepare(grad_output, q, k, v)
    dQ = torch.empty_like(q, memory_format=torch.contiguous_format)
    dK = torch.empty_like(k, memory_format=torch.contiguous_format)
    dV = torch.empty_like(v, memory_format=torch.contiguous_format)
    with device_guard(q.device):
        call(
            "fla_linear_attn_bwd",
            grad_output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(),
            batch, nh, sq, hd,
            _lib.strides_arg(grad_output), _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v),
            _lib.strides_arg(dQ), _lib.strides_arg(dK), _lib.strides_arg(dV),
            dtype_code(q), stream_handle(q.device),
        )
    return dQ, dK, dV


def linear_flash_wrapper_bwd_fused_dkdv(
    grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) like :func:`linear_flash_wrapper_bwd`, with dV and dK formed by one kernel from one
    stream of (Q, dO) tiles -- the loop structure of the reference's backward kernel
    (flashlinear/kernels/linear_attn_kernels.py:160-227).  Head dims up to 128 (q/k and v may differ
    within one padded width).  Measured slower than :func:`linear_flash_wrapper_bwd` on MI355X; kept
    as the measured alternative (``fla_linear_attn_bwd_fused_dkdv``)."""
    batch, nh, sq, hd = q.shape
    hd_v = v.shape[-1]
    assert hd <= 128 and hd_v <= 128, "Only head_dims <= 128 are supported by the fused dK / dV kernel."
    assert k.shape == q.shape and v.shape[:3] == q.shape[:3] and grad_output.shape == v.shape, \
        "grad_output must match v; q, k, v must agree in batch, heads and sequence"
    grad_output, q, k, v = prepare(grad_output, q, k, v)
    dQ = torch.empty_like(q, memory_format=torch.contiguous_format)
    dK = torch.empty_like(k, memory_format=torch.contiguous_format)
    dV = torch.empty_like(v, memory_format=torch.contiguous_format)
    with device_guard(q.device):
        call(
            "fla_linear_attn_bwd_fused_dkdv",
            grad_output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(),
            batch, nh, sq, hd, hd_v,
            _lib.strides_arg(grad_output), _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v),
            _lib.strides_arg(dQ), _lib.strides_arg(dK), _lib.strides_arg(dV),
            dtype_code(q), stream_handle(q.device),
        )
    return dQ, dK, dV
