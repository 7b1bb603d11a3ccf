"""Launch wrappers for causal linear attention whose query/key head dim is
larger than the value head dim.

Same names, arguments and assertions as the reference's wrappers
(flashlinear/kernels/linear_attn_kernels_smallv_hd.py:320-405); the work is done
by ``fla_linear_attn_smallv_fwd`` / ``fla_linear_attn_smallv_bwd``.
"""

from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib
from ._common import call, device_guard, dtype_code, next_power_of_2, prepare, stream_handle


def linear_flash_wrapper_fwd_smallv_hd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """O = tril(Q K^T) V with q, k of width hd_qk and v, O of width hd_v."""
    batch, nh, sq, hd_qk = q.shape
    batch, nh, sq, hd_v = v.shape

    BLOCK_HD = next_power_of_2(hd_qk)
    BLOCK_HD_V = next_power_of_2(hd_v)
    BLOCK_SQ = 64 if BLOCK_HD <= 128 else 32

    assert next_power_of_2(hd_v) == hd_v, "Expected value head dimension to be a power of 2."
    assert BLOCK_HD_V <= BLOCK_HD, "Value head dimension must be less than Query/Key head dimension."
    assert hd_qk <= 256, "Only head_dims <= 256 are supported."
    assert sq % BLOCK_SQ == 0, f"Number of elements in sequence must be a multiple of {BLOCK_SQ}, {sq, BLOCK_SQ}"
    assert k.shape == q.shape and v.shape[:3] == q.shape[:3], "q, k, v must agree in batch, heads and sequence"

    q, k, v = prepare(q, k, v)
    out = torch.empty_like(v, memory_format=torch.contiguous_format)
    with device_guard(q.device):
        call(
            "fla_linear_attn_smallv_fwd",
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
            batch, nh, sq, hd_qk, hd_v,
            _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v), _lib.strides_arg(out),
            dtype_code(q), stream_handle(q.device),
        )
    return out


def linear_flash_wrapper_bwd_smallv_hd(
    grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dQ, dK, dV) of :func:`linear_flash_wrapper_fwd_smallv_hd`."""
    batch, nh, sq, hd_qk = q.shape
    batch, nh, sq, hd_v = v.shape
    BLOCK_SQ = 64

    assert hd_qk <= 256, "Only head_dims <= 256 are supported."
    assert sq % BLOCK_SQ == 0, f"Number of elements in sequence must be a multiple of {BLOCK_SQ}"
    assert k.shape == q.shape and grad_output.shape == v.shape and v.shape[:3] == q.shape[:3], \
        "grad_output must match v; q, k, v must agree in batch, heads and sequence"

    grad_output, q, k, v = prepare(grad_output, q, k, v)
    dQ = torch.empty_like(q, memory_format=torch.contiguous_format)
    dK = torch.empty_like(k, memory_format=torch.contiguous_format)
    dV = torch.empty_like(v, memory_format=torch.contiguous_format)
    with device_guard(q.device):
        call(
            "fla_linear_attn_smallv_bwd",
            grad_output.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(),
            batch, nh, sq, hd_qk, hd_v,
            _lib.strides_arg(grad_output), _lib.strides_arg(q), _lib.strides_arg(k), _lib.strides_arg(v),
            _lib.strides_arg(dQ), _lib.strides_arg(dK), _lib.strides_arg(dV),
            dtype_code(q), stream_handle(q.device),
        )
    return dQ, dK, dV
