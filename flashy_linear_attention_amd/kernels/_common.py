"""Shared plumbing of the launch wrappers: argument normalisation and the call
into the C ABI.  PyTorch is used only for device memory and the stream."""

from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib

_DTYPES = {torch.bfloat16: _lib.FLA_DTYPE_BF16, torch.float16: _lib.FLA_DTYPE_F16}


def next_power_of_2(x: int) -> int:
    return 1 if x <= 1 else 1 << (x - 1).bit_length()


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"expected torch.bfloat16 or torch.float16 tensors, got {t.dtype}") from None


def prepare(*tensors: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """Check device/dtype agreement and make the innermost dimension dense."""
    first = tensors[0]
    if not first.is_cuda:
        raise RuntimeError("flashy_linear_attention_amd operators need tensors on a ROCm GPU (device 'cuda')")
    out = []
    for t in tensors:
        if t.dim() != 4:
            raise ValueError(f"expected (batch, heads, seq, head_dim) tensors, got shape {tuple(t.shape)}")
        if t.device != first.device:
            raise RuntimeError("all tensors must be on the same device")
        if t.dtype != first.dtype:
            raise TypeError(f"all tensors must share one dtype, got {first.dtype} and {t.dtype}")
        if t.stride(-1) != 1 and t.shape[-1] > 1:
            t = t.contiguous()
        out.append(t)
    return tuple(out)


def stream_handle(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def call(name: str, *args) -> None:
    _lib.check(name, getattr(_lib.load(), name)(*args))
