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
    # (get_device() is the device index, -1 on the CPU: an integer comparison per tensor where comparing
    # torch.device objects costs several times as much)
    index, dtype = first.get_device(), first.dtype
    dense = True
    for t in tensors:
        if t.dim() != 4:
            raise ValueError(f"expected (batch, heads, seq, head_dim) tensors, got shape {tuple(t.shape)}")
        if t.get_device() != index:
            raise RuntimeError("all tensors must be on the same device")
        if t.dtype != dtype:
            raise TypeError(f"all tensors must share one dtype, got {dtype} and {t.dtype}")
        dense = dense and t.stride(3) == 1
    if dense:  # (the usual case: nothing to copy, the caller's tuple goes back as it came)
        return tensors
    return tuple(t.contiguous() if (t.stride(3) != 1 and t.shape[3] > 1) else t for t in tensors)


try:  # the current stream's handle as a plain integer, without building a torch.cuda.Stream object
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:  # pragma: no cover - older or differently built torch
    _raw_stream = None


def stream_handle(device: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


try:  # the current device's index without the checks of torch.cuda.current_device (lazy initialisation, a Python frame)
    _current_device = torch._C._cuda_getDevice
except AttributeError:  # pragma: no cover - older or differently built torch
    _current_device = torch.cuda.current_device


def device_guard(device: torch.device):
    """Context that makes `device` the current one for the call into the library (which launches on
    the current device).  When it already is -- the usual case -- nothing is switched: entering and
    leaving torch.cuda.device costs two device exchanges per call.  (The callers hold a tensor on
    `device`, so the GPU runtime is initialised.)"""
    index = device.index
    if index is None or index == _current_device():
        return _NO_GUARD
    return torch.cuda.device(device)


_FUNCS = {}


def call(name: str, *args) -> None:
    fn = _FUNCS.get(name)
    if fn is None:
        fn = _FUNCS[name] = getattr(_lib.load(), name)
    status = fn(*args)
    if status != 0:
        _lib.check(name, status)
