"""Chunk-wise evaluation of causal linear attention (an extension: the reference has only
the quadratic kernels, flashlinear/kernels/linear_attn_kernels.py:63,166-171).

``LinearAttentionChunked.apply(q, k, v)`` computes the same ``O = tril(Q K^T) V`` and the same
gradients as ``LinearAttention`` / ``LinearAttentionSmallVHD``, but through per-chunk KV states
(``fla_tri_xyt_z_chunked``): O(N) instead of O(N^2) work, meant for long sequences.  Results
agree with the quadratic path up to rounding (the running state is rounded once to the storage
dtype before it multiplies the queries).
"""

from __future__ import annotations

from typing import Any, Tuple

import torch
from torch.autograd import Function

from . import _lib
from .kernels._common import dtype_code, prepare, stream_handle


def tri_xyt_z_chunked(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor, upper: bool) -> torch.Tensor:
    """``mask(X Y^T) Z`` for (B, H, N, D_c) x, y and (B, H, N, D_o) z, evaluated chunk-wise."""
    assert x.shape == y.shape and z.shape[:3] == x.shape[:3], "x, y: (B,H,N,Dc); z: (B,H,N,Do)"
    x, y, z = prepare(x, y, z)
    b, h, n, dc = x.shape
    do = z.shape[-1]
    out = torch.empty_like(z, memory_format=torch.contiguous_format)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        nbytes = lib.fla_chunked_workspace_bytes(b, h, n, dc, do)
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


def linear_attention_chunked_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    assert q.shape[-1] <= 256 and v.shape[-1] <= 256, "Only head_dims <= 256 are supported."
    return tri_xyt_z_chunked(q, k, v, upper=False)


def linear_attention_chunked_bwd(
    grad_output: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    dq = tri_xyt_z_chunked(grad_output, v, k, upper=False)   # lower(dO V^T) K
    dv = tri_xyt_z_chunked(k, q, grad_output, upper=True)    # upper(K Q^T) dO
    dk = tri_xyt_z_chunked(v, grad_output, q, upper=True)    # upper(V dO^T) Q
    return dq, dk, dv


class LinearAttentionChunked(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        out = linear_attention_chunked_fwd(q, k, v)
        ctx.save_for_backward(q, k, v)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        q, k, v = ctx.saved_tensors
        return linear_attention_chunked_bwd(grad_output, q, k, v)
