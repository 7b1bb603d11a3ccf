"""``LinearAttentionAuto``: the reference's operator with the evaluation chosen by shape.

``LinearAttentionAuto.apply(q, k, v)`` takes the arguments of both ``LinearAttention`` and
``LinearAttentionSmallVHD`` (flashlinear/linear_attn.py:11-31, linear_attn_smallv_hd.py:14-36) and
returns the same ``tril(Q K^T) V``; it runs the quadratic kernels where they are faster (short
sequences, few heads) and the chunk-wise ones elsewhere, by the library's table of measured
thresholds (``fla_linear_attn_prefers_chunked``) -- the reference lists autotuning as a to-do
(README.md:68).  The two reference-named Functions keep the quadratic kernels whatever the shape.
"""

from __future__ import annotations

from typing import Any, Tuple

import torch
from torch.autograd import Function

from . import _lib
from .chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd
from .kernels import (
    linear_flash_wrapper_bwd,
    linear_flash_wrapper_bwd_smallv_hd,
    linear_flash_wrapper_fwd,
    linear_flash_wrapper_fwd_smallv_hd,
)


def prefers_chunked(q: torch.Tensor, v: torch.Tensor) -> bool:
    """Whether the chunk-wise kernels are the faster choice for (B, H, N, D_qk) q and (B, H, N, D_v) v."""
    b, h, n, dqk = q.shape
    return bool(_lib.query("fla_linear_attn_prefers_chunked", b, h, n, dqk, v.shape[-1]))


class LinearAttentionAuto(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        assert q.dim() == 4 and q.shape == k.shape and v.shape[:3] == q.shape[:3], "q, k: (B,H,N,D_qk); v: (B,H,N,D_v)"
        # (the quadratic wrappers keep the reference's limits: N a multiple of 64 and, with unequal head dims,
        # D_v a power of two not above D_qk -- what they refuse goes to the chunk-wise kernels)
        dqk, dv = q.shape[-1], v.shape[-1]
        ctx.equal = dqk == dv
        refused = q.shape[2] % 64 != 0 or (not ctx.equal and (dv > dqk or dv & (dv - 1)))
        ctx.chunked = prefers_chunked(q, v) or refused
        state = None
        if ctx.chunked:
            if any(ctx.needs_input_grad[:3]):
                out, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
            else:
                out = linear_attention_chunked_fwd(q, k, v)
        else:
            out = linear_flash_wrapper_fwd(q, k, v) if ctx.equal else linear_flash_wrapper_fwd_smallv_hd(q, k, v)
        ctx.has_state = state is not None
        ctx.save_for_backward(*((q, k, v, state) if state is not None else (q, k, v)))
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        if ctx.has_state:
            q, k, v, state = ctx.saved_tensors
        else:
            (q, k, v), state = ctx.saved_tensors, None
        if ctx.chunked:
            return linear_attention_chunked_bwd(grad_output, q, k, v, state)
        if ctx.equal:
            return linear_flash_wrapper_bwd(grad_output, q, k, v)
        return linear_flash_wrapper_bwd_smallv_hd(grad_output, q, k, v)
