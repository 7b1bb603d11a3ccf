"""``LinearAttention``: un-normalised causal linear attention, O = tril(Q K^T) V.

Drop-in for the reference's autograd Function (flashlinear/linear_attn.py:11-31):
same ``apply(q, k, v)`` surface, same AMP behaviour (inputs are cast to bf16
under autocast), saves (q, k, v) for backward.  The denominator of full linear
attention stays with the caller in PyTorch (README.md:27-30).
"""

from typing import Any, Tuple

import torch
from torch.autograd import Function

from .kernels import linear_flash_wrapper_bwd, linear_flash_wrapper_fwd


class LinearAttention(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        out = linear_flash_wrapper_fwd(q, k, v)
        ctx.save_for_backward(q, k, v)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        query, key, value = ctx.saved_tensors
        gradq, gradk, gradv = linear_flash_wrapper_bwd(grad_output, query, key, value)
        return gradq, gradk, gradv
