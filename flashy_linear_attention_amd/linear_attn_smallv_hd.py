"""``LinearAttentionSmallVHD``: causal linear attention whose query/key head dim
exceeds the value head dim (e.g. 256-wide Taylor features over 64-wide values).

Drop-in for the reference's autograd Function
(flashlinear/linear_attn_smallv_hd.py:14-36).
"""

from typing import Any, Tuple

import torch
from torch.autograd import Function

from .kernels import linear_flash_wrapper_bwd_smallv_hd, linear_flash_wrapper_fwd_smallv_hd


class LinearAttentionSmallVHD(Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx: Any, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        out = linear_flash_wrapper_fwd_smallv_hd(q, k, v)
        ctx.save_for_backward(q, k, v)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad_output: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        query, key, value = ctx.saved_tensors
        gradq, gradk, gradv = linear_flash_wrapper_bwd_smallv_hd(grad_output, query, key, value)
        return gradq, gradk, gradv
