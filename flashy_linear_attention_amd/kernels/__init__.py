from .linear_attn_kernels import linear_flash_wrapper_bwd, linear_flash_wrapper_fwd
from .linear_attn_kernels_smallv_hd import (
    linear_flash_wrapper_bwd_smallv_hd,
    linear_flash_wrapper_fwd_smallv_hd,
)
