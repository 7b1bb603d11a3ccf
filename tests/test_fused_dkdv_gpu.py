"""The backward with dV and dK formed by one kernel from one stream of (Q, dO) tiles
(fla_linear_attn_bwd_fused_dkdv; the loop structure of the reference's backward kernel,
flashlinear/kernels/linear_attn_kernels.py:160-227) against the CPU oracle and against the library's
own three-product backward (``-m gpu``).

Tolerance against the fp32 oracle: Frobenius-relative and max-abs/max both <= 1e-2 (the reference's
criterion, flashlinear/test_attn.py:17,24-25).  Against the three-product backward: bit-identical up
to padded head dim 64 (same tiles, same order of sums); at 128 the fused kernel's row tiles are half
as tall, the fp32 sums run in another order, and the two agree to 1e-4 Frobenius-relative.
"""

import ctypes

import pytest
import torch

from flashy_linear_attention_amd import _lib
from flashy_linear_attention_amd.kernels import linear_flash_wrapper_bwd
from flashy_linear_attention_amd.kernels.linear_attn_kernels import linear_flash_wrapper_bwd_fused_dkdv
from oracle import naive

from helpers import assert_close, reference_style_inputs, rel_fro

pytestmark = pytest.mark.gpu

# (batch, heads, seq, d_qk, d_v): one tile, tile pairs and single tiles, ragged lengths, widths below the
# padded width, unequal widths within one padded width, many heads, every padded width
CASES = [
    (1, 2, 64, 64, 64),
    (1, 2, 256, 64, 64),
    (2, 3, 320, 64, 64),
    (1, 16, 2048, 64, 64),
    (1, 5, 1000, 48, 64),
    (2, 2, 1984, 32, 32),
    (1, 130, 300, 24, 32),
    (1, 2, 4160, 40, 56),
    (1, 300, 512, 64, 64),
    (1, 2, 128, 128, 128),
    (2, 3, 1000, 128, 128),
    (1, 130, 384, 96, 128),
    (1, 2, 4160, 128, 72),
    (3, 3, 1984, 128, 128),
]


def _raw(fn_name, dy, q, k, v):
    """through the C ABI (any length; the Python wrappers of the reference-named functions keep its N % 64 rule)"""
    lib = _lib.load()
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    dq, dk, dvv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    rc = getattr(lib, fn_name)(dy.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                               dvv.data_ptr(), b, h, n, dqk, dv, *(_lib.strides_arg(t) for t in (dy, q, k, v, dq, dk, dvv)),
                               0 if q.dtype == torch.bfloat16 else 1,
                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.fla_strerror(rc)
    return dq, dk, dvv


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dims", CASES, ids=lambda d: "x".join(map(str, d)))
def test_fused_dkdv_backward(dims, dtype, gpu_device):
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(*dims, dtype, seed=sum(dims)))
    got = _raw("fla_linear_attn_bwd_fused_dkdv", dy, q, k, v)
    plain = _raw("fla_linear_attn_smallv_bwd", dy, q, k, v)
    torch.cuda.synchronize()
    same_order = max(dims[3], dims[4]) <= 64
    for name, g, p in zip(("dQ", "dK", "dV"), got, plain):
        if same_order or name == "dQ":
            assert torch.equal(g, p), f"{name}: differs from the three-product backward"
        else:
            assert rel_fro(g, p) <= 1e-4, f"{name}: {rel_fro(g, p):.2e} from the three-product backward"
    if dims[0] * dims[1] * dims[2] <= 40000:
        want = naive.causal_dot_product_grads(q.float().cpu(), k.float().cpu(), v.float().cpu(), dy.float().cpu())
        for name, g, w in zip(("dQ", "dK", "dV"), got, want):
            assert_close(name, g, w)


def test_fused_dkdv_wrapper_and_limits(gpu_device):
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(2, 4, 512, 64, 64, torch.bfloat16, seed=5))
    got = linear_flash_wrapper_bwd_fused_dkdv(dy, q, k, v)
    want = linear_flash_wrapper_bwd(dy, q, k, v)
    for g, w in zip(got, want):
        assert g.is_contiguous() and torch.equal(g, w)
    lib = _lib.load()
    # unequal padded widths, widths above 128 and rows that are not 16-byte aligned have no fused kernel
    for dqk, dv, row in ((128, 64, None), (256, 256, None), (64, 64, 65)):
        n = 128
        qq = torch.zeros(1, 1, n, row or dqk, dtype=torch.bfloat16, device=gpu_device)[..., :dqk]
        vv = torch.zeros(1, 1, n, row or dv, dtype=torch.bfloat16, device=gpu_device)[..., :dv]
        outs = [torch.empty(1, 1, n, w, dtype=torch.bfloat16, device=gpu_device) for w in (dqk, dqk, dv)]
        rc = lib.fla_linear_attn_bwd_fused_dkdv(vv.data_ptr(), qq.data_ptr(), qq.data_ptr(), vv.data_ptr(),
                                                *(t.data_ptr() for t in outs), 1, 1, n, dqk, dv,
                                                *(_lib.strides_arg(t) for t in (vv, qq, qq, vv, *outs)), 0,
                                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == -8, (dqk, dv, row, rc)  # FLA_ERR_UNSUPPORTED
    torch.cuda.synchronize()
