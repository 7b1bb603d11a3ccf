"""Polynomial score map (fla_poly_attn_fwd/bwd, PolynomialLinearAttention) against the CPU
oracle and against LinearAttentionSmallVHD on the explicit Taylor features (``-m gpu``).

Tolerances as for the product kernels: Frobenius-relative and max-abs/max <= 1e-2 against the
fp32 oracle fed the rounded 16-bit inputs."""

import pytest
import torch

from flashy_linear_attention_amd import LinearAttentionSmallVHD, PolynomialLinearAttention, _lib
from flashy_linear_attention_amd.poly import poly_attention_bwd, poly_attention_fwd
from oracle import naive

from helpers import assert_close

pytestmark = pytest.mark.gpu

SQUARE = (0.0, 0.0, 0.5)   # flatten(x (x) x) / sqrt 2, the reference's small-V feature recipe
TAYLOR = (1.0, 1.0, 0.5)   # 1 + u + u^2 / 2

# (batch, heads, seq, r, d_v)
CASES = [
    (1, 2, 256, 16, 64),
    (2, 3, 1024, 16, 64),
    (1, 2, 576, 32, 128),
    (1, 2, 320, 8, 32),
    (1, 1, 1088, 24, 48),
    (1, 5, 200, 16, 16),
    (1, 2, 64, 16, 128),
]


def _inputs(dims, dtype, seed):
    b, h, n, r, dv = dims
    g = torch.Generator().manual_seed(seed)
    xq = 0.5 * torch.randn(b, h, n, r, generator=g)
    xk = 0.5 * torch.randn(b, h, n, r, generator=g)
    v = torch.randn(b, h, n, dv, generator=g)
    do = torch.randn(b, h, n, dv, generator=g)
    return tuple(t.to(dtype) for t in (xq, xk, v, do))


@pytest.mark.parametrize("coef", [SQUARE, TAYLOR], ids=["square", "taylor"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dims", CASES, ids=lambda d: "x".join(map(str, d)))
def test_poly_fwd_bwd_vs_oracle(dims, dtype, coef, gpu_device):
    xq, xk, v, do = _inputs(dims, dtype, seed=sum(dims))
    want_o = naive.poly_causal_dot_product(xq.float(), xk.float(), v.float(), coef)
    want_g = naive.poly_causal_dot_product_grads(xq.float(), xk.float(), v.float(), do.float(), coef)
    a, b, c = (t.to(gpu_device).requires_grad_(True) for t in (xq, xk, v))
    out = PolynomialLinearAttention.apply(a, b, c, *coef)
    assert out.dtype == dtype and out.shape == v.shape
    out.backward(do.to(gpu_device))
    assert_close("O", out, want_o)
    for name, got, want in (("dXq", a.grad, want_g[0]), ("dXk", b.grad, want_g[1]), ("dV", c.grad, want_g[2])):
        assert got.dtype == dtype and got.shape == want.shape
        assert_close(name, got, want)


def test_poly_equals_small_v_operator_on_explicit_features(gpu_device):
    """The reference's way (256 explicit features through LinearAttentionSmallVHD, gradients chained
    through the feature map by autograd) and the polynomial operator on the 16-wide x agree."""
    dims = (2, 4, 1024, 16, 64)
    xq, xk, v, do = (t.to(gpu_device) for t in _inputs(dims, torch.bfloat16, seed=9))
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    phi_q = naive.taylor2_features(a.float(), SQUARE).bfloat16()
    phi_k = naive.taylor2_features(b.float(), SQUARE).bfloat16()
    ref = LinearAttentionSmallVHD.apply(phi_q, phi_k, c)
    ref.backward(do)
    a2, b2, c2 = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    out = PolynomialLinearAttention.apply(a2, b2, c2, *SQUARE)
    out.backward(do)
    assert_close("O", out, ref.detach().float())
    for name, got, want in (("dXq", a2.grad, a.grad), ("dXk", b2.grad, b.grad), ("dV", c2.grad, c.grad)):
        assert_close(name, got, want.float(), tol_fro=1.5e-2, tol_max=2e-2)  # two 16-bit pipelines against each other


def test_poly_normalised_forward(gpu_device):
    """denom is the row sum of the masked scores plus eps, and out * denom the plain product."""
    dims = (1, 3, 768, 16, 64)
    xq, xk, v, _ = _inputs(dims, torch.bfloat16, seed=4)
    u = torch.matmul(xq.float(), xk.float().transpose(-2, -1))
    scores = (1.0 + u + 0.5 * u * u).tril()
    want_n = scores.sum(-1) + 1e-5
    want_o = torch.matmul(scores, v.float()) / want_n[..., None]
    out, denom = poly_attention_fwd(xq.to(gpu_device), xk.to(gpu_device), v.to(gpu_device), TAYLOR, normalise=True)
    assert_close("out", out, want_o)
    assert_close("denom", denom, want_n, tol_fro=1e-5, tol_max=1e-5)


# the bias column of the normalised backward: first operand fits half of the contraction
# (d_v + 8 <= 32, 64, 128 with the padded widths 64, 128, 256) or takes the tail layout
NORM_CASES = [
    (1, 2, 256, 16, 16),
    (2, 3, 1024, 16, 64),
    (1, 2, 576, 32, 128),
    (1, 2, 320, 8, 32),
    (1, 1, 1088, 24, 48),
    (1, 2, 200, 16, 96),
    (1, 2, 640, 16, 120),
    (1, 2, 64, 32, 24),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dims", NORM_CASES, ids=lambda d: "x".join(map(str, d)))
def test_poly_normalised_fwd_bwd_vs_oracle(dims, dtype, gpu_device):
    """Gradients through the normaliser.  Element bound 5e-2 of the largest magnitude as for the
    normalised linear operator: dO = g / n and the bias dn pass through 16-bit storage and the
    two terms of the score gradient cancel."""
    xq, xk, v, do = _inputs(dims, dtype, seed=sum(dims) + 2)
    a, b, c = (t.float().requires_grad_(True) for t in (xq, xk, v))
    want = naive.poly_linear_attention_normalised(a, b, c, TAYLOR, 1e-5)
    want.backward(do.float())
    ag, bg, cg = (t.to(gpu_device).requires_grad_(True) for t in (xq, xk, v))
    out = PolynomialLinearAttention.apply(ag, bg, cg, *TAYLOR, True, 1e-5)
    out.backward(do.to(gpu_device))
    assert_close("out", out, want.detach())
    for name, got, w in (("dXq", ag.grad, a.grad), ("dXk", bg.grad, b.grad), ("dV", cg.grad, c.grad)):
        assert got.dtype == dtype and got.shape == w.shape
        assert_close(name, got, w, tol_fro=1e-2, tol_max=5e-2)


def test_poly_normalised_equals_normalised_operator_on_explicit_features(gpu_device):
    """LinearAttentionNormalised on the 73 explicit Taylor features of an 8-wide x (padded to 80
    for the 16-byte rows) and the normalised polynomial operator on x itself."""
    from flashy_linear_attention_amd import LinearAttentionNormalised
    dims = (1, 2, 512, 8, 64)
    xq, xk, v, do = (t.to(gpu_device) for t in _inputs(dims, torch.bfloat16, seed=12))
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    pad = torch.nn.functional.pad
    phi_q = pad(naive.taylor2_features(a.float(), TAYLOR), (0, 7)).bfloat16()
    phi_k = pad(naive.taylor2_features(b.float(), TAYLOR), (0, 7)).bfloat16()
    ref = LinearAttentionNormalised.apply(phi_q, phi_k, c, 1e-5)
    ref.backward(do)
    a2, b2, c2 = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    out = PolynomialLinearAttention.apply(a2, b2, c2, *TAYLOR, True, 1e-5)
    out.backward(do)
    assert_close("out", out, ref.detach().float())
    for name, got, want in (("dXq", a2.grad, a.grad), ("dXk", b2.grad, b.grad), ("dV", c2.grad, c.grad)):
        assert_close(name, got, want.float(), tol_fro=2e-2, tol_max=5e-2)  # two 16-bit pipelines against each other


def test_poly_rejects_what_it_has_no_kernel_for(gpu_device):
    lib = _lib.load()
    xq, xk, v, do = (t.to(gpu_device) for t in _inputs((1, 1, 128, 16, 64), torch.bfloat16, seed=1))
    with pytest.raises(AssertionError):
        PolynomialLinearAttention.apply(xq[..., :12], xk[..., :12], v)          # R not a multiple of 8
    with pytest.raises(AssertionError):
        PolynomialLinearAttention.apply(torch.cat([xq] * 3, -1), torch.cat([xk] * 3, -1), v)   # R = 48 > 32
    assert lib.fla_poly_attn_workspace_bytes(1, 1, 128, 48, 64) == 0
    # both packed operands at the widest layout (96 + 32 columns with the bias), dO = g / n, dn
    assert lib.fla_poly_attn_workspace_bytes(1, 1, 128, 16, 64) == 2 * 128 * 128 * 2 + 128 * 64 * 2 + 128 * 4
    # backward without workspace
    dq, dk, dv = torch.empty_like(xq), torch.empty_like(xk), torch.empty_like(v)
    st = _lib.strides_arg
    import ctypes
    coef = (ctypes.c_float * 3)(0.0, 0.0, 0.5)
    rc = lib.fla_poly_attn_bwd(do.data_ptr(), xq.data_ptr(), xk.data_ptr(), v.data_ptr(), None, None, dq.data_ptr(),
                               dk.data_ptr(), dv.data_ptr(), 1, 1, 128, 16, 64, st(do), st(xq), st(xk), st(v), None,
                               st(dq), st(dk), st(dv), coef, 0, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == -9
    # a misaligned view has no fast-path kernel
    xq_odd = torch.empty(1, 1, 128, 24, dtype=torch.bfloat16, device=gpu_device)[..., 4:20]
    out = torch.empty_like(v)
    rc = lib.fla_poly_attn_fwd(xq_odd.data_ptr(), xk.data_ptr(), v.data_ptr(), out.data_ptr(), None, 1, 1, 128, 16, 64,
                               st(xq_odd), st(xk), st(v), st(out), coef, ctypes.c_float(0.0), 0,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == -8
    torch.cuda.synchronize()
