"""The extension operators at the full size of the benchmark workloads (``-m gpu``): the
chunk-wise operator (C3, C4, C5), the normalised operator with the quadratic and with the
chunk-wise product (C3, C4) and the polynomial score map at C4's size from the 16-wide x.

Scheme of tests/test_workloads_gpu.py::test_benchmark_workload: every head against the
oracle's formula evaluated in fp32 on the GPU, and a sample of heads against the oracle run in
fp32 on the CPU.  Tolerances (helpers.py): Frobenius-relative and max-abs/max <= 1e-2, the
reference's criterion (flashlinear/test_attn.py:17,24-25); gradients of the normalised
operators: Frobenius-relative <= 1e-2 and max-abs/max <= 5e-2 (reasoning in
tests/test_normalised_gpu.py).

Normalised gradients on Taylor features (C4) are compared from row 128 on.  There the
normaliser of row i is a sum of i + 1 squares (x_i . x_j)^2 / 2, which for the first rows can
be arbitrarily close to zero; the gradient is the difference of two terms of size |g| |k| / n
that cancel almost entirely (for row 0 exactly, up to eps), and each term passes through
16-bit storage once (dO = g / n, and the product's dQ / dK), so one ulp of a term exceeds the
true value by orders of magnitude.  Gradient rows >= 128 depend only on rows >= 128 (dK_j and
dV_j sum over i >= j), so the cut is clean; outputs are compared on every row.
"""

import math

import pytest
import torch

from flashy_linear_attention_amd import LinearAttentionChunked, LinearAttentionNormalised, PolynomialLinearAttention
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
from oracle import naive

from helpers import assert_close, gpu_fp32_reference, rel_max

pytestmark = pytest.mark.gpu


ILL_CONDITIONED_ROWS = 128  # see the module docstring


def _sample_heads(w):
    return [(0, 0), (w.batch - 1, w.heads - 1)] if w.seq <= 4096 else [(0, w.heads // 2)]


@pytest.mark.parametrize("name", ["C3", "C4", "C5"])
def test_chunked_operator_full_size(name, gpu_device):
    w = WORKLOADS[name]
    q, k, v, do = (t.to(gpu_device) for t in make_inputs(w))
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionChunked.apply(qg, kg, vg)
    assert out.dtype == w.dtype and out.shape == v.shape
    out.backward(do)
    got = [out.detach(), qg.grad, kg.grad, vg.grad]
    names = ["O", "dQ", "dK", "dV"]
    o_ref, g_ref = gpu_fp32_reference(q, k, v, do, True, heads_per_chunk=8 if w.seq <= 4096 else 1)
    for n, x, y in zip(names, got, [o_ref] + g_ref):
        assert_close(f"{name} chunked {n} (all heads, fp32 GPU)", x, y)
    del o_ref, g_ref
    for bi, hi in _sample_heads(w):
        sl = (slice(bi, bi + 1), slice(hi, hi + 1))
        qc, kc, vc, doc = (t[sl].float().cpu() for t in (q, k, v, do))
        want = [naive.causal_dot_product_blocked(qc, kc, vc, block=2048)]
        want += list(naive.causal_dot_product_grads_blocked(qc, kc, vc, doc, block=2048))
        for n, x, y in zip(names, got, want):
            assert_close(f"{name} chunked {n} head {(bi, hi)} (CPU oracle)", x[sl], y)


def _normalised_reference(q, k, v, dy, eps):
    """out, n, dq, dk, dv of the reference's recipe (README.md:27-30) in fp32 by autograd, on
    whatever device the inputs live."""
    qo, ko, vo = (t.float().requires_grad_(True) for t in (q, k, v))
    out = naive.linear_attention_normalised(qo, ko, vo, eps=eps)
    dq, dk, dv = torch.autograd.grad(out, (qo, ko, vo), dy.float())
    denom = (q.float() * k.float().cumsum(-2)).sum(-1) + eps
    return out.detach(), denom, dq, dk, dv


@pytest.mark.parametrize("chunked", [False, True], ids=["quadratic", "chunked"])
@pytest.mark.parametrize("name", ["C3", "C4"])
def test_normalised_operator_full_size(name, chunked, gpu_device):
    w = WORKLOADS[name]
    eps = 1e-5
    q, k, v, dy = (t.to(gpu_device) for t in make_inputs(w))
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionNormalised.apply(qg, kg, vg, eps, chunked)
    assert out.dtype == w.dtype and out.shape == v.shape
    out.backward(dy)
    got = [out.detach(), qg.grad, kg.grad, vg.grad]
    names = ["out", "dQ", "dK", "dV"]
    tols = [(1e-2, 1e-2)] + [(1e-2, 5e-2)] * 3
    r0 = [0] + [ILL_CONDITIONED_ROWS if w.features == "taylor2" else 0] * 3  # first row compared, per tensor
    # every head, fp32 on the GPU, four heads at a time (the autograd graph keeps several N x N tensors)
    ref = [torch.empty(t.shape, dtype=torch.float32, device=gpu_device) for t in (v, q, k, v)]
    for bi in range(w.batch):
        for h0 in range(0, w.heads, 4):
            sl = (slice(bi, bi + 1), slice(h0, h0 + 4))
            o_r, _, dq_r, dk_r, dv_r = _normalised_reference(q[sl], k[sl], v[sl], dy[sl], eps)
            for buf, val in zip(ref, (o_r, dq_r, dk_r, dv_r)):
                buf[sl] = val
    for n, x, y, (tf, tm), r in zip(names, got, ref, tols, r0):
        assert_close(f"{name} normalised {n} (all heads, fp32 GPU)", x[:, :, r:], y[:, :, r:], tol_fro=tf, tol_max=tm)
    del ref
    for bi, hi in _sample_heads(w):
        sl = (slice(bi, bi + 1), slice(hi, hi + 1))
        want = _normalised_reference(*(t[sl].cpu() for t in (q, k, v, dy)), eps)
        for n, x, y, (tf, tm), r in zip(names, got, (want[0],) + want[2:], tols, r0):
            assert_close(f"{name} normalised {n} head {(bi, hi)} (CPU oracle)", x[sl][:, :, r:], y[:, :, r:],
                         tol_fro=tf, tol_max=tm)


@pytest.mark.parametrize("normalise", [False, True], ids=["plain", "normalised"])
def test_polynomial_operator_at_c4_size(normalise, gpu_device):
    """C4's function from the 16-wide x behind its 256 Taylor features: f(u) = u^2 / 2."""
    w = WORKLOADS["C4"]
    r, coef, eps = math.isqrt(w.d_qk), (0.0, 0.0, 0.5), 1e-5
    gen = torch.Generator().manual_seed(0)
    xq = (0.5 * torch.randn(w.batch, w.heads, w.seq, r, generator=gen)).to(w.dtype).to(gpu_device)
    xk = (0.5 * torch.randn(w.batch, w.heads, w.seq, r, generator=gen)).to(w.dtype).to(gpu_device)
    v = torch.randn(w.batch, w.heads, w.seq, w.d_v, generator=gen).to(w.dtype).to(gpu_device)
    do = torch.randn(w.batch, w.heads, w.seq, w.d_v, generator=gen).to(w.dtype).to(gpu_device)
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    out = PolynomialLinearAttention.apply(a, b, c, *coef, normalise, eps)
    assert out.dtype == w.dtype and out.shape == v.shape
    out.backward(do)
    got = [out.detach(), a.grad, b.grad, c.grad]
    names = ["O", "dXq", "dXk", "dV"]
    tols = [(1e-2, 1e-2)] + [(1e-2, 5e-2 if normalise else 1e-2)] * 3
    r0 = [0] + [ILL_CONDITIONED_ROWS if normalise else 0] * 3

    def reference(xq_, xk_, v_, do_):
        xo, yo, vo = (t.float().requires_grad_(True) for t in (xq_, xk_, v_))
        fn = naive.poly_linear_attention_normalised if normalise else naive.poly_causal_dot_product
        o = fn(xo, yo, vo, coef, eps) if normalise else fn(xo, yo, vo, coef)
        return (o.detach(),) + torch.autograd.grad(o, (xo, yo, vo), do_.float())

    ref = [torch.empty(t.shape, dtype=torch.float32, device=gpu_device) for t in (v, xq, xk, v)]
    for bi in range(w.batch):
        for h0 in range(0, w.heads, 4):
            sl = (slice(bi, bi + 1), slice(h0, h0 + 4))
            for buf, val in zip(ref, reference(xq[sl], xk[sl], v[sl], do[sl])):
                buf[sl] = val
    for n, x, y, (tf, tm), r in zip(names, got, ref, tols, r0):
        assert_close(f"poly {n} (all heads, fp32 GPU)", x[:, :, r:], y[:, :, r:], tol_fro=tf, tol_max=tm)
    del ref
    for bi, hi in _sample_heads(w):
        sl = (slice(bi, bi + 1), slice(hi, hi + 1))
        want = reference(*(t[sl].cpu() for t in (xq, xk, v, do)))
        for n, x, y, (tf, tm), r in zip(names, got, want, tols, r0):
            assert_close(f"poly {n} head {(bi, hi)} (CPU oracle)", x[sl][:, :, r:], y[:, :, r:], tol_fro=tf, tol_max=tm)
