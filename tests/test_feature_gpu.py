"""Feature map inside the operator (fla_feature_attn_fwd/bwd, FeatureMapLinearAttention)
against the CPU oracle's statement of the caller's recipe -- feature map, then the product
(README.md:27-30 and flashlinear/test_attn.py:36-40 of the reference) -- and against this
package's own chunk-wise operator on features materialised in PyTorch (``-m gpu``).

Tolerances as for the product kernels: Frobenius-relative and max-abs/max <= 1e-2 against the
fp32 oracle fed the rounded 16-bit inputs (the oracle evaluates phi in fp32; the kernels round
phi(x) once to the storage dtype, the same quantisation a materialised q, k would have).
"""

import pytest
import torch

from flashy_linear_attention_amd import FeatureMapLinearAttention, LinearAttentionChunked
from flashy_linear_attention_amd.synthetic import WORKLOADS
from oracle import naive

from helpers import assert_close, gpu_fp32_reference

pytestmark = pytest.mark.gpu

# (batch, heads, seq, d_qk, d_v): one chunk, several chunks with shared states (equal padded widths
# up to 128), ragged ends, widths below the padded width, and shapes whose products run one by one
CASES = [
    (1, 2, 64, 64, 64),
    (1, 2, 256, 64, 64),
    (2, 3, 1024, 128, 128),
    (1, 2, 1088, 128, 128),
    (1, 2, 2112, 64, 64),
    (1, 2, 840, 32, 32),
    (1, 2, 1000, 64, 64),
    (1, 3, 1536, 104, 120),
    (1, 2, 768, 48, 40),
    (1, 2, 768, 256, 64),
    (1, 1, 640, 64, 128),
    (1, 1, 200, 256, 64),
    # two segments per (b, h): the totals kernel hands the walks their entry states itself
    (1, 100, 330, 128, 128),
    (2, 100, 1024, 64, 64),
    (1, 72, 512, 128, 128),  # (three segments per (b, h))
    (2, 80, 330, 128, 128),  # (no room for a second segment per (b, h): one)
]


def _inputs(dims, dtype, seed):
    b, h, n, dqk, dv = dims
    g = torch.Generator().manual_seed(seed)
    xq = torch.randn(b, h, n, dqk, generator=g)
    xk = torch.randn(b, h, n, dqk, generator=g)
    v = torch.randn(b, h, n, dv, generator=g)
    do = torch.randn(b, h, n, dv, generator=g)
    return tuple(t.to(dtype) for t in (xq, xk, v, do))


@pytest.mark.parametrize("kind", ["elu1", "softplus"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dims", CASES, ids=lambda d: "x".join(map(str, d)))
def test_feature_fwd_bwd_vs_oracle(dims, dtype, kind, gpu_device):
    xq, xk, v, do = _inputs(dims, dtype, seed=sum(dims))
    want_o = naive.feature_causal_dot_product(xq.float(), xk.float(), v.float(), kind)
    want_g = naive.feature_causal_dot_product_grads(xq.float(), xk.float(), v.float(), do.float(), kind)
    a, b, c = (t.to(gpu_device).requires_grad_(True) for t in (xq, xk, v))
    out = FeatureMapLinearAttention.apply(a, b, c, kind)
    assert out.dtype == dtype and out.shape == v.shape
    out.backward(do.to(gpu_device))
    assert_close("O", out, want_o)
    for name, got, want in (("dXq", a.grad, want_g[0]), ("dXk", b.grad, want_g[1]), ("dV", c.grad, want_g[2])):
        assert got.dtype == dtype and got.shape == want.shape
        assert_close(name, got, want)


def test_feature_operator_equals_chunked_operator_on_materialised_features(gpu_device):
    """phi applied by PyTorch in fp32 and rounded once, then LinearAttentionChunked: the same
    function and the same kernels, so results differ only where the kernels' fast exponential
    and PyTorch's round phi(x) to different 16-bit neighbours (a handful of elements)."""
    xq, xk, v, do = (t.to(gpu_device) for t in _inputs((2, 4, 1536, 64, 64), torch.bfloat16, seed=3))
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    out = FeatureMapLinearAttention.apply(a, b, c, "elu1")
    out.backward(do)
    q = (torch.nn.functional.elu(xq.float()) + 1).to(torch.bfloat16)
    k = (torch.nn.functional.elu(xk.float()) + 1).to(torch.bfloat16)
    c2 = v.clone().requires_grad_(True)
    ref = LinearAttentionChunked.apply(q, k, c2)
    ref.backward(do)
    assert_close("O", out, ref.float(), tol_fro=5e-4, tol_max=2e-3)
    assert_close("dV", c.grad, c2.grad.float(), tol_fro=5e-4, tol_max=2e-3)


def test_feature_operator_without_grad_and_under_autocast(gpu_device):
    xq, xk, v, _ = (t.to(gpu_device) for t in _inputs((1, 2, 512, 64, 64), torch.bfloat16, seed=5))
    with torch.no_grad():
        base = FeatureMapLinearAttention.apply(xq, xk, v, "softplus")
    with torch.autocast("cuda", dtype=torch.bfloat16):
        cast = FeatureMapLinearAttention.apply(xq.float(), xk.float(), v.float(), "softplus")
    assert cast.dtype == torch.bfloat16 and torch.equal(base, cast)
    with pytest.raises(ValueError, match="feature map"):
        FeatureMapLinearAttention.apply(xq, xk, v, "relu")


@pytest.mark.parametrize("name", ["C3", "C5"])
def test_feature_operator_full_size(name, gpu_device):
    """The benchmark workloads from their raw inputs: xq, xk ~ randn (what the workloads' q, k are
    the elu(.) + 1 of), every head against the oracle's formula in fp32 on the GPU."""
    w = WORKLOADS[name]
    gen = torch.Generator().manual_seed(0)
    xq, xk = (torch.randn(w.batch, w.heads, w.seq, w.d_qk, generator=gen).to(w.dtype).to(gpu_device) for _ in range(2))
    v, do = (torch.randn(w.batch, w.heads, w.seq, w.d_v, generator=gen).to(w.dtype).to(gpu_device) for _ in range(2))
    a, b, c = (t.clone().requires_grad_(True) for t in (xq, xk, v))
    out = FeatureMapLinearAttention.apply(a, b, c, "elu1")
    out.backward(do)
    q32, k32 = naive.feature_map(xq.float(), "elu1"), naive.feature_map(xk.float(), "elu1")
    o_ref, (dq_ref, dk_ref, dv_ref) = gpu_fp32_reference(q32, k32, v, do, True, heads_per_chunk=8 if w.seq <= 4096 else 1)
    assert_close(f"{name} O", out, o_ref)
    assert_close(f"{name} dV", c.grad, dv_ref)
    assert_close(f"{name} dXq", a.grad, dq_ref * naive.feature_map_slope(xq.float(), "elu1"))
    assert_close(f"{name} dXk", b.grad, dk_ref * naive.feature_map_slope(xk.float(), "elu1"))
    # one head against the CPU oracle
    sl = (slice(0, 1), slice(w.heads // 2, w.heads // 2 + 1))
    xqc, xkc, vc, doc = (t[sl].float().cpu() for t in (xq, xk, v, do))
    qc, kc = naive.feature_map(xqc, "elu1"), naive.feature_map(xkc, "elu1")
    assert_close(f"{name} O (CPU oracle)", out[sl], naive.causal_dot_product_blocked(qc, kc, vc, block=2048))
    dq_c, dk_c, dv_c = naive.causal_dot_product_grads_blocked(qc, kc, vc, doc, block=2048)
    assert_close(f"{name} dXq (CPU oracle)", a.grad[sl], dq_c * naive.feature_map_slope(xqc, "elu1"))
    assert_close(f"{name} dXk (CPU oracle)", b.grad[sl], dk_c * naive.feature_map_slope(xkc, "elu1"))
    assert_close(f"{name} dV (CPU oracle)", c.grad[sl], dv_c)


NORMALISED_CASES = [
    (1, 2, 256, 64, 64),
    (2, 3, 1024, 128, 128),
    (1, 2, 1088, 128, 128),
    (1, 2, 2112, 64, 64),
    (1, 2, 1000, 64, 64),
    (1, 2, 768, 256, 64),
    (1, 1, 200, 96, 32),
    (1, 100, 330, 128, 128),
    (2, 100, 1024, 64, 64),
    (1, 72, 512, 128, 128),  # (three segments per (b, h))
    (2, 80, 330, 128, 128),  # (no room for a second segment per (b, h): one)
]


@pytest.mark.parametrize("chunked", [True, False], ids=["chunked", "quadratic"])
@pytest.mark.parametrize("kind", ["elu1", "softplus"])
@pytest.mark.parametrize("dims", NORMALISED_CASES, ids=lambda d: "x".join(map(str, d)))
def test_feature_normalised_fwd_bwd_vs_oracle(dims, kind, chunked, gpu_device):
    """The whole caller-side recipe (map, product, normaliser) as one operator.  Gradient
    tolerances as for the normalised operator (tests/test_normalised_gpu.py): Frobenius-relative
    <= 1e-2, element bound 5e-2 of the largest magnitude."""
    xq, xk, v, do = _inputs(dims, torch.bfloat16, seed=sum(dims) + 1)
    eps = 1e-5
    a0, b0, c0 = (t.float().requires_grad_(True) for t in (xq, xk, v))
    want = naive.feature_linear_attention_normalised(a0, b0, c0, kind, eps)
    want_g = torch.autograd.grad(want, (a0, b0, c0), do.float())
    a, b, c = (t.to(gpu_device).requires_grad_(True) for t in (xq, xk, v))
    out = FeatureMapLinearAttention.apply(a, b, c, kind, True, eps, chunked)
    assert out.dtype == torch.bfloat16 and out.shape == v.shape
    out.backward(do.to(gpu_device))
    assert_close("out", out, want.detach())
    for name, got, w_ in (("dXq", a.grad, want_g[0]), ("dXk", b.grad, want_g[1]), ("dV", c.grad, want_g[2])):
        assert_close(name, got, w_, tol_fro=1e-2, tol_max=5e-2)
