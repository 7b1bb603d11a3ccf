"""Normalised causal linear attention (fla_linear_attn_normalised_fwd/bwd) against the CPU
oracle's statement of the reference's recipe, README.md:27-30 of the reference (``-m gpu``).

Tolerances.  Output and normaliser: Frobenius-relative and max-abs/max both <= 1e-2 against
the fp32 oracle fed the rounded 16-bit inputs (the normaliser itself is fp32 and is held to
1e-5).  Gradients: Frobenius-relative <= 1e-2; the element bound is 5e-2 of the largest
magnitude, because the gradient of a normalised average is a difference of two terms of
order one that both pass through 16-bit storage (dO = g / n and the product's dQ / dK), so
where few keys contribute one ulp of the cancelling terms is a few percent of the largest
gradient (the same bound and reasoning as the end-to-end test of the PyTorch recipe).
"""

import ctypes

import pytest
import torch

from flashy_linear_attention_amd import LinearAttention, LinearAttentionNormalised, _lib
from flashy_linear_attention_amd.normalised import linear_attention_normalised_bwd, linear_attention_normalised_fwd
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
from oracle import naive

from helpers import assert_close, reference_style_inputs, rel_max

pytestmark = pytest.mark.gpu

# (batch, heads, seq, d_qk, d_v): a single chunk, several chunks, ragged ends, every lane
# grouping (<= 32, 64, 128, 256 wide), small V, widths that take the scalar load path
CASES = [
    (1, 2, 256, 64, 64),
    (2, 3, 1024, 128, 128),
    (1, 2, 1088, 128, 128),
    (1, 2, 2112, 64, 64),
    (1, 2, 768, 256, 64),
    (1, 1, 640, 32, 32),
    (1, 2, 4160, 16, 16),
    (1, 2, 320, 100, 100),
    (1, 1, 192, 91, 64),
    (1, 1, 64, 256, 256),
    (1, 2, 1000, 64, 64),
    # two segments per (b, h): the totals kernel hands the walks their entry states itself
    (1, 100, 330, 128, 128),
    (2, 100, 1024, 64, 64),
    (1, 72, 512, 128, 128),  # (three segments per (b, h))
    (2, 80, 330, 128, 128),  # (no room for a second segment per (b, h): one)
    # fast-path widths that are whole 16-byte chunks but no power of two, many heads, ragged length:
    # single row tiles per workgroup with chunks of the padded width out of range
    (2, 80, 300, 72, 72),
    (1, 200, 513, 104, 120),
    (2, 32, 300, 48, 64),
    (1, 160, 257, 120, 72),
]


def _oracle(q, k, v, dy, eps):
    qo, ko, vo = (t.float().requires_grad_(True) for t in (q, k, v))
    out = naive.linear_attention_normalised(qo, ko, vo, eps=eps)
    out.backward(dy.float())
    denom = (q.float() * k.float().cumsum(-2)).sum(-1) + eps
    return out.detach(), denom, qo.grad, ko.grad, vo.grad


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dims", CASES, ids=lambda d: "x".join(map(str, d)))
def test_normalised_fwd_bwd_vs_oracle(dims, dtype, gpu_device):
    bs, nh, sq, dqk, dv = dims
    q, k, v, dy = reference_style_inputs(bs, nh, sq, dqk, dv, dtype, seed=sum(dims))
    eps = 1e-5
    want_o, want_n, want_dq, want_dk, want_dv = _oracle(q, k, v, dy, eps)
    qg, kg, vg = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionNormalised.apply(qg, kg, vg, eps)
    assert out.dtype == dtype and out.shape == v.shape
    out.backward(dy.to(gpu_device))
    assert_close("out", out, want_o)
    _, denom = linear_attention_normalised_fwd(qg.detach(), kg.detach(), vg.detach(), eps)
    assert denom.dtype == torch.float32 and denom.shape == q.shape[:3]
    assert rel_max(denom, want_n) <= 1e-5
    for name, got, want in (("dQ", qg.grad, want_dq), ("dK", kg.grad, want_dk), ("dV", vg.grad, want_dv)):
        assert got.dtype == dtype
        assert_close(name, got, want, tol_fro=1e-2, tol_max=5e-2)


def test_normalised_equals_recipe_around_the_product_op(gpu_device):
    """The fused operator against the reference's recipe built from this package's own
    LinearAttention and PyTorch ops in fp32: same output and gradients up to the one extra
    16-bit rounding of dQ and dK."""
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(2, 4, 1536, 128, 128, torch.bfloat16, seed=5))
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    num = LinearAttention.apply(qa, ka, va)
    denom = (qa.float() * ka.float().cumsum(-2)).sum(dim=-1, keepdim=True) + 1e-5
    ref = num.float() / denom
    ref.backward(dy.float())
    qb, kb, vb = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionNormalised.apply(qb, kb, vb, 1e-5)
    out.backward(dy)
    assert_close("out", out, ref.detach(), tol_fro=4e-3, tol_max=8e-3)
    for name, got, want in (("dQ", qb.grad, qa.grad), ("dK", kb.grad, ka.grad), ("dV", vb.grad, va.grad)):
        assert_close(name, got, want.float(), tol_fro=1e-2, tol_max=5e-2)


def test_normalised_rows_are_weighted_averages(gpu_device):
    """With positive q, k every output row is a convex combination of the value rows seen so
    far (eps aside): constant values come back unchanged, and outputs stay inside the running
    min / max of v."""
    g = torch.Generator().manual_seed(11)
    q = (torch.rand(1, 2, 1024, 64, generator=g) + 0.1).bfloat16().to(gpu_device)
    k = (torch.rand(1, 2, 1024, 64, generator=g) + 0.1).bfloat16().to(gpu_device)
    v = torch.full((1, 2, 1024, 64), 0.75).bfloat16().to(gpu_device)
    out, _ = linear_attention_normalised_fwd(q, k, v, 1e-6)
    assert (out.float() - 0.75).abs().max() <= 0.75 * 2 ** -7
    v = torch.randn(1, 2, 1024, 64, generator=g).bfloat16().to(gpu_device)
    out, _ = linear_attention_normalised_fwd(q, k, v, 1e-6)
    hi = v.float().cummax(dim=-2).values
    lo = v.float().cummin(dim=-2).values
    slack = 2 ** -6 * v.float().abs().max()
    assert (out.float() <= hi + slack).all() and (out.float() >= lo - slack).all()


def test_normalised_strided_layout_and_autocast(gpu_device):
    """(B, N, H, D) storage is taken as it is; fp32 inputs under autocast are cast to bf16."""
    bs, nh, sq, d = 2, 3, 512, 64
    q, k, v, dy = reference_style_inputs(bs, nh, sq, d, d, torch.bfloat16, seed=3)
    want_o, _, want_dq, want_dk, want_dv = _oracle(q, k, v, dy, 1e-5)

    def bnhd(t):
        return t.to(gpu_device).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)

    qs, ks, vs = (bnhd(t).requires_grad_(True) for t in (q, k, v))
    assert not qs.is_contiguous()
    out = LinearAttentionNormalised.apply(qs, ks, vs, 1e-5)
    out.backward(bnhd(dy))
    assert_close("out (strided)", out, want_o)
    for name, got, want in (("dQ", qs.grad, want_dq), ("dK", ks.grad, want_dk), ("dV", vs.grad, want_dv)):
        assert_close(name + " (strided)", got, want, tol_fro=1e-2, tol_max=5e-2)

    q32, k32, v32 = (t.float().to(gpu_device) for t in (q, k, v))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = LinearAttentionNormalised.apply(q32, k32, v32, 1e-5)
    assert out.dtype == torch.bfloat16
    assert_close("out (autocast)", out, want_o)


def test_normalised_c5_shape_against_recipe(gpu_device):
    """Long sequence (N = 32768, D = 64, two of the workload's heads): many chunks of running
    sums.  Checked on the GPU against the fp32 recipe around the product operator."""
    w = WORKLOADS["C5"]
    q, k, v, dy = (t.to(gpu_device) for t in make_inputs(w, heads=2))
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    num = LinearAttention.apply(qa, ka, va)
    denom = (qa.float() * ka.float().cumsum(-2)).sum(dim=-1, keepdim=True) + 1e-5
    ref = num.float() / denom
    ref.backward(dy.float())
    qb, kb, vb = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionNormalised.apply(qb, kb, vb, 1e-5)
    out.backward(dy)
    assert_close("out", out, ref.detach(), tol_fro=4e-3, tol_max=8e-3)
    for name, got, want in (("dQ", qb.grad, qa.grad), ("dK", kb.grad, ka.grad), ("dV", vb.grad, va.grad)):
        assert_close(name, got, want.float(), tol_fro=1e-2, tol_max=5e-2)


def test_normalised_workspace_is_checked(gpu_device):
    lib = _lib.load()
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 1024, 64, 64, torch.bfloat16, seed=1))
    out = torch.empty_like(v)
    denom = torch.empty(1, 2, 1024, dtype=torch.float32, device=gpu_device)
    st = _lib.strides_arg
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.fla_normalised_workspace_bytes(1, 2, 1024, 64, 64, 0)
    assert need > 0
    rc = lib.fla_linear_attn_normalised_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                            denom.data_ptr(), 1, 2, 1024, 64, 64, st(q), st(k), st(v), st(out),
                                            ctypes.c_float(1e-5), 0, 0, None, None, None, 0, stream)
    assert rc == -9  # FLA_ERR_WORKSPACE: several chunks need the chunk sums
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    work = torch.empty(need, dtype=torch.uint8, device=gpu_device)
    rc = lib.fla_linear_attn_normalised_bwd(dy.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                            denom.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                            1, 2, 1024, 64, 64, st(dy), st(q), st(k), st(v), st(out), st(dq), st(dk),
                                            st(dv), 0, 0, None, work.data_ptr(), need - 1, stream)
    assert rc == -9
    torch.cuda.synchronize()


@pytest.mark.parametrize("dims", [(2, 2, 1536, 128, 128), (1, 2, 2304, 64, 64), (1, 2, 1024, 256, 64), (1, 1, 256, 64, 64),
                                  (2, 8, 2450, 128, 128), (8, 8, 2100, 64, 64), (1, 4, 1500, 104, 120), (1, 3, 777, 32, 24)],
                         ids=lambda d: "x".join(map(str, d)))
def test_normalised_with_chunkwise_product(dims, gpu_device):
    """chunked=True: equal padded head dims up to 128 form the normaliser and its gradient terms
    inside the chunk-wise walk kernels (ragged last chunks and segments, several chunks per
    workgroup, padded widths among the cases), other shapes run the chunk states and the normaliser
    passes; parity against the oracle as for the quadratic product."""
    bs, nh, sq, dqk, dv = dims
    q, k, v, dy = reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=sum(dims) + 1)
    want_o, _, want_dq, want_dk, want_dv = _oracle(q, k, v, dy, 1e-5)
    qg, kg, vg = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionNormalised.apply(qg, kg, vg, 1e-5, True)
    out.backward(dy.to(gpu_device))
    assert_close("out", out, want_o)
    for name, got, want in (("dQ", qg.grad, want_dq), ("dK", kg.grad, want_dk), ("dV", vg.grad, want_dv)):
        assert_close(name, got, want, tol_fro=1e-2, tol_max=5e-2)


@pytest.mark.parametrize("dims", [(2, 3, 1280, 128, 128), (2, 3, 1280, 64, 64)], ids=lambda d: "x".join(map(str, d)))
def test_normalised_chunkwise_backward_with_and_without_the_forward_state(dims, gpu_device):
    """Backward given what the chunk-wise forward saved, and backward without it, both match the oracle;
    forward returns the same output and normaliser either way."""
    bs, nh, sq, dqk, dv = dims
    q, k, v, dy = reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=77)
    want_o, want_n, want_dq, want_dk, want_dv = _oracle(q, k, v, dy, 1e-5)
    q, k, v, dy = (t.to(gpu_device) for t in (q, k, v, dy))
    out, denom, state = linear_attention_normalised_fwd(q, k, v, 1e-5, True, want_state=True)
    out2, denom2 = linear_attention_normalised_fwd(q, k, v, 1e-5, True)
    assert state is not None and torch.equal(out, out2) and torch.equal(denom, denom2)
    assert_close("out", out, want_o)
    assert_close("n", denom, want_n.reshape(denom.shape), tol_fro=1e-4, tol_max=1e-3)
    for st in (state, None):
        got = linear_attention_normalised_bwd(dy, q, k, v, out, denom, True, st)
        for name, g, w in zip(("dQ", "dK", "dV"), got, (want_dq, want_dk, want_dv)):
            assert_close(f"{name} ({'with' if st is not None else 'without'} state)", g, w, tol_fro=1e-2, tol_max=5e-2)
