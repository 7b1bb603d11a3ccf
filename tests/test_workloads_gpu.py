"""Full-size benchmark workloads, golden fixtures, direct C-ABI calls and
size-independent properties on the GPU (``-m gpu``)."""

import ctypes

import numpy as np
import pytest
import torch

from flashy_linear_attention_amd import LinearAttention, LinearAttentionSmallVHD, _lib
from flashy_linear_attention_amd.kernels import (
    linear_flash_wrapper_bwd,
    linear_flash_wrapper_bwd_smallv_hd,
    linear_flash_wrapper_fwd,
    linear_flash_wrapper_fwd_smallv_hd,
)
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
from oracle import c_oracle, naive

from helpers import GOLDEN_CASES, assert_close, gpu_fp32_reference, load_golden, reference_style_inputs

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------- golden data
@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_hip_path_reproduces_golden_fixtures(name, gpu_device):
    ins, outs = load_golden(name)
    small_v = ins["v"].shape[-1] != ins["q"].shape[-1]
    fwd = linear_flash_wrapper_fwd_smallv_hd if small_v else linear_flash_wrapper_fwd
    bwd = linear_flash_wrapper_bwd_smallv_hd if small_v else linear_flash_wrapper_bwd
    q, k, v, do = (ins[n].to(gpu_device) for n in ("q", "k", "v", "do"))
    assert_close("O", fwd(q, k, v), outs["o"])
    for got, n in zip(bwd(do, q, k, v), ("dq", "dk", "dv")):
        assert_close(n, got, outs[n])


# ------------------------------------------------- raw C ABI against the C oracle
def _tri_call(x, y, z, d_out, upper):
    """Out = mask(X Y^T) Z through fla_tri_xyt_z with nothing but pointers and sizes."""
    lib = _lib.load()
    b, h, n, dc = x.shape
    out = torch.empty(b, h, n, d_out, dtype=x.dtype, device=x.device)
    code = {torch.bfloat16: 0, torch.float16: 1}[x.dtype]
    rc = lib.fla_tri_xyt_z(
        x.data_ptr(), y.data_ptr(), z.data_ptr(), out.data_ptr(), b, h, n, dc, d_out,
        _lib.strides_arg(x), _lib.strides_arg(y), _lib.strides_arg(z), _lib.strides_arg(out),
        int(upper), code, torch.cuda.current_stream().cuda_stream,
    )
    assert rc == 0, lib.fla_strerror(rc)
    return out


@pytest.mark.parametrize("shape", [(1, 2, 64, 32, 32), (2, 1, 128, 64, 16), (1, 1, 96, 24, 40), (1, 3, 37, 16, 16)])
def test_c_abi_matches_c_oracle(shape, gpu_device):
    """All four products of the path through the exported primitive, checked
    against the brute-force C oracle (including N that is not a multiple of 64,
    which the C ABI accepts although the Python wrappers do not)."""
    b, h, n, dqk, dv = shape
    q, k, v, do = reference_style_inputs(b, h, n, dqk, dv, torch.bfloat16, seed=n + dqk)
    o_w = c_oracle.fwd(q.float(), k.float(), v.float())
    dq_w, dk_w, dv_w = c_oracle.bwd(q.float(), k.float(), v.float(), do.float())
    qg, kg, vg, dog = (t.to(gpu_device) for t in (q, k, v, do))
    assert_close("O", _tri_call(qg, kg, vg, dv, upper=False), torch.from_numpy(o_w))
    assert_close("dQ", _tri_call(dog, vg, kg, dqk, upper=False), torch.from_numpy(dq_w))
    assert_close("dV", _tri_call(kg, qg, dog, dv, upper=True), torch.from_numpy(dv_w))
    assert_close("dK", _tri_call(vg, dog, qg, dqk, upper=True), torch.from_numpy(dk_w))


def test_c_abi_runs_on_a_side_stream(gpu_device):
    q, k, v, _ = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 256, 64, 64, torch.bfloat16, seed=2))
    base = linear_flash_wrapper_fwd(q, k, v)
    side = torch.cuda.Stream(device=gpu_device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        again = linear_flash_wrapper_fwd(q, k, v)
    side.synchronize()
    assert torch.equal(base, again)


# ------------------------------------------------------------------ properties
def test_causality_bit_exact(gpu_device):
    """Perturbing token j must leave every output row < j bit-identical; for the
    gradients, dK/dV rows > j' are untouched when dO changes at row j'."""
    q, k, v, do = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 512, 64, 64, torch.bfloat16, seed=4))
    base = linear_flash_wrapper_fwd(q, k, v)
    j = 300
    k2, v2 = k.clone(), v.clone()
    k2[:, :, j] += 1
    v2[:, :, j] -= 2
    moved = linear_flash_wrapper_fwd(q, k2, v2)
    assert torch.equal(moved[:, :, :j], base[:, :, :j])
    assert not torch.equal(moved[:, :, j:], base[:, :, j:])
    dq, dk, dv = linear_flash_wrapper_bwd(do, q, k, v)
    do2 = do.clone()
    do2[:, :, j] *= -3
    dq2, dk2, dv2 = linear_flash_wrapper_bwd(do2, q, k, v)
    assert torch.equal(dk2[:, :, j + 1:], dk[:, :, j + 1:]) and torch.equal(dv2[:, :, j + 1:], dv[:, :, j + 1:])
    assert torch.equal(dq2[:, :, :j], dq[:, :, :j]) and torch.equal(dq2[:, :, j + 1:], dq[:, :, j + 1:])


def test_heads_independent_and_deterministic(gpu_device):
    q, k, v, do = (t.to(gpu_device) for t in reference_style_inputs(2, 5, 384, 128, 128, torch.bfloat16, seed=6))
    perm = torch.tensor([3, 0, 4, 1, 2], device=gpu_device)
    a = linear_flash_wrapper_fwd(q, k, v)
    assert torch.equal(a, linear_flash_wrapper_fwd(q, k, v))
    b = linear_flash_wrapper_fwd(q[:, perm].contiguous(), k[:, perm].contiguous(), v[:, perm].contiguous())
    assert torch.equal(a[:, perm], b)
    g1 = linear_flash_wrapper_bwd(do, q, k, v)
    g2 = linear_flash_wrapper_bwd(do[:, perm].contiguous(), q[:, perm].contiguous(), k[:, perm].contiguous(),
                                  v[:, perm].contiguous())
    for x, y in zip(g1, g2):
        assert torch.equal(x[:, perm], y)


def test_power_of_two_scaling_is_exact(gpu_device):
    """O is linear in v and in q: scaling by 2 only shifts exponents, so the
    result must scale bit-exactly."""
    q, k, v, _ = (t.to(gpu_device) for t in reference_style_inputs(1, 3, 256, 64, 64, torch.bfloat16, seed=8))
    base = linear_flash_wrapper_fwd(q, k, v)
    assert torch.equal(linear_flash_wrapper_fwd(q, k, v * 2), base * 2)
    assert torch.equal(linear_flash_wrapper_fwd(q * 0.5, k, v), base * 0.5)


def test_zero_padding_head_dim_is_bit_exact(gpu_device):
    """A 48-wide problem and the same data zero-padded to 64 run the same MFMA
    sequence: outputs must agree bit for bit."""
    q, k, v, do = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 256, 48, 48, torch.bfloat16, seed=9))
    pad = lambda t: torch.nn.functional.pad(t, (0, 16))
    o = linear_flash_wrapper_fwd(q, k, v)
    op = linear_flash_wrapper_fwd(pad(q), pad(k), pad(v))
    assert torch.equal(op[..., :48], o) and torch.count_nonzero(op[..., 48:]) == 0
    g = linear_flash_wrapper_bwd(do, q, k, v)
    gp = linear_flash_wrapper_bwd(pad(do), pad(q), pad(k), pad(v))
    for x, y in zip(g, gp):
        assert torch.equal(y[..., :48], x) and torch.count_nonzero(y[..., 48:]) == 0


def test_small_v_equals_equal_d_on_padded_v(gpu_device):
    q, k, v, do = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 256, 64, 32, torch.bfloat16, seed=10))
    pad = lambda t: torch.nn.functional.pad(t, (0, 32))
    o = linear_flash_wrapper_fwd_smallv_hd(q, k, v)
    assert torch.equal(linear_flash_wrapper_fwd(q, k, pad(v))[..., :32], o)
    dq, dk, dv = linear_flash_wrapper_bwd_smallv_hd(do, q, k, v)
    dq2, dk2, dv2 = linear_flash_wrapper_bwd(pad(do), q, k, pad(v))
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2[..., :32])


# ------------------------------------------------------- benchmark workloads
@pytest.mark.parametrize("name", ["C2", "C3", "C4", "C5"])
def test_benchmark_workload(name, gpu_device):
    """Each benchmark workload at full size: every head against the oracle's
    formula in fp32 on the GPU, and a sample of heads against the oracle run in
    fp32 on the CPU (one head of C5 alone is 2x137 GFLOP there)."""
    w = WORKLOADS[name]
    q, k, v, do = (t.to(gpu_device) for t in make_inputs(w))
    op = LinearAttentionSmallVHD if w.small_v else LinearAttention
    qg, kg, vg = (t.clone().requires_grad_(w.backward) for t in (q, k, v))
    out = op.apply(qg, kg, vg)
    assert out.dtype == w.dtype and out.shape == v.shape
    if w.backward:
        out.backward(do)
    got = [out.detach()] + ([qg.grad, kg.grad, vg.grad] if w.backward else [])
    names = ["O", "dQ", "dK", "dV"][: len(got)]

    o_ref, g_ref = gpu_fp32_reference(q, k, v, do, w.backward, heads_per_chunk=8 if w.seq <= 4096 else 1)
    for n, x, y in zip(names, got, [o_ref] + (g_ref or [])):
        assert_close(f"{name} {n} (all heads, fp32 GPU)", x, y)

    sample = [(0, 0), (w.batch - 1, w.heads - 1)] if w.seq <= 4096 else [(0, w.heads // 2)]
    for bi, hi in sample:
        sl = (slice(bi, bi + 1), slice(hi, hi + 1))
        qc, kc, vc, doc = (t[sl].float().cpu() for t in (q, k, v, do))
        want = [naive.causal_dot_product_blocked(qc, kc, vc, block=2048)]
        if w.backward:
            want += list(naive.causal_dot_product_grads_blocked(qc, kc, vc, doc, block=2048))
        for n, x, y in zip(names, got, want):
            assert_close(f"{name} {n} head {(bi, hi)} (CPU oracle)", x[sl], y)


def test_c5_end_to_end_with_denominator(gpu_device):
    """Long-context case through the README recipe with eps = 1e-5
    (README.md:27-30), four heads, against the same recipe in fp32."""
    w = WORKLOADS["C5"]
    q, k, v, _ = (t.to(gpu_device) for t in make_inputs(w, heads=4))
    with torch.no_grad():
        num = LinearAttention.apply(q, k, v).float()
        denom = (q.float() * k.float().cumsum(-2)).sum(-1, keepdim=True) + 1e-5
        got = num / denom
        want = naive.causal_dot_product_blocked(q.float(), k.float(), v.float(), block=2048) / denom
    assert_close("normalised O", got, want)
