"""Host-side checks that run without a GPU: the shared library loads and exports
the declared ABI, argument validation in the C ABI and in the Python wrappers,
and the oracle against the committed golden fixtures."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

from flashy_linear_attention_amd import LinearAttention, LinearAttentionSmallVHD, _lib
from flashy_linear_attention_amd import kernels
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
from oracle import c_oracle, naive

from helpers import GOLDEN_CASES, load_golden

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "fla.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fla_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert {"fla_linear_attn_fwd", "fla_linear_attn_bwd", "fla_linear_attn_smallv_fwd",
            "fla_linear_attn_smallv_bwd", "fla_tri_xyt_z", "fla_abi_version", "fla_strerror"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/fla.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert lib.fla_abi_version() == _lib.ABI_VERSION


def test_package_surface_matches_reference_names():
    """flashlinear/__init__.py:1-2 and flashlinear/kernels/__init__.py:1-5."""
    assert issubclass(LinearAttention, torch.autograd.Function)
    assert issubclass(LinearAttentionSmallVHD, torch.autograd.Function)
    for n in ("linear_flash_wrapper_fwd", "linear_flash_wrapper_bwd",
              "linear_flash_wrapper_fwd_smallv_hd", "linear_flash_wrapper_bwd_smallv_hd"):
        assert callable(getattr(kernels, n))


def _null_call(name, *tail):
    fn = getattr(_lib.load(), name)
    nptr = {"fla_linear_attn_fwd": 4, "fla_linear_attn_bwd": 7, "fla_linear_attn_smallv_fwd": 4,
            "fla_linear_attn_smallv_bwd": 7, "fla_tri_xyt_z": 4}[name]
    return fn, nptr


S = (ctypes.c_int64 * 4)(4096, 2048, 32, 1)
BAD_S = (ctypes.c_int64 * 4)(4096, 2048, 64, 2)
# fake device pointers 4 GiB apart (distinct tensors must not overlap); never dereferenced:
# every call below fails validation first
A = [ctypes.c_void_p((i + 1) << 32) for i in range(10)]
P = A[0]


def test_c_abi_validation_codes():
    lib = _lib.load()
    f = lib.fla_linear_attn_fwd
    assert f(A[0], A[1], A[2], A[3], 1, 2, 64, 32, S, S, S, S, 7, None) == -2          # dtype
    assert f(A[0], A[1], A[2], A[3], 1, 2, 64, 257, S, S, S, S, 0, None) == -3         # head dim
    assert f(A[0], A[1], A[2], A[3], 1, 2, 64, 0, S, S, S, S, 0, None) == -3
    assert f(A[0], A[1], A[2], A[3], -1, 2, 64, 32, S, S, S, S, 0, None) == -5         # shape
    assert f(None, A[1], A[2], A[3], 1, 2, 64, 32, S, S, S, S, 0, None) == -1       # null pointer
    assert f(A[0], A[1], A[2], A[3], 1, 2, 64, 32, S, BAD_S, S, S, 0, None) == -6      # innermost stride
    assert f(A[0], A[1], A[2], A[3], 1, 2, 64, 32, S, S, None, S, 0, None) == -6       # missing strides
    assert f(A[0], A[1], A[2], A[3], 0, 2, 64, 32, S, S, S, S, 0, None) == 0           # empty problem: no-op
    assert f(A[0], A[1], A[2], A[3], 1, 2, 0, 32, S, S, S, S, 1, None) == 0
    b = lib.fla_linear_attn_bwd
    assert b(A[0], A[1], A[2], A[3], A[4], A[5], A[6], 1, 2, 64, 300, S, S, S, S, S, S, S, 0, None) == -3
    assert b(A[0], A[1], A[2], A[3], A[4], None, A[6], 1, 2, 64, 32, S, S, S, S, S, S, S, 0, None) == -1
    sf = lib.fla_linear_attn_smallv_fwd
    assert sf(A[0], A[1], A[2], A[3], 1, 2, 64, 64, 24, S, S, S, S, 0, None) == -4     # D_v not a power of two
    assert sf(A[0], A[1], A[2], A[3], 1, 2, 64, 32, 64, S, S, S, S, 0, None) == -4     # D_v above padded D_qk
    assert sf(A[0], A[1], A[2], A[3], 1, 2, 64, 300, 64, S, S, S, S, 0, None) == -3
    assert sf(A[0], A[1], A[2], A[3], 1, 0, 64, 37, 64, S, S, S, S, 0, None) == 0      # 64 <= next_pow2(37): accepted
    sb = lib.fla_linear_attn_smallv_bwd
    assert sb(A[0], A[1], A[2], A[3], A[4], A[5], A[6], 1, 2, 64, 257, 16, S, S, S, S, S, S, S, 0, None) == -3
    t = lib.fla_tri_xyt_z
    assert t(A[0], A[1], A[2], A[3], 1, 2, 64, 32, 300, S, S, S, S, 0, 0, None) == -3
    assert t(A[0], A[1], A[2], A[3], 1, 2, 64, 32, 32, S, S, S, S, 1, 5, None) == -2
    nf = lib.fla_linear_attn_normalised_fwd
    eps = ctypes.c_float(1e-5)
    assert nf(A[0], A[1], A[2], A[3], A[4], 1, 2, 64, 32, 32, S, S, S, S, eps, 9, 0, None, None, None, 0, None) == -2
    assert nf(A[0], A[1], A[2], A[3], A[4], 1, 2, 64, 257, 32, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == -3
    assert nf(A[0], A[1], A[2], A[3], A[4], 1, 2, 64, 32, 0, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == -4
    assert nf(A[0], A[1], A[2], A[3], A[4], 300, 300, 64, 32, 32, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == -5   # B H > 65535
    assert nf(A[0], A[1], A[2], A[3], None, 1, 2, 64, 32, 32, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == -1    # denom
    assert nf(A[0], A[1], A[2], A[3], A[4], 1, 2, 64, 32, 32, S, S, BAD_S, S, eps, 0, 0, None, None, None, 0, None) == -6
    assert nf(A[0], A[1], A[2], A[3], A[4], 1, 2, 4096, 32, 32, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == -9     # chunk sums need workspace
    assert nf(A[0], A[1], A[2], A[3], A[4], 1, 0, 64, 32, 32, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == 0
    nb = lib.fla_linear_attn_normalised_bwd
    assert nb(A[0], A[1], A[2], A[3], A[4], A[5], A[6], A[7], A[8], 1, 2, 64, 32, 32, S, S, S, S, S, S, S, S, 0, 0, None, None, 0, None) == -9
    assert nb(A[0], A[1], A[2], A[3], A[4], None, A[6], A[7], A[8], 1, 2, 64, 32, 32, S, S, S, S, S, S, S, S, 0, 1, None, A[9], 1 << 30, None) == -1
    assert lib.fla_normalised_workspace_bytes(1, 2, 64, 32, 32, 0) >= 2 * 64 * 32 * 2 + 2 * 64 * 4
    assert lib.fla_normalised_workspace_bytes(1, 2, 64, 300, 32, 0) == 0
    assert (lib.fla_normalised_workspace_bytes(1, 2, 4096, 64, 64, 1)
            > lib.fla_normalised_workspace_bytes(1, 2, 4096, 64, 64, 0))
    for code in range(0, -11, -1):
        assert lib.fla_strerror(code)
    assert lib.fla_strerror(-3) == b"Only head_dims <= 256 are supported."


def test_c_abi_rejects_outputs_that_overlap_inputs():
    """The reference's wrappers allocate fresh outputs (linear_attn_kernels.py:327,366-368); the C
    ABI takes caller-owned outputs, so an overlap with an input or another output is an error."""
    lib = _lib.load()
    q, k, v, o, g, dq, dk, dv = A[:8]
    inside_q = ctypes.c_void_p(q.value + 2 * 64 * 32)  # second head of q
    just_past_q = ctypes.c_void_p(q.value + 2 * (4096 + 2048 + 63 * 32 + 32))
    f = lib.fla_linear_attn_fwd
    assert f(q, k, v, q, 2, 2, 64, 32, S, S, S, S, 0, None) == -10
    assert f(q, k, v, inside_q, 2, 2, 64, 32, S, S, S, S, 0, None) == -10
    assert f(q, k, v, just_past_q, 2, 0, 64, 32, S, S, S, S, 0, None) == 0     # empty problem: nothing to overlap
    assert f(q, k, q, q, 2, 2, 64, 32, S, S, S, S, 7, None) == -2              # argument errors come first
    b = lib.fla_linear_attn_bwd
    assert b(g, q, k, v, dq, dk, q, 1, 2, 64, 32, S, S, S, S, S, S, S, 0, None) == -10     # dV on q
    assert b(g, q, k, v, dq, dq, dv, 1, 2, 64, 32, S, S, S, S, S, S, S, 0, None) == -10    # dQ and dK shared
    assert b(g, q, k, v, g, dk, dv, 1, 2, 64, 32, S, S, S, S, S, S, S, 0, None) == -10     # in-place on dO
    sb = lib.fla_linear_attn_smallv_bwd
    assert sb(g, q, k, v, dq, k, dv, 1, 2, 64, 64, 16, S, S, S, S, S, S, S, 0, None) == -10
    t = lib.fla_tri_xyt_z
    assert t(q, k, v, v, 1, 2, 64, 32, 32, S, S, S, S, 0, 0, None) == -10
    tc = lib.fla_tri_xyt_z_chunked
    assert tc(q, k, v, k, 1, 2, 64, 32, 32, S, S, S, S, 0, 0, None, 0, None) == -10
    cf = lib.fla_linear_attn_chunked_fwd
    assert cf(q, k, v, q, 1, 2, 64, 32, 32, S, S, S, S, 0, None, None, None, 0, None) == -10
    cb = lib.fla_linear_attn_chunked_bwd
    assert cb(g, q, k, v, dq, dk, v, 1, 2, 64, 32, 32, S, S, S, S, S, S, S, 0, None, None, 0, None) == -10
    eps = ctypes.c_float(1e-5)
    nf = lib.fla_linear_attn_normalised_fwd
    assert nf(q, k, v, k, A[8], 1, 2, 64, 32, 32, S, S, S, S, eps, 0, 0, None, None, None, 0, None) == -10
    nb = lib.fla_linear_attn_normalised_bwd
    # the forward's output is an input of backward: a gradient must not land on it
    assert nb(g, q, k, v, o, A[8], dq, o, dv, 1, 2, 64, 32, 32, S, S, S, S, S, S, S, S, 0, 0, None, A[9], 1 << 30, None) == -10
    coef = (ctypes.c_float * 3)(0.0, 0.0, 0.5)
    pf = lib.fla_poly_attn_fwd
    assert pf(q, k, v, v, None, 1, 2, 64, 16, 32, S, S, S, S, coef, eps, 0, None) == -10
    assert lib.fla_strerror(-10)


def test_wrapper_assertions_match_reference():
    """The reference raises AssertionError before launching
    (linear_attn_kernels.py:322-325,361-364; linear_attn_kernels_smallv_hd.py:336-342,381-384)."""
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="Only head_dims <= 256"):
        kernels.linear_flash_wrapper_fwd(z(1, 1, 64, 320), z(1, 1, 64, 320), z(1, 1, 64, 320))
    with pytest.raises(AssertionError, match="multiple of 64"):
        kernels.linear_flash_wrapper_fwd(z(1, 1, 96, 64), z(1, 1, 96, 64), z(1, 1, 96, 64))
    with pytest.raises(AssertionError, match="multiple of 32"):
        kernels.linear_flash_wrapper_fwd(z(1, 1, 48, 200), z(1, 1, 48, 200), z(1, 1, 48, 200))
    with pytest.raises(AssertionError, match="multiple of 64"):
        kernels.linear_flash_wrapper_bwd(z(1, 1, 100, 64), z(1, 1, 100, 64), z(1, 1, 100, 64), z(1, 1, 100, 64))
    with pytest.raises(AssertionError, match="power of 2"):
        kernels.linear_flash_wrapper_fwd_smallv_hd(z(1, 1, 64, 64), z(1, 1, 64, 64), z(1, 1, 64, 24))
    with pytest.raises(AssertionError, match="less than Query/Key"):
        kernels.linear_flash_wrapper_fwd_smallv_hd(z(1, 1, 64, 32), z(1, 1, 64, 32), z(1, 1, 64, 64))
    with pytest.raises(AssertionError, match="Only head_dims <= 256"):
        kernels.linear_flash_wrapper_bwd_smallv_hd(z(1, 1, 64, 16), z(1, 1, 64, 260), z(1, 1, 64, 260), z(1, 1, 64, 16))
    with pytest.raises(AssertionError, match="multiple of 64"):
        kernels.linear_flash_wrapper_bwd_smallv_hd(z(1, 1, 96, 16), z(1, 1, 96, 64), z(1, 1, 96, 64), z(1, 1, 96, 16))


def test_cpu_tensors_fail_loudly_instead_of_falling_back():
    q = torch.ones(1, 1, 64, 32, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        LinearAttention.apply(q, q, q)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        LinearAttentionSmallVHD.apply(q, q, q)


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_oracle_reproduces_golden_fixtures(name):
    ins, outs = load_golden(name)
    q, k, v, do = (ins[n].float() for n in ("q", "k", "v", "do"))
    torch.testing.assert_close(naive.causal_dot_product(q, k, v), outs["o"], rtol=2e-5, atol=2e-4)
    for got, n in zip(naive.causal_dot_product_grads(q, k, v, do), ("dq", "dk", "dv")):
        torch.testing.assert_close(got, outs[n], rtol=2e-5, atol=2e-4)
    np.testing.assert_allclose(c_oracle.fwd(q, k, v), outs["o"].numpy(), rtol=2e-6, atol=2e-5)
    for got, n in zip(c_oracle.bwd(q, k, v, do), ("dq", "dk", "dv")):
        np.testing.assert_allclose(got, outs[n].numpy(), rtol=2e-6, atol=2e-5)


def test_synthetic_workloads_have_the_stated_shapes_and_features():
    w = WORKLOADS["C3"]
    assert (w.batch, w.heads, w.seq, w.d_qk, w.d_v, w.dtype) == (4, 32, 4096, 128, 128, torch.bfloat16)
    assert abs(w.flops_fwd + w.flops_bwd - 1.924e12) < 1e9
    q, k, v, do = make_inputs(WORKLOADS["C4"], batch=1, heads=1, seq=64)
    assert q.shape == (1, 1, 64, 256) and v.shape == (1, 1, 64, 64) and q.dtype == torch.bfloat16
    q1, k1, v1, _ = make_inputs(WORKLOADS["C2"], batch=1, heads=2, seq=64)
    assert (q1 > 0).all() and (k1 > 0).all() and q1.dtype == torch.float16
    q2, *_ = make_inputs(WORKLOADS["C2"], batch=1, heads=2, seq=64)
    assert torch.equal(q1, q2)


def test_chunkwise_state_and_workspace_sizes():
    """The size queries are host arithmetic on the chunk-wise plan (no GPU): values derived by hand.
    State = what forward hands to backward: the fp32 entry state of every walk segment plus the final
    state, or, if larger, the 16-bit states of the chunks (D <= 64: per 128-row chunk, what the
    normalised operator hands over; D = 128: of the 256-row chunks) plus an fp32 vector of D per chunk for the normalised operator."""
    lib = _lib.load()
    sb = lib.fla_linear_attn_chunked_state_bytes
    # B H = 128, N = 4096, D = 128: 16 chunks of 256 rows x 32 KiB > 2 segments x 64 KiB; 64 chunks of 64 rows
    assert sb(4, 32, 4096, 128, 128) == 128 * 16 * 128 * 128 * 2 + 128 * 64 * 128 * 4
    # B H = 16, N = 32768, D = 64: 256 chunks of 128 rows
    assert sb(1, 16, 32768, 64, 64) == 16 * 256 * 64 * 64 * 2 + 16 * 256 * 64 * 4
    # ragged: N = 2450 at D = 128 is 39 chunks of 64 rows in 13 walk segments of 3 (16 segments per (b, h) would
    # fill the chip; their entry states, and the state after the last chunk); ten 256-row chunks are less
    assert sb(2, 8, 2450, 128, 128) == 16 * 14 * 128 * 128 * 4 + 16 * 39 * 128 * 4
    # three single-chunk segments at D = 32: their fp32 entry states and the final state outweigh three 16-bit states
    assert sb(1, 1, 300, 32, 32) == 4 * 32 * 32 * 4 + 3 * 32 * 4
    # D_qk = 256, D_v = 64: the fp32 entry states of both 128-column halves, 4 walk segments per (b, h), and their
    # states after the last chunk
    assert sb(4, 16, 4096, 256, 64) == 2 * 64 * 5 * 128 * 128 * 4
    # D_v = 256 against D_qk = 64: the two column halves of v, each a 64 / 128 problem on the D = 128 walks (4 segments)
    assert sb(4, 16, 4096, 64, 256) == 2 * 64 * 5 * 128 * 128 * 4
    # padded widths that differ run at the larger one: 128 / 64 as D = 128, 64 / 32 as D = 64 (room for 32 chunk states)
    assert sb(4, 16, 4096, 128, 64) == 64 * 5 * 128 * 128 * 4 and sb(4, 16, 4096, 64, 32) == 64 * 32 * 64 * 64 * 2
    # nothing to hand over: a single chunk
    assert sb(1, 2, 256, 128, 128) == 0 and sb(1, 2, 128, 64, 64) == 0 and sb(1, 2, 256, 64, 256) == 0
    ws = lib.fla_linear_attn_chunked_workspace_bytes
    for shape in [(4, 32, 4096, 128, 128), (1, 16, 32768, 64, 64), (2, 8, 2450, 128, 128), (1, 4, 1500, 104, 120)]:
        assert ws(*shape) >= 4 * (sb(*shape) - shape[0] * shape[1] * 4)  # room for the 256-row path's four buffers
        assert lib.fla_normalised_workspace_bytes(*shape, 1) > ws(*shape)
    assert ws(4, 16, 4096, 256, 64) > 0 and ws(4, 16, 4096, 64, 256) > 0 and ws(1, 2, 256, 128, 128) == 0


def test_algorithm_table():
    """fla_linear_attn_prefers_chunked is host arithmetic on measured thresholds: the benchmark workloads
    with long sequences go chunk-wise, short or single-chunk problems stay with the quadratic kernels,
    and the answer grows monotonically with the sequence length."""
    pick = _lib.load().fla_linear_attn_prefers_chunked
    assert pick(4, 32, 4096, 128, 128) == 1 and pick(1, 16, 32768, 64, 64) == 1 and pick(4, 16, 4096, 256, 64) == 1
    assert pick(1, 2, 256, 64, 64) == 0 and pick(1, 16, 1024, 64, 64) == 0 and pick(1, 128, 512, 128, 128) == 0
    assert pick(1, 128, 1024, 128, 128) == 1 and pick(1, 512, 512, 64, 64) == 1
    assert pick(1, 16, 256, 256, 64) == 0 and pick(1, 64, 512, 256, 64) == 1 and pick(1, 64, 2048, 256, 64) == 1
    assert pick(1, 16, 2048, 256, 256) == 0 and pick(1, 16, 4096, 256, 256) == 1 and pick(1, 64, 2048, 256, 256) == 1
    assert pick(1, 16, 512, 128, 64) == 1 and pick(1, 16, 512, 64, 32) == 0 and pick(1, 16, 1024, 64, 32) == 1
    assert pick(1, 16, 1024, 192, 128) == 0 and pick(1, 16, 2048, 192, 128) == 1 and pick(1, 128, 512, 192, 128) == 0
    assert pick(0, 4, 4096, 64, 64) == 0 and pick(1, 4, 4096, 300, 64) == 0
    for shape in [(1, 16, 64, 64), (2, 8, 128, 128), (1, 64, 256, 64), (1, 4, 192, 128), (1, 8, 256, 256)]:
        b, h, dqk, dv = shape
        answers = [pick(b, h, n, dqk, dv) for n in (256, 512, 1024, 2048, 4096, 8192, 16384, 32768)]
        assert answers == sorted(answers) and answers[-1] == 1
