"""Chunk-wise evaluation (fla_tri_xyt_z_chunked) against the CPU oracle and against the
quadratic kernels (``-m gpu``)."""

import math

import pytest
import torch

from flashy_linear_attention_amd import LinearAttention, LinearAttentionChunked, LinearAttentionSmallVHD
from flashy_linear_attention_amd.chunked import tri_xyt_z_chunked
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
from oracle import naive

from helpers import assert_close, reference_style_inputs

pytestmark = pytest.mark.gpu

# (batch, heads, seq, d_qk, d_v): one chunk (falls through to the quadratic kernel), exact
# multiples of the 256- and 128-row chunks, ragged last chunks, both chunk sizes, wide outputs
CASES = [
    (1, 2, 256, 64, 64),
    (1, 3, 512, 64, 64),
    (2, 2, 1024, 128, 128),
    (1, 2, 1984, 128, 128),
    (1, 2, 832, 64, 32),
    (1, 2, 768, 256, 64),
    (1, 2, 640, 64, 256),
    (1, 1, 512, 128, 256),
    (1, 2, 576, 48, 48),
    (1, 1, 1024, 32, 32),
    # several chunks per walking workgroup with a ragged last segment: D = 128 with segments of three and
    # of five chunks, padded widths, and D = 64
    (2, 8, 2450, 128, 128),
    (2, 8, 4136, 128, 128),
    (1, 4, 1500, 104, 120),
    (8, 8, 2100, 64, 64),
    # D_qk in (128, 256] with D_v <= 128: two 128-column halves of q and k through the D = 128 walk kernels
    (2, 4, 1300, 256, 64),
    (1, 2, 1024, 200, 128),
    (2, 8, 2450, 136, 24),
    # (a second half of at most 64 columns against a v wider than 64: the forward walk built for a narrow q / k side)
    (1, 3, 1100, 160, 96),
    # a B H that leaves no room for a second segment per (b, h) among the workgroups that run at once: one segment
    (2, 80, 320, 128, 128),
    (4, 80, 640, 64, 64),
    # two segments per (b, h): the totals kernel writes the entry states itself, half a segment per workgroup (three
    # chunks: two and one), and the walks add the two partial sums; padded widths, a wide q / k, D = 64
    (1, 100, 330, 128, 128),
    (2, 50, 330, 104, 120),
    (1, 100, 330, 128, 72),
    (1, 100, 330, 256, 64),
    (2, 100, 1024, 64, 64),
    (2, 100, 900, 64, 64),
    # three and four segments per (b, h)
    (1, 72, 512, 128, 128),
    (1, 64, 1024, 128, 128),
    (1, 72, 512, 256, 64),
    (1, 160, 1500, 64, 64),
    # a wide q / k in one walk over both halves, with segment totals that the walks add up themselves: six segments
    # (two groups of loads for the late ones), four with a second half of 32 columns, and a v wider than 64
    # (one forward walk, two reverse walks)
    (1, 40, 700, 200, 48),
    (3, 20, 900, 160, 64),
    (1, 40, 700, 256, 96),
    # a v wider than 128 columns as two column halves: over the walks for a wide q / k (256 / 256, a second half of
    # 8 columns, 200 / 200) and over the D = 128 walks (128 / 256, 96 / 200)
    (2, 8, 1300, 256, 256),
    (1, 5, 900, 256, 136),
    (1, 64, 640, 200, 200),
    (1, 3, 1100, 128, 256),
    (1, 40, 700, 96, 200),
    # padded widths that differ, on the walk kernels at the larger one (the small-V operator's shapes among them)
    (2, 8, 1300, 128, 64),
    (1, 40, 700, 128, 32),
    (1, 5, 900, 64, 128),
    (2, 8, 1300, 64, 32),
    (1, 70, 600, 32, 64),
    (1, 3, 1100, 24, 128),
    (1, 6, 1000, 64, 256),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dims", CASES, ids=lambda d: "x".join(map(str, d)))
def test_chunked_fwd_bwd_vs_oracle(dims, dtype, gpu_device):
    bs, nh, sq, dqk, dv = dims
    q, k, v, dy = reference_style_inputs(bs, nh, sq, dqk, dv, dtype, seed=sum(dims))
    want_o = naive.causal_dot_product(q.float(), k.float(), v.float())
    want_g = naive.causal_dot_product_grads(q.float(), k.float(), v.float(), dy.float())
    qg, kg, vg = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionChunked.apply(qg, kg, vg)
    assert out.dtype == dtype and out.shape == v.shape
    out.backward(dy.to(gpu_device))
    assert_close("O", out, want_o)
    for name, got, want in (("dQ", qg.grad, want_g[0]), ("dK", kg.grad, want_g[1]), ("dV", vg.grad, want_g[2])):
        assert_close(name, got, want)


def test_chunked_matches_quadratic_closely(gpu_device):
    """Same inputs through both algorithms: they differ only by the rounding of the running
    state, far inside the tolerance against the oracle."""
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(2, 4, 2048, 128, 128, torch.bfloat16, seed=21))
    a = LinearAttention.apply(q, k, v)
    b = LinearAttentionChunked.apply(q, k, v)
    assert_close("chunked vs quadratic", b, a.float(), tol_fro=5e-3, tol_max=1e-2)
    q2, k2, v2, _ = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 1024, 256, 64, torch.bfloat16, seed=22))
    assert_close("small-V", LinearAttentionChunked.apply(q2, k2, v2), LinearAttentionSmallVHD.apply(q2, k2, v2).float(),
                 tol_fro=5e-3, tol_max=1e-2)


def test_chunked_upper_mask_and_unaligned_fallback(gpu_device):
    x, y, z, _ = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 768, 64, 64, torch.bfloat16, seed=23))
    want = torch.matmul(torch.triu(torch.matmul(x.float().cpu(), y.float().cpu().transpose(-1, -2))), z.float().cpu())
    assert_close("upper", tri_xyt_z_chunked(x, y, z, upper=True), want)
    # width 50 is not a multiple of 8: evaluated by the quadratic generic kernel, same answer
    x2, y2, z2, _ = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 512, 50, 50, torch.bfloat16, seed=24))
    want2 = naive.causal_dot_product(x2.float().cpu(), y2.float().cpu(), z2.float().cpu())
    assert_close("unaligned", tri_xyt_z_chunked(x2, y2, z2, upper=False), want2)


def test_chunked_long_context_workload(gpu_device):
    """C5 (N = 32768, D = 64, bf16) forward + backward through the chunked path; four heads
    against the oracle formula in fp32 on the GPU."""
    w = WORKLOADS["C5"]
    q, k, v, do = (t.to(gpu_device) for t in make_inputs(w, heads=4))
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionChunked.apply(qg, kg, vg)
    out.backward(do)
    for hh in range(4):
        sl = (slice(0, 1), slice(hh, hh + 1))
        qs, ks, vs, ds = (t[sl].float() for t in (q, k, v, do))
        assert_close(f"O head {hh}", out[sl], naive.causal_dot_product_blocked(qs, ks, vs, block=2048))
        for name, got, want in zip(("dQ", "dK", "dV"), (qg.grad, kg.grad, vg.grad),
                                   naive.causal_dot_product_grads_blocked(qs, ks, vs, ds, block=2048)):
            assert_close(f"{name} head {hh}", got[sl], want)


def test_chunked_workspace_errors(gpu_device):
    from flashy_linear_attention_amd import _lib

    lib = _lib.load()
    x = torch.zeros(1, 1, 1024, 64, dtype=torch.bfloat16, device=gpu_device)
    out = torch.empty_like(x)
    need = lib.fla_chunked_workspace_bytes(1, 1, 1024, 64, 64)
    assert need == 1 * 1 * 4 * 64 * 64 * 6
    assert lib.fla_chunked_workspace_bytes(1, 1, 256, 64, 64) == 0  # a single chunk needs none
    st = _lib.strides_arg(x)
    small = torch.empty(need - 16, dtype=torch.uint8, device=gpu_device)
    rc = lib.fla_tri_xyt_z_chunked(x.data_ptr(), x.data_ptr(), x.data_ptr(), out.data_ptr(), 1, 1, 1024, 64, 64,
                                   st, st, st, st, 0, 0, small.data_ptr(), need - 16, None)
    assert rc == -9 and b"workspace" in lib.fla_strerror(rc)
    rc = lib.fla_tri_xyt_z_chunked(x.data_ptr(), x.data_ptr(), x.data_ptr(), out.data_ptr(), 1, 1, 1024, 64, 64,
                                   st, st, st, st, 0, 0, None, 0, None)
    assert rc == -9


@pytest.mark.parametrize("dims", [(2, 3, 1280, 128, 128), (1, 100, 330, 128, 128), (1, 100, 330, 256, 64), (1, 72, 512, 128, 128),
                                  (2, 100, 900, 64, 64), (1, 40, 700, 200, 48), (1, 40, 700, 256, 96),
                                  (2, 8, 1300, 256, 256), (1, 3, 1100, 128, 256), (2, 8, 1300, 128, 64), (2, 8, 1300, 64, 32),
                                  (1, 5, 900, 64, 128)],
                         ids=lambda d: "x".join(map(str, d)))
def test_chunked_backward_with_and_without_the_forward_state(dims, gpu_device):
    """Backward given what the forward pass saved, and backward without it (D = 128: two walks from entry
    states it forms again; below: the 256-row chunks with states of their own), both match the oracle -- on
    plans of many, two and three segments per (b, h); shapes that cannot share a state report none."""
    from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd

    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(*dims, torch.bfloat16, seed=31))
    out, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
    assert state is not None
    plain = linear_attention_chunked_fwd(q, k, v)
    assert torch.equal(out, plain)
    with_state = linear_attention_chunked_bwd(dy, q, k, v, state)
    without = linear_attention_chunked_bwd(dy, q, k, v, None)
    want = naive.causal_dot_product_grads(q.float().cpu(), k.float().cpu(), v.float().cpu(), dy.float().cpu())
    for name, got, other, w in zip(("dQ", "dK", "dV"), with_state, without, want):
        assert_close(name, got, w)
        assert_close(name + " (no saved state)", other, w)
    if dims != (2, 3, 1280, 128, 128):
        return
    # rows that do not meet the alignment rules of the walk kernels (product by product then), and a single chunk:
    # no shared state
    q2, k2, v2, _ = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 1024, 64, 264, torch.bfloat16, seed=32))
    assert linear_attention_chunked_fwd(q2, k2, v2[..., 4:260], want_state=True)[1] is None
    assert linear_attention_chunked_fwd(q[:, :, :256], k[:, :, :256], v[:, :, :256], want_state=True)[1] is None


@pytest.mark.parametrize("dims", [(64, 64), (128, 128), (256, 64)])
def test_chunked_backward_when_late_rows_dwarf_early_ones(dims, gpu_device):
    """The backward walk forms dQ's state -- the sum of K^T V over the chunks BEFORE -- by subtracting
    chunks from the forward state at the end of a segment, in fp32.  Its error
    is a rounding of the LARGEST state, so rows whose own state is much smaller are where it would
    show: k and v grow by a factor of 64 over the sequence (4096 in their products), and the first
    quarter of the rows of every gradient is held to the usual tolerance on its own."""
    from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd

    dqk, dv = dims
    n = 2048
    q, k, v, dy = reference_style_inputs(1, 4, n, dqk, dv, torch.bfloat16, seed=77)
    ramp = torch.logspace(0, math.log10(64.0), n).view(1, 1, n, 1)
    k = (k.float() * ramp).to(torch.bfloat16)
    v = (v.float() * ramp).to(torch.bfloat16)
    want = naive.causal_dot_product_grads(q.float(), k.float(), v.float(), dy.float())
    q, k, v, dy = (t.to(gpu_device) for t in (q, k, v, dy))
    out, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
    assert state is not None
    got = linear_attention_chunked_bwd(dy, q, k, v, state)
    for name, g, w in zip(("dQ", "dK", "dV"), got, want):
        assert_close(name, g, w)
        assert_close(name + ", first quarter of the rows", g[:, :, : n // 4], w[:, :, : n // 4])


def test_chunked_operator_workspace_is_checked(gpu_device):
    import ctypes

    from flashy_linear_attention_amd import _lib

    lib = _lib.load()
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(1, 2, 1024, 64, 64, torch.bfloat16, seed=2))
    out = torch.empty_like(v)
    st = _lib.strides_arg
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.fla_linear_attn_chunked_workspace_bytes(1, 2, 1024, 64, 64)
    sbytes = lib.fla_linear_attn_chunked_state_bytes(1, 2, 1024, 64, 64)
    # the fp32 entry state of each of the eight single-chunk segments and the final state, per head (more than
    # the normalised operator's 16-bit state per 128-row chunk), and an fp32 vector per chunk
    assert need > 0 and sbytes == 2 * 9 * 64 * 64 * 4 + 2 * 8 * 64 * 4
    # D = 128: the fp32 entry state of every segment (here single 64-row chunks) and the state after the
    # last chunk, which is more than a 16-bit state per 256-row chunk
    assert lib.fla_linear_attn_chunked_state_bytes(1, 2, 1024, 128, 128) == 2 * 17 * 128 * 128 * 4 + 2 * 16 * 128 * 4
    valid = ctypes.c_int32(7)
    rc = lib.fla_linear_attn_chunked_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), 1, 2, 1024, 64, 64,
                                         st(q), st(k), st(v), st(out), 0, None, ctypes.byref(valid), None, 0, stream)
    assert rc == -9 and valid.value == 0
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    work = torch.empty(need, dtype=torch.uint8, device=gpu_device)
    rc = lib.fla_linear_attn_chunked_bwd(dy.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), dq.data_ptr(),
                                         dk.data_ptr(), dv.data_ptr(), 1, 2, 1024, 64, 64, st(dy), st(q), st(k), st(v),
                                         st(dq), st(dk), st(dv), 0, None, work.data_ptr(), 3 * sbytes, stream)
    assert rc == -9  # without a saved state the call needs room for four
    torch.cuda.synchronize()


@pytest.mark.parametrize("dims", [(2, 4, 1664, 64, 64), (2, 4, 1664, 128, 128), (1, 3, 1100, 40, 56)],
                         ids=lambda d: "x".join(map(str, d)))
def test_chunked_on_strided_operands(dims, gpu_device):
    """(B, N, H, D) storage viewed as (B, H, N, D), and rows padded to a wider pitch: the chunk-wise
    kernels honour every operand's own strides, so the results equal those on contiguous copies bit
    for bit (outputs and gradients come back contiguous either way)."""
    from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd

    bs, nh, sq, dqk, dv = dims
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=5))

    def bnhd(t):
        return t.transpose(1, 2).contiguous().transpose(1, 2)

    def pitched(t):
        wide = torch.zeros(*t.shape[:-1], t.shape[-1] + 24, dtype=t.dtype, device=t.device)
        wide[..., : t.shape[-1]] = t
        return wide[..., : t.shape[-1]]

    want_o, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
    want_g = linear_attention_chunked_bwd(dy, q, k, v, state)
    for name, f in (("(B, N, H, D) storage", bnhd), ("padded rows", pitched)):
        qs, ks, vs, ds = f(q), f(k), f(v), f(dy)
        assert not qs.is_contiguous()
        out, st = linear_attention_chunked_fwd(qs, ks, vs, want_state=True)
        assert torch.equal(out, want_o), f"{name}: O differs"
        for gname, g, w in zip(("dQ", "dK", "dV"), linear_attention_chunked_bwd(ds, qs, ks, vs, st), want_g):
            assert torch.equal(g, w), f"{name}: {gname} differs"


def test_chunked_small_v_state_hand_over(gpu_device):
    """D_qk = 256, D_v = 64: forward hands both halves' states to backward; backward without them
    recomputes the entry states and takes the two-walk path; both match the oracle."""
    from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd

    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(2, 8, 4200, 256, 64, torch.bfloat16, seed=41))
    out, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
    assert state is not None and torch.equal(out, linear_attention_chunked_fwd(q, k, v))
    assert_close("O", out, naive.causal_dot_product(q.float().cpu(), k.float().cpu(), v.float().cpu()))
    want = naive.causal_dot_product_grads(q.float().cpu(), k.float().cpu(), v.float().cpu(), dy.float().cpu())
    with_state = linear_attention_chunked_bwd(dy, q, k, v, state)
    without = linear_attention_chunked_bwd(dy, q, k, v, None)
    # (with the states: one reverse walk over both halves; without: per half, dQ's forward-direction walk and the dK / dV walk)
    for name, a, b, w in zip(("dQ", "dK", "dV"), with_state, without, want):
        assert_close(name, a, w)
        assert_close(name + " (no saved state)", b, w)


@pytest.mark.parametrize("dims", [(1, 2, 256, 64, 64, 0), (1, 16, 4096, 64, 64, 1), (1, 2, 1000, 128, 128, 0),
                                  (1, 32, 2048, 256, 64, 1), (1, 2, 512, 256, 64, 0), (1, 2, 384, 160, 96, 0)],
                         ids=lambda d: "x".join(map(str, d)))
def test_auto_operator_picks_an_evaluation_and_matches_the_oracle(dims, gpu_device):
    """LinearAttentionAuto: quadratic kernels for the short shapes, chunk-wise for the long ones and
    for what the quadratic wrappers refuse (N not a multiple of 64, a value head dim that is no power
    of two); same function either way."""
    from flashy_linear_attention_amd import LinearAttentionAuto
    from flashy_linear_attention_amd.auto import prefers_chunked

    b, h, n, dqk, dv, chunked = dims
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(b, h, n, dqk, dv, torch.bfloat16, seed=91))
    assert prefers_chunked(q, v) == bool(chunked)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    out = LinearAttentionAuto.apply(q, k, v)
    got = torch.autograd.grad(out, (q, k, v), dy)
    qc, kc, vc = (t.detach().float().cpu() for t in (q, k, v))
    assert_close("O", out.detach(), naive.causal_dot_product(qc, kc, vc))
    for name, g, w in zip(("dQ", "dK", "dV"), got, naive.causal_dot_product_grads(qc, kc, vc, dy.float().cpu())):
        assert_close(name, g, w)
