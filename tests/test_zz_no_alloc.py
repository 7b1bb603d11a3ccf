"""fla_linear_attn_chunked_fwd_static (scratch in a static device array, nothing allocated)
against fla_linear_attn_chunked_fwd (caller-owned workspace), through the C ABI: same kernels,
so the outputs must be bit-identical; two calls in a row, the second on a smaller problem, so
that what the first call left in the shared array is seen to do no harm."""

import ctypes

import pytest
import torch

from flashy_linear_attention_amd import _lib
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
from oracle import naive

from helpers import assert_close

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 * 1024 * 1024  # FLA_STATIC_SCRATCH_BYTES in include/fla.h


def _st(t):
    return (ctypes.c_int64 * 4)(*t.stride())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _with_workspace(lib, q, k, v):
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    out = torch.empty_like(v)
    nbytes = lib.fla_linear_attn_chunked_workspace_bytes(b, h, n, dqk, dv)
    work = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
    rc = lib.fla_linear_attn_chunked_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b, h, n, dqk, dv,
                                         _st(q), _st(k), _st(v), _st(out), 0, None, None, work.data_ptr(), nbytes,
                                         _stream())
    assert rc == 0, lib.fla_strerror(rc)
    return out, nbytes


def _static(lib, q, k, v, out):
    b, h, n, dqk = q.shape
    dv = v.shape[-1]
    return lib.fla_linear_attn_chunked_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), b, h, n,
                                                  dqk, dv, _st(q), _st(k), _st(v), _st(out), 0, _stream())


def test_static_scratch_entry_point_matches_the_workspace_one(gpu_device):
    lib = _lib.load()
    w = WORKLOADS["C5"]  # D = 64: the scratch holds the segments' totals and entry states
    # first a problem of many chunks, then a smaller one whose states land on the first one's
    for case, (heads, seq) in enumerate(((6, 4096), (3, 1280))):
        q, k, v, _ = (t.to(gpu_device) for t in make_inputs(w, seed=11 + case, batch=1, heads=heads, seq=seq))
        want, nbytes = _with_workspace(lib, q, k, v)
        assert 0 < nbytes <= STATIC_BYTES, "the case must exercise the scratch array"
        out = torch.full_like(v, float("nan"))
        before = torch.cuda.memory_allocated()
        rc = _static(lib, q, k, v, out)
        assert rc == 0, lib.fla_strerror(rc)
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"case {case}: static-scratch result differs from the workspace one"
        ref = naive.causal_dot_product(q.float().cpu(), k.float().cpu(), v.float().cpu())
        assert_close(f"O (case {case})", out, ref)


def test_static_scratch_entry_point_rejects_what_does_not_fit(gpu_device):
    """Rows that are not 16-byte aligned take the 256-row chunks, whose states (about 200 MB at this
    size) do not fit the array; the same size with aligned rows needs 16 MiB of entry states and runs
    (first case of the test above at a smaller size, and the benchmark shape below)."""
    lib = _lib.load()
    b, h, n, d = 4, 32, 4096, 128
    assert lib.fla_chunked_workspace_bytes(b, h, n, d, d) > STATIC_BYTES
    q = torch.zeros(1, 1, 64, d, dtype=torch.bfloat16, device=gpu_device)  # never read: the call is refused first
    rs = d + 1  # row stride in elements: rows start at odd multiples of 2 bytes
    s = (ctypes.c_int64 * 4)(h * n * rs, n * rs, rs, 1)
    fake = [ctypes.c_void_p(q.data_ptr() + (i << 32)) for i in range(4)]
    rc = lib.fla_linear_attn_chunked_fwd_static(*fake, b, h, n, d, d, s, s, s, s, 0, _stream())
    assert rc == -9, lib.fla_strerror(rc)
    torch.cuda.synchronize()


def test_static_scratch_entry_point_at_the_benchmark_shape(gpu_device):
    """B 4, H 32, N 4096, D 128: two segments per (b, h), 16 MiB of the array."""
    from helpers import reference_style_inputs

    lib = _lib.load()
    q, k, v, _ = (t.to(gpu_device) for t in reference_style_inputs(4, 32, 4096, 128, 128, torch.bfloat16, seed=97))
    want, _ = _with_workspace(lib, q, k, v)
    out = torch.full_like(v, float("nan"))
    before = torch.cuda.memory_allocated()
    rc = _static(lib, q, k, v, out)
    assert rc == 0, lib.fla_strerror(rc)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_static_scratch_entry_point_at_other_widths(gpu_device):
    """D = 128 (two sets of tiles) and D_qk = 256 / D_v = 64 (two halves, the second adding to the
    first one's results), after the calls above have used the array."""
    from helpers import reference_style_inputs

    lib = _lib.load()
    # (the last one: two segments per (b, h), whose entry states the totals kernel writes itself)
    for case, dims in enumerate(((1, 4, 2048, 128, 128), (1, 2, 1024, 256, 64), (1, 3, 700, 128, 128), (1, 200, 900, 64, 64))):
        q, k, v, _ = (t.to(gpu_device) for t in reference_style_inputs(*dims, torch.bfloat16, seed=90 + case))
        want, nbytes = _with_workspace(lib, q, k, v)
        assert 0 < nbytes <= STATIC_BYTES
        out = torch.full_like(v, float("nan"))
        before = torch.cuda.memory_allocated()
        rc = _static(lib, q, k, v, out)
        assert rc == 0, lib.fla_strerror(rc)
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"{dims}: static-scratch result differs from the workspace one"
