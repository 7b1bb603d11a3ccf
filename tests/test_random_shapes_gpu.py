"""Seeded sweep over shapes the fixed grids do not hit: arbitrary N (the C ABI accepts any
length, the reference-named Python wrappers do not), head counts that are not multiples of 8,
every pairing of widths, both masks, both dtypes -- through the raw C ABI, against the CPU
oracle (``-m gpu``)."""

import ctypes
import random

import pytest
import torch

from flashy_linear_attention_amd import _lib
from oracle import naive

from helpers import assert_close

pytestmark = pytest.mark.gpu

_CODE = {torch.bfloat16: 0, torch.float16: 1}


def _cases(seed: int, count: int):
    rng = random.Random(seed)
    widths8 = [8, 16, 24, 32, 40, 64, 72, 96, 128, 136, 200, 256]
    out = []
    for i in range(count):
        b, h = rng.choice([1, 1, 2, 3]), rng.choice([1, 2, 3, 5, 7, 9])
        n = rng.choice([1, 2, 31, 33, 63, 65, 100, 127, 129, 255, 257, 300, 511, 513, 640, 777])
        if i % 4 == 3:  # widths that are not multiples of 8: the bounds-checked generic kernel
            dc, do = rng.randint(1, 140), rng.randint(1, 140)
        else:
            dc, do = rng.choice(widths8), rng.choice(widths8)
        out.append((b, h, n, dc, do, rng.randint(0, 1), rng.choice([torch.bfloat16, torch.float16]), 1000 + i))
    return out


def _inputs(b, h, n, dc, do, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.rand(b, h, n, dc, generator=g) + 0.05) / dc ** 0.5
    y = torch.rand(b, h, n, dc, generator=g) + 0.05
    z = torch.randn(b, h, n, do, generator=g)
    return tuple(t.to(dtype) for t in (x, y, z))


def _oracle(x, y, z, upper):
    """mask(X Y^T) Z; the upper mask is the lower one on the reversed sequence."""
    x, y, z = x.float(), y.float(), z.float()
    if upper:
        return naive.causal_dot_product(x.flip(-2), y.flip(-2), z.flip(-2)).flip(-2)
    return naive.causal_dot_product(x, y, z)


def _call(name, x, y, z, upper, chunked):
    lib = _lib.load()
    b, h, n, dc = x.shape
    do = z.shape[-1]
    out = torch.full((b, h, n, do), float("nan"), dtype=x.dtype, device=x.device)
    st = _lib.strides_arg
    stream = torch.cuda.current_stream().cuda_stream
    if chunked:
        nbytes = lib.fla_chunked_workspace_bytes(b, h, n, dc, do)
        work = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        rc = lib.fla_tri_xyt_z_chunked(x.data_ptr(), y.data_ptr(), z.data_ptr(), out.data_ptr(), b, h, n, dc, do,
                                       st(x), st(y), st(z), st(out), int(upper), _CODE[x.dtype], work.data_ptr(),
                                       nbytes, stream)
    else:
        rc = lib.fla_tri_xyt_z(x.data_ptr(), y.data_ptr(), z.data_ptr(), out.data_ptr(), b, h, n, dc, do,
                               st(x), st(y), st(z), st(out), int(upper), _CODE[x.dtype], stream)
    assert rc == 0, (name, lib.fla_strerror(rc))
    return out


@pytest.mark.parametrize("case", _cases(7, 36), ids=lambda c: "b%d_h%d_n%d_c%d_o%d_u%d_%s" % (c[:6] + (str(c[6])[6:],)))
def test_primitive_on_arbitrary_shapes(case, gpu_device):
    b, h, n, dc, do, upper, dtype, seed = case
    x, y, z = _inputs(b, h, n, dc, do, dtype, seed)
    want = _oracle(x, y, z, upper)
    xg, yg, zg = (t.to(gpu_device) for t in (x, y, z))
    assert_close("quadratic", _call("tri", xg, yg, zg, upper, chunked=False), want)
    assert_close("chunked", _call("tri_chunked", xg, yg, zg, upper, chunked=True), want)


@pytest.mark.parametrize("dims", [(2, 3, 333, 64), (1, 5, 700, 128), (1, 2, 257, 40), (3, 1, 65, 96), (1, 7, 1, 32)],
                         ids=lambda d: "x".join(map(str, d)))
def test_backward_entry_point_on_ragged_lengths(dims, gpu_device):
    """fla_linear_attn_bwd (the three products in one launch) and the chunk-wise operator with N
    that is no multiple of any tile, against the oracle's closed-form gradients."""
    lib = _lib.load()
    b, h, n, d = dims
    g = torch.Generator().manual_seed(sum(dims))
    q = ((torch.rand(b, h, n, d, generator=g) + 0.05) / d ** 0.5).bfloat16()
    k = (torch.rand(b, h, n, d, generator=g) + 0.05).bfloat16()
    v = torch.randn(b, h, n, d, generator=g).bfloat16()
    do = torch.randn(b, h, n, d, generator=g).bfloat16()
    want = naive.causal_dot_product_grads(q.float(), k.float(), v.float(), do.float())
    qg, kg, vg, dog = (t.to(gpu_device) for t in (q, k, v, do))
    st = _lib.strides_arg
    stream = torch.cuda.current_stream().cuda_stream
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (qg, kg, vg))
    rc = lib.fla_linear_attn_bwd(dog.data_ptr(), qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), dq.data_ptr(),
                                 dk.data_ptr(), dv.data_ptr(), b, h, n, d, st(dog), st(qg), st(kg), st(vg), st(dq),
                                 st(dk), st(dv), 0, stream)
    assert rc == 0
    for name, got, w in zip(("dQ", "dK", "dV"), (dq, dk, dv), want):
        assert_close(name, got, w)
    # chunk-wise operator, forward state handed to backward when the shape allows it
    o = torch.full_like(vg, float("nan"))
    sbytes = lib.fla_linear_attn_chunked_state_bytes(b, h, n, d, d)
    wbytes = lib.fla_linear_attn_chunked_workspace_bytes(b, h, n, d, d)
    state = torch.empty(max(sbytes, 16), dtype=torch.uint8, device=gpu_device)
    work = torch.empty(max(wbytes, 16), dtype=torch.uint8, device=gpu_device)
    valid = ctypes.c_int32(0)
    rc = lib.fla_linear_attn_chunked_fwd(qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), o.data_ptr(), b, h, n, d, d,
                                         st(qg), st(kg), st(vg), st(o), 0, state.data_ptr() if sbytes else None,
                                         ctypes.byref(valid), work.data_ptr(), wbytes, stream)
    assert rc == 0 and valid.value == (1 if sbytes else 0)
    assert_close("O (chunked)", o, naive.causal_dot_product(q.float(), k.float(), v.float()))
    dq, dk, dv = (torch.full_like(t, float("nan")) for t in (qg, kg, vg))
    rc = lib.fla_linear_attn_chunked_bwd(dog.data_ptr(), qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), dq.data_ptr(),
                                         dk.data_ptr(), dv.data_ptr(), b, h, n, d, d, st(dog), st(qg), st(kg), st(vg),
                                         st(dq), st(dk), st(dv), 0, state.data_ptr() if valid.value else None,
                                         work.data_ptr(), wbytes, stream)
    assert rc == 0
    for name, got, w in zip(("dQ", "dK", "dV"), (dq, dk, dv), want):
        assert_close(name + " (chunked)", got, w)


@pytest.mark.parametrize("dims", [(1, 64, 2300, 64, 64), (2, 26, 2300, 128, 128), (1, 64, 1990, 32, 64)],
                         ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("upper", [0, 1], ids=["lower", "upper"])
def test_paired_row_tiles_on_ragged_lengths(dims, upper, gpu_device):
    """Enough (head, tile-pair) work for one workgroup to take two row tiles (the second tile's
    first loads overlap the first tile's epilogue), with an odd tile count (the middle tile has
    no partner) and a last tile that is cut short.  Every head against the formula in fp32 on
    the GPU, four heads against the CPU oracle."""
    b, h, n, dc, do = dims
    x, y, z = _inputs(b, h, n, dc, do, torch.bfloat16, seed=sum(dims) + upper)
    xg, yg, zg = (t.to(gpu_device) for t in (x, y, z))
    got = _call("tri", xg, yg, zg, upper, chunked=False)
    s = torch.matmul(xg.float(), yg.float().transpose(-2, -1))
    s = s.triu() if upper else s.tril()
    assert_close("all heads (fp32 GPU)", got, torch.matmul(s, zg.float()).cpu())
    heads = [0, h // 3, h // 2, h - 1]
    want = _oracle(x[-1:, heads], y[-1:, heads], z[-1:, heads], upper)
    assert_close("sampled heads (CPU oracle)", got[-1:, heads], want)


@pytest.mark.parametrize("dims", [(8, 40, 300, 64, 64), (5, 13, 520, 128, 128), (4, 80, 257, 32, 32)],
                         ids=lambda d: "x".join(map(str, d)))
@pytest.mark.parametrize("upper", [0, 1], ids=["lower", "upper"])
def test_many_heads_short_sequences(dims, upper, gpu_device):
    """Many heads, few row tiles each: single-tile workgroups ordered heaviest first across heads,
    head counts that are no multiple of 8 (idle slots in the last group of eight)."""
    b, h, n, dc, do = dims
    x, y, z = _inputs(b, h, n, dc, do, torch.float16, seed=sum(dims) + upper)
    want = _oracle(x, y, z, upper)
    xg, yg, zg = (t.to(gpu_device) for t in (x, y, z))
    assert_close("quadratic", _call("tri", xg, yg, zg, upper, chunked=False), want)
    assert_close("chunked", _call("tri_chunked", xg, yg, zg, upper, chunked=True), want)
