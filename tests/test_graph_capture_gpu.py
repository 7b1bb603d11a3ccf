"""The entry points only enqueue kernels on the caller's stream (no allocation, no
synchronisation, no memset), so a caller may record them into a HIP graph.  Forward and
backward of both operators are captured once and replayed several times on fresh input
contents, with eager work between the replays; every replay must equal the eager result bit
for bit (``-m gpu``)."""

import pytest
import torch

from flashy_linear_attention_amd.kernels import (
    linear_flash_wrapper_bwd,
    linear_flash_wrapper_bwd_smallv_hd,
    linear_flash_wrapper_fwd,
    linear_flash_wrapper_fwd_smallv_hd,
)

from helpers import reference_style_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dims,fwd,bwd", [
    ((2, 4, 1024, 64, 64), linear_flash_wrapper_fwd, linear_flash_wrapper_bwd),
    ((1, 8, 2048, 128, 128), linear_flash_wrapper_fwd, linear_flash_wrapper_bwd),
    ((2, 4, 1024, 256, 64), linear_flash_wrapper_fwd_smallv_hd, linear_flash_wrapper_bwd_smallv_hd),
], ids=["d64", "d128", "smallv"])
def test_replayed_graph_equals_eager(dims, fwd, bwd, gpu_device):
    bs, nh, sq, dqk, dv = dims
    static = [t.to(gpu_device) for t in reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=0)]
    q, k, v, do = static
    # warm-up on a side stream, as graph capture requires
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fwd(q, k, v)
            bwd(do, q, k, v)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out = fwd(q, k, v)
        g_dq, g_dk, g_dv = bwd(do, q, k, v)
    for replay in range(3):
        fresh = [t.to(gpu_device) for t in reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=10 + replay)]
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        # eager work between replays, on the same inputs
        want_out = fwd(q, k, v)
        want = bwd(do, q, k, v)
        torch.cuda.synchronize()
        assert torch.equal(g_out, want_out), f"replay {replay}: O differs"
        for name, got, w in zip(("dQ", "dK", "dV"), (g_dq, g_dk, g_dv), want):
            assert torch.equal(got, w), f"replay {replay}: {name} differs"


@pytest.mark.parametrize("dims,normalised", [((2, 4, 2048, 64, 64), False), ((1, 8, 2048, 128, 128), False),
                                             ((2, 4, 2048, 64, 64), True), ((1, 8, 2048, 128, 128), True),
                                             ((1, 64, 1024, 256, 64), False), ((1, 8, 2048, 256, 64), False)],
                         ids=["d64", "d128", "d64-normalised", "d128-normalised", "wide-4-segments", "wide-scan"])
def test_replayed_graph_of_the_chunkwise_operators_equals_eager(dims, normalised, gpu_device):
    """The chunk-wise walk kernels (totals, scan, walks; with the normaliser also the vector sums and
    the dO pass), forward handing its state to backward: captured once, replayed on fresh inputs."""
    from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd
    from flashy_linear_attention_amd.normalised import linear_attention_normalised_bwd, linear_attention_normalised_fwd

    bs, nh, sq, dqk, dv = dims
    static = [t.to(gpu_device) for t in reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=0)]
    q, k, v, do = static

    def step():
        if normalised:
            out, denom, state = linear_attention_normalised_fwd(q, k, v, 1e-5, True, want_state=True)
            return (out,) + tuple(linear_attention_normalised_bwd(do, q, k, v, out, denom, True, state))
        out, state = linear_attention_chunked_fwd(q, k, v, want_state=True)
        return (out,) + tuple(linear_attention_chunked_bwd(do, q, k, v, state))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = step()
    for replay in range(3):
        fresh = [t.to(gpu_device) for t in reference_style_inputs(bs, nh, sq, dqk, dv, torch.bfloat16, seed=20 + replay)]
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        want = step()  # eager work between replays, on the same inputs
        torch.cuda.synchronize()
        for name, g, w in zip(("out", "dQ", "dK", "dV"), got, want):
            assert torch.equal(g, w), f"replay {replay}: {name} differs"
