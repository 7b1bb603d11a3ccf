"""Run-to-run determinism at full workload sizes: the kernels use no atomics and every output
element has one owner, so repeated launches on the same inputs must agree bit for bit -- a
data race on the LDS ring (a tile overwritten while another wave still reads it, a barrier
that does not cover a load) would show up here as a difference (``-m gpu``)."""

import pytest
import torch

from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd
from flashy_linear_attention_amd.kernels import linear_flash_wrapper_bwd, linear_flash_wrapper_fwd
from flashy_linear_attention_amd.normalised import linear_attention_normalised_fwd
from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["C3", "C5"])
def test_repeated_launches_are_bit_identical(name, gpu_device):
    w = WORKLOADS[name]
    q, k, v, do = (t.to(gpu_device) for t in make_inputs(w))

    def run():
        out = linear_flash_wrapper_fwd(q, k, v)
        grads = linear_flash_wrapper_bwd(do, q, k, v)
        nout, denom = linear_attention_normalised_fwd(q, k, v, 1e-5)
        cout, state = linear_attention_chunked_fwd(q, k, v, True)
        cgrads = linear_attention_chunked_bwd(do, q, k, v, state)
        return (out, *grads, nout, denom, cout, *cgrads)

    ref = run()
    for it in range(8):
        for i, (a, b) in enumerate(zip(run(), ref)):
            assert torch.equal(a, b), f"{name}: output {i} differs on repeat {it}"


@pytest.mark.parametrize("dims", [(4, 16, 4096, 256, 64), (1, 40, 1400, 200, 48), (2, 8, 2100, 256, 96)],
                         ids=lambda d: "x".join(map(str, d)))
def test_repeated_wide_walks_are_bit_identical(dims, gpu_device):
    """q and k wider than 128 columns, chunk-wise: one walk over both 128-column halves whose states take turns in
    one LDS buffer and whose V (V, dO) tiles alternate between two slots -- four, six and many segments per (b, h)
    (segment totals added up by the walks themselves, or entry states from the scan), a v of 64, 48 and 96 columns."""
    from helpers import reference_style_inputs

    q, k, v, do = (t.to(gpu_device) for t in reference_style_inputs(*dims, torch.bfloat16, seed=5))

    def run():
        out, state = linear_attention_chunked_fwd(q, k, v, True)
        return (out, *linear_attention_chunked_bwd(do, q, k, v, state), *linear_attention_chunked_bwd(do, q, k, v, None))

    ref = run()
    for it in range(8):
        for i, (a, b) in enumerate(zip(run(), ref)):
            assert torch.equal(a, b), f"output {i} differs on repeat {it}"
