"""Seeded sweep of the chunk-wise operators over shapes the fixed grids do not hit: the plan of
segments per (b, h) and chunks per segment depends on B H and N, the kernels
on the padded head dims -- so head counts, lengths (ragged against 64, 128 and the segment length)
and widths are drawn at random; forward and backward, with the forward state handed over, against
the oracle's formula evaluated in fp32 on the GPU (``-m gpu``)."""

import random

import pytest
import torch

from flashy_linear_attention_amd import LinearAttentionChunked, LinearAttentionNormalised
from oracle import naive

from helpers import assert_close, gpu_fp32_reference, reference_style_inputs

pytestmark = pytest.mark.gpu


def _cases(seed: int, count: int):
    rng = random.Random(seed)
    out = []
    for i in range(count):
        kind = i % 4
        if kind == 0:    # equal padded head dims <= 64
            dqk, dv = rng.choice([(64, 64), (32, 32), (48, 64), (64, 40), (16, 24)])
        elif kind == 1:  # padded to 128
            dqk, dv = rng.choice([(128, 128), (96, 128), (128, 72), (104, 120)])
        elif kind == 2:  # wide query / key, narrow value; padded widths that differ
            dqk, dv = rng.choice([(256, 64), (192, 64), (256, 128), (136, 32), (200, 8), (128, 64), (128, 24), (64, 32)])
        else:            # a value wider than the query / key; a v of more than 128 columns; widths that are no multiples of 8
            dqk, dv = rng.choice([(64, 256), (256, 256), (64, 128), (32, 96), (100, 250), (20, 100)])
        bh = rng.choice([1, 3, 8, 17, 40, 96])
        b = rng.choice([d for d in (1, 2, 3, 4) if bh % d == 0])
        n = rng.choice([129, 257, 300, 513, 640, 777, 1000, 1301, 2049, 2450, 3000, 4100, 6000])
        if bh * n * max(dqk, dv) > 40 * 4100 * 256:
            n = 1301
        out.append((b, bh // b, n, dqk, dv, 500 + i))
    return out


# (every third case in fp16: both storage types of the walk kernels, whose reverse walk issues its state
# MFMAs from per-type inline assembly)
@pytest.mark.parametrize("case", _cases(20240607, 48), ids=lambda c: "x".join(map(str, c[:5])))
def test_chunked_random_shapes_vs_fp32_formula(case, gpu_device):
    b, h, n, dqk, dv, seed = case
    dtype = torch.float16 if seed % 3 == 0 else torch.bfloat16
    q, k, v, dy = (t.to(gpu_device) for t in reference_style_inputs(b, h, n, dqk, dv, dtype, seed=seed))
    want_o, want_g = gpu_fp32_reference(q, k, v, dy, True)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionChunked.apply(qg, kg, vg)
    out.backward(dy)
    assert_close("O", out, want_o)
    for name, got, want in zip(("dQ", "dK", "dV"), (qg.grad, kg.grad, vg.grad), want_g):
        assert_close(name, got, want)


@pytest.mark.parametrize("case", [c for c in _cases(77, 32) if c[3] <= 128 and c[4] <= 128][:16],
                         ids=lambda c: "x".join(map(str, c[:5])))
def test_normalised_chunked_random_shapes_vs_oracle(case, gpu_device):
    b, h, n, dqk, dv, seed = case
    q, k, v, dy = reference_style_inputs(b, h, n, dqk, dv, torch.float16 if seed % 3 == 0 else torch.bfloat16, seed=seed)
    qo, ko, vo = (t.to(gpu_device).float().requires_grad_(True) for t in (q, k, v))
    want = naive.linear_attention_normalised(qo, ko, vo, eps=1e-5)
    want.backward(dy.to(gpu_device).float())
    qg, kg, vg = (t.to(gpu_device).requires_grad_(True) for t in (q, k, v))
    out = LinearAttentionNormalised.apply(qg, kg, vg, 1e-5, True)
    out.backward(dy.to(gpu_device))
    assert_close("out", out, want.detach())
    # the first rows' normalisers are tiny sums: their gradients are ill-conditioned in 16-bit inputs
    for name, got, w in (("dQ", qg.grad, qo.grad), ("dK", kg.grad, ko.grad), ("dV", vg.grad, vo.grad)):
        assert_close(name, got, w, tol_fro=1e-2, tol_max=5e-2)
