"""Shared helpers of the test-suite: error metrics and input builders."""

from __future__ import annotations

import math
from typing import Tuple

import torch

# Tolerances against the fp32 oracle, for 16-bit storage with fp32 accumulation.
# E1 is the reference's criterion (flashlinear/test_attn.py:17,24-25); E2 bounds
# the worst element relative to the largest magnitude of the expected tensor.
TOL_FRO = 1e-2
TOL_MAX = 1e-2


def rel_fro(x: torch.Tensor, y: torch.Tensor) -> float:
    x, y = x.detach().double().cpu(), y.detach().double().cpu()
    return float(torch.linalg.norm(x - y) / torch.linalg.norm(y).clamp_min(1e-300))


def rel_max(x: torch.Tensor, y: torch.Tensor) -> float:
    x, y = x.detach().double().cpu(), y.detach().double().cpu()
    return float((x - y).abs().max() / y.abs().max().clamp_min(1e-300))


def assert_close(name: str, got: torch.Tensor, want: torch.Tensor, tol_fro: float = TOL_FRO, tol_max: float = TOL_MAX):
    assert got.shape == want.shape, f"{name}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    e1, e2 = rel_fro(got, want), rel_max(got, want)
    assert e1 <= tol_fro, f"{name}: Frobenius-relative error {e1:.3e} > {tol_fro}"
    assert e2 <= tol_max, f"{name}: max-abs/max error {e2:.3e} > {tol_max}"


def reference_style_inputs(
    bs: int, nh: int, sq: int, hd_qk: int, hd_v: int, dtype: torch.dtype, seed: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Inputs distributed like the reference's tests draw them
    (flashlinear/test_attn.py:28-46,105): q, k = softplus(randn), q scaled by
    1/sqrt(hd); v = randn; upstream gradient 0.1 * randn.  Drawn on the CPU."""
    g = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.softplus(torch.randn(bs, nh, sq, hd_qk, generator=g)) / math.sqrt(hd_qk)
    k = torch.nn.functional.softplus(torch.randn(bs, nh, sq, hd_qk, generator=g))
    v = torch.randn(bs, nh, sq, hd_v, generator=g)
    dy = 0.1 * torch.randn(bs, nh, sq, hd_v, generator=g)
    return tuple(t.to(dtype) for t in (q, k, v, dy))


def load_golden(name: str):
    """A fixture from tests/golden as torch tensors: bf16 inputs, fp32 expected outputs."""
    import os

    import numpy as np

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name + ".npz")
    z = np.load(path, allow_pickle=False)
    ins = {n: torch.from_numpy(z[n + "_bf16"].view(np.int16).copy()).view(torch.bfloat16) for n in ("q", "k", "v", "do")}
    outs = {n: torch.from_numpy(z[n].copy()) for n in ("o", "dq", "dk", "dv")}
    return ins, outs


GOLDEN_CASES = ("equal_d_b1_h1_n128_d32", "small_v_b1_h1_n128_dqk64_dv16")


def _naive():
    from oracle import naive

    return naive


def gpu_fp32_reference(q, k, v, do, backward, heads_per_chunk=8):
    """The oracle's blocked formula evaluated in fp32 on the GPU, a few heads at
    a time (the full score tensor of C3 would be 8.6 GB)."""
    b, h = q.shape[:2]
    o = torch.empty(*q.shape[:3], v.shape[-1], dtype=torch.float32, device=q.device)
    grads = [torch.empty(t.shape, dtype=torch.float32, device=q.device) for t in (q, k, v)] if backward else None
    for bi in range(b):
        for h0 in range(0, h, heads_per_chunk):
            sl = (slice(bi, bi + 1), slice(h0, h0 + heads_per_chunk))
            qs, ks, vs = q[sl].float(), k[sl].float(), v[sl].float()
            o[sl] = _naive().causal_dot_product_blocked(qs, ks, vs, block=2048)
            if backward:
                for gbuf, gval in zip(grads, _naive().causal_dot_product_grads_blocked(qs, ks, vs, do[sl].float(), block=2048)):
                    gbuf[sl] = gval
    return o, grads
