#!/usr/bin/env python3
"""Benchmark of the causal-linear-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3]

One step = one forward (``linear_flash_wrapper_fwd``) plus one backward
(``linear_flash_wrapper_bwd``) over one synthetic batch of the workload, through
the C ABI of libfla_gfx950.so, inputs resident in HBM.  The default workload is
the one the headline metric is quoted on: bf16, B=4 H=32 N=4096 D_qk=D_v=128.

Before the W warm-up steps the same step runs untimed for ``--settle-seconds``
(default 0.3 s) so that the shader clock has left its idle state; the timed
region is exactly K steps between two synchronisations.

Prints ONE JSON line.  ``value`` is causal-counted algorithmic TFLOP/s of the
whole step, N^2 (4 D_qk + 3 D_v) per (b, h) (five products: S, dS, dV, dK, dQ
in backward, two in forward).  ``roofline`` describes the dominant kernel.  All
launches evaluate products Out = mask(X Y^T) Z of N^2 (D_c + D_o) B H algorithmic
FLOPs each; forward is one such launch, and with equal head dims up to 128 the
three backward products are ONE launch of the batched kernel, which is then the
dominant one: its FLOPs (three products) over the duration of the backward-only
region timed here with HIP events on the launch stream, against the dense bf16
MFMA peak.  ``cpu_baseline`` times the oracle's naive PyTorch formula on the
host cores over a bounded sample (whole (b, h) slices at full N and D), in the
same unit.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0}  # MI355X dense MFMA, published
HBM_PEAK_GBS = 8000.0
# HBM bytes per kernel launch (mean over the launches of one step), measured with
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`, each scaled by what the same counter
# reads for a 256 MiB device copy (fetch x2.0, write x1.0); see profiles/*_pmc.md.
MEASURED_TRAFFIC_BYTES = {"C3": 2.420e9}


def _parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--settle-seconds", type=float, default=0.3,
                    help="run untimed steps for this long before the warm-up steps: an idle MI355X sits at a "
                         "95 MHz shader clock and needs about 50 ms of load to reach its sustained clock "
                         "(a 10 ms idle gap is enough to drop it again)")
    ap.add_argument("--workload", default="C3", choices=["C2", "C3", "C4", "C5"])
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-CPU oracle timing")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target seconds of CPU work for the baseline")
    ap.add_argument("--algo", default="quadratic", choices=["quadratic", "chunked", "normalised", "normalised-chunked", "poly"],
                    help="quadratic: the tiled O(N^2 D) kernels the headline metric is defined on (default); "
                         "chunked: the O(N) chunk-state path, reported with its own FLOP count and an HBM roofline; "
                         "normalised: the quadratic kernels plus the fused normaliser (out / (q . cumsum(k) + eps)), "
                         "with the normaliser's own time, bytes and the PyTorch recipe's time beside it; "
                         "normalised-chunked: the same with the chunk-wise product; "
                         "poly (workload C4 only): the same function as C4 computed from the 16-wide x behind its "
                         "Taylor features with the polynomial score map, priced in its own FLOPs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain device copy of 256 MiB (a known-size reference for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


def _time_region(torch, fn, steps):
    """Milliseconds for `steps` calls of fn, HIP events on the current stream."""
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1)


def _cpu_baseline(torch, w, target_seconds):
    """The oracle's naive formula, fp32, on the host: whole (b, h) slices of the
    workload at full N and D, forward (+ backward), until ~target_seconds."""
    from flashy_linear_attention_amd.synthetic import make_inputs
    from oracle import naive

    q, k, v, do = (t.float() for t in make_inputs(w, seed=1, batch=1, heads=1))
    flops_slice = (w.flops_fwd + (w.flops_bwd if w.backward else 0.0)) / (w.batch * w.heads)

    def one():
        naive.causal_dot_product_blocked(q, k, v, block=2048)
        if w.backward:
            naive.causal_dot_product_grads_blocked(q, k, v, do, block=2048)

    one()  # warm-up (thread pool, allocator)
    n, t0 = 0, time.perf_counter()
    while True:
        one()
        n += 1
        dt = time.perf_counter() - t0
        if dt >= target_seconds or n >= 4 * w.batch * w.heads:
            break
    return {
        "value": round(flops_slice * n / dt / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{n} of {w.batch * w.heads} (b,h) slices at full N={w.seq}, D_qk={w.d_qk}, D_v={w.d_v}, "
                  f"fp32 naive PyTorch fwd{'+bwd' if w.backward else ''}, {dt:.1f} s; os.cpu_count()={os.cpu_count()}",
        "ms_per_step_extrapolated": round(dt / n * w.batch * w.heads * 1e3, 1),
    }


def _bench_poly(torch, args, w, dev, time_region) -> int:
    """C4's function, O = tril(phi(xq) phi(xk)^T) V with phi(x) = flatten(x (x) x) / sqrt 2, evaluated
    from the 16-wide x with the polynomial score map f(u) = u^2 / 2, next to the same step on the
    materialised 256-wide features (LinearAttentionSmallVHD's kernels) in the same run."""
    import math

    from flashy_linear_attention_amd.kernels import linear_flash_wrapper_bwd_smallv_hd, linear_flash_wrapper_fwd_smallv_hd
    from flashy_linear_attention_amd.poly import poly_attention_bwd, poly_attention_fwd

    if w.features != "taylor2":
        print("bench.py: --algo poly needs a workload whose q, k are Taylor features (C4)", file=sys.stderr)
        return 2
    r = math.isqrt(w.d_qk)
    gen = torch.Generator().manual_seed(0)
    xq = (0.5 * torch.randn(w.batch, w.heads, w.seq, r, generator=gen)).to(w.dtype)
    xk = (0.5 * torch.randn(w.batch, w.heads, w.seq, r, generator=gen)).to(w.dtype)
    v = torch.randn(w.batch, w.heads, w.seq, w.d_v, generator=gen).to(w.dtype)
    do = torch.randn(w.batch, w.heads, w.seq, w.d_v, generator=gen).to(w.dtype)

    def phi(x):
        return ((x.float()[..., :, None] * x.float()[..., None, :]).flatten(-2) / math.sqrt(2.0)).to(w.dtype)

    q, k = phi(xq).to(dev), phi(xk).to(dev)
    xq, xk, v, do = (t.to(dev) for t in (xq, xk, v, do))
    coef = (0.0, 0.0, 0.5)

    def step():
        poly_attention_fwd(xq, xk, v, coef)
        poly_attention_bwd(do, xq, xk, v, coef)

    def plain_step():
        linear_flash_wrapper_fwd_smallv_hd(q, k, v)
        linear_flash_wrapper_bwd_smallv_hd(do, q, k, v)

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < args.settle_seconds:
        for _ in range(8):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    ms_step = time_region(torch, step, args.steps) / args.steps
    ms_fwd = time_region(torch, lambda: poly_attention_fwd(xq, xk, v, coef), args.steps) / args.steps
    ms_bwd = time_region(torch, lambda: poly_attention_bwd(do, xq, xk, v, coef), args.steps) / args.steps
    for _ in range(20):
        plain_step()
    ms_plain = time_region(torch, plain_step, args.steps) / args.steps
    bh, n = float(w.batch * w.heads), float(w.seq)
    # causal-counted FLOPs of what is evaluated: scores over r columns, second products as they are
    f_fwd = bh * n * n * (r + w.d_v)
    f_bwd = bh * n * n * ((r + w.d_v) + 2 * (w.d_v + r + r))
    value = (f_fwd + f_bwd) / (ms_step * 1e-3) / 1e12
    result = {
        "metric": f"causal linear attention with polynomial score map fwd+bwd TFLOP/s (its own causal-counted FLOPs), "
                  f"B={w.batch} H={w.heads} N={w.seq} R={r} D_v={w.d_v}, 1 MI355X",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"{w.name} evaluated from x: q, k = flatten(x (x) x) / sqrt 2 of a {r}-wide x = 0.5 randn, "
                        f"f(u) = u^2 / 2; v and dO randn, seed 0",
            "flops_per_step": f_fwd + f_bwd, "fwd_ms": round(ms_fwd, 4), "bwd_ms": round(ms_bwd, 4),
            "materialised_features_step_ms": round(ms_plain, 4),
            "speedup_vs_materialised_features": round(ms_plain / ms_step, 2),
        },
        "roofline": {"bound": "mfma", "kernel": "fla::tri_xyt_z_fast_kernel, polynomial and dual-score variants",
                     "achieved": round(value, 2), "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                     "frac": round(value / PEAK_TFLOPS["bf16"], 4), "traffic": None},
    }
    print(json.dumps(result))
    return 0


def main() -> int:
    args = _parse()
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU only (every (batch, head) slice is independent; "
              "no collective exists on this path). Re-run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from flashy_linear_attention_amd import _lib
    from flashy_linear_attention_amd.kernels import (
        linear_flash_wrapper_bwd,
        linear_flash_wrapper_bwd_smallv_hd,
        linear_flash_wrapper_fwd,
        linear_flash_wrapper_fwd_smallv_hd,
    )
    from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs

    if not torch.cuda.is_available():
        print("bench.py: no ROCm GPU visible", file=sys.stderr)
        return 2
    _lib.load()  # fails loudly if the HIP library is missing

    w = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    q, k, v, do = (t.to(dev) for t in make_inputs(w, seed=0))
    fwd = linear_flash_wrapper_fwd_smallv_hd if w.small_v else linear_flash_wrapper_fwd
    bwd = linear_flash_wrapper_bwd_smallv_hd if w.small_v else linear_flash_wrapper_bwd
    if args.algo == "poly":
        return _bench_poly(torch, args, w, dev, _time_region)
    normalised = args.algo.startswith("normalised")
    chunked = args.algo in ("chunked", "normalised-chunked")
    if chunked:
        from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd

        # as under autograd: forward hands its running state to backward
        _, chunk_state = linear_attention_chunked_fwd(q, k, v, want_state=True)

        def fwd(q_, k_, v_):
            return linear_attention_chunked_fwd(q_, k_, v_, want_state=True)

        def bwd(do_, q_, k_, v_):
            return linear_attention_chunked_bwd(do_, q_, k_, v_, chunk_state)
    plain_fwd, plain_bwd = fwd, bwd
    if normalised:
        from flashy_linear_attention_amd.normalised import (
            linear_attention_normalised_bwd,
            linear_attention_normalised_fwd,
        )

        norm_out, norm_denom = linear_attention_normalised_fwd(q, k, v, 1e-5, chunked)

        def fwd(q_, k_, v_):
            return linear_attention_normalised_fwd(q_, k_, v_, 1e-5, chunked)

        def bwd(do_, q_, k_, v_):
            return linear_attention_normalised_bwd(do_, q_, k_, v_, norm_out, norm_denom, chunked)

    def step():
        fwd(q, k, v)
        if w.backward:
            bwd(do, q, k, v)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    settle_steps = 0
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < args.settle_seconds:
        for _ in range(8):
            step()
        settle_steps += 8
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    ms_total = _time_region(torch, step, args.steps)
    ms_step = ms_total / args.steps

    # secondary figures: each half alone (same event method)
    ms_fwd = _time_region(torch, lambda: fwd(q, k, v), args.steps) / args.steps
    ms_bwd = _time_region(torch, lambda: bwd(do, q, k, v), args.steps) / args.steps if w.backward else None

    flops_step = w.flops_fwd + (w.flops_bwd if w.backward else 0.0)
    dt_name = {torch.bfloat16: "bf16", torch.float16: "f16"}[w.dtype]
    peak = PEAK_TFLOPS[dt_name]
    tflops = flops_step / (ms_step * 1e-3) / 1e12

    # The dominant kernel and its launches.  Every launch evaluates products Out = mask(X Y^T) Z of
    # N^2 (D_c + D_o) B H algorithmic FLOPs each.  With equal padded widths up to 128 the three
    # backward products go out as ONE launch of fla::tri_xyt_z_fast_batch_kernel (the dominant
    # kernel: three quarters of the step); its duration is the backward-only region timed above.
    # Otherwise every product is a launch of its own (two when an output wider than 128 columns
    # meets a <=64- or 256-wide contraction: one per 128-column half) and the figures are means
    # over the launches of a step.
    def n_launches(dc, dout):
        return 2 if dout > 128 and (dc <= 64 or dc > 128) else 1

    def pad(d):
        return 32 if d <= 32 else 64 if d <= 64 else 128 if d <= 128 else 256

    flops_product = float(w.batch * w.heads) * w.seq * w.seq * (w.d_qk + w.d_v)
    batched_bwd = w.backward and pad(w.d_qk) == pad(w.d_v) and pad(w.d_qk) <= 128
    if batched_bwd:
        launches = 2
        kernel_name = "fla::tri_xyt_z_fast_batch_kernel (dQ, dV, dK: three products Out = mask(X Y^T) Z in one launch)"
        flops_launch = 3.0 * flops_product
        ms_launch = ms_bwd
    else:
        launches = n_launches(w.d_qk, w.d_v)
        if w.backward:
            launches += n_launches(w.d_v, w.d_qk) * 2 + n_launches(w.d_qk, w.d_v)
        products = 1 + (3 if w.backward else 0)
        kernel_name = "fla::tri_xyt_z_fast_kernel (Out = mask(X Y^T) Z)"
        flops_launch = flops_product * products / launches
        ms_launch = ms_step / launches
    achieved = flops_launch / (ms_launch * 1e-3) / 1e12

    result = {
        "metric": f"causal linear attention {'fwd+bwd' if w.backward else 'fwd'} TFLOP/s "
                  f"(causal-counted), B={w.batch} H={w.heads} N={w.seq} D_qk={w.d_qk} D_v={w.d_v}, 1 MI355X",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dt_name,
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: LinearAttention{'SmallVHD' if w.small_v else ''} "
                        f"{'fwd+bwd' if w.backward else 'fwd'}, {dt_name}, B={w.batch} H={w.heads} N={w.seq} "
                        f"D_qk={w.d_qk} D_v={w.d_v}, q/k features {w.features}, v and dO randn, seed 0",
            "flops_per_step": flops_step,
            "clock_settle_steps": settle_steps,
            "fwd_ms": round(ms_fwd, 4),
            "bwd_ms": None if ms_bwd is None else round(ms_bwd, 4),
            "fwd_tflops": round(w.flops_fwd / (ms_fwd * 1e-3) / 1e12, 2),
            "bwd_tflops": None if ms_bwd is None else round(w.flops_bwd / (ms_bwd * 1e-3) / 1e12, 2),
            "pct_of_mfma_peak": round(100.0 * tflops / peak, 2),
        },
        "roofline": {
            "bound": "mfma",
            "kernel": kernel_name,
            "achieved": round(achieved, 2),
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": round(achieved / peak, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(w.name),
            "traffic_note": "HBM bytes per launch of the dominant kernel, rocprofv3 FETCH_SIZE/WRITE_SIZE (profiles/)",
            "launches_per_step": launches,
            "flops_per_launch": flops_launch,
            "avg_launch_ms": round(ms_launch, 4),
        },
    }
    if chunked:
        # The chunked path does different (far less) arithmetic, so it is never priced in the
        # quadratic algorithm's FLOPs: its own count, and the HBM roofline that bounds it.
        chunk = 256 if (w.d_qk // 2 + w.d_v <= 192 and w.d_v // 2 + w.d_qk <= 192) else 128
        bh, n = w.batch * w.heads, w.seq
        f_intra = float(bh) * n * chunk * (w.d_qk + w.d_v)          # causal-counted diagonal blocks
        f_state = 4.0 * bh * n * w.d_qk * w.d_v                     # Y^T Z per chunk + X . S
        flops_fwd = f_intra + f_state
        flops_bwd = 3.0 * flops_fwd if w.backward else 0.0          # three products of the same shape
        bytes_step = w.bytes_fwd + (w.bytes_bwd if w.backward else 0.0)
        result["metric"] = result["metric"].replace("TFLOP/s (causal-counted)", "TFLOP/s (chunked algorithm's own FLOPs)")
        result["value"] = round((flops_fwd + flops_bwd) / (ms_step * 1e-3) / 1e12, 2)
        result["config"]["workload"] += f"; chunk-wise evaluation, {chunk}-row chunks"
        result["config"]["flops_per_step"] = flops_fwd + flops_bwd
        result["config"]["fwd_tflops"] = round(flops_fwd / (ms_fwd * 1e-3) / 1e12, 2)
        result["config"]["bwd_tflops"] = None if ms_bwd is None else round(flops_bwd / (ms_bwd * 1e-3) / 1e12, 2)
        result["config"]["pct_of_mfma_peak"] = round(100.0 * result["value"] / peak, 2)
        gbs = bytes_step / (ms_step * 1e-3) / 1e9
        result["roofline"] = {
            "bound": "hbm",
            "kernel": "chunk_state + chunk_scan (two running states per step when shared, else one per product) + tri_xyt_z_fast (chunked) per product",
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": None,
            "algorithmic_bytes_per_step": bytes_step,
        }
    if normalised:
        # What is new are the memory-bound passes around the product kernels.  Their time is the
        # difference to the plain step in this same run, their algorithmic bytes: forward (separate pass)
        # reads q, k, O and writes out (+ n); backward reads g, out (pre-pass, writes dO) and
        # q, k, dq, dk (post-pass, writes dq, dk); 2 bytes per element, fp32 vectors of length N aside.
        def plain_step():
            plain_fwd(q, k, v)
            if w.backward:
                plain_bwd(do, q, k, v)

        ms_plain = _time_region(torch, plain_step, args.steps) / args.steps
        # (with the quadratic product the forward normaliser lives inside the product kernel -- row sums
        # of the scores -- and moves no extra bytes; only the chunk-wise product needs the forward pass)
        e = float(w.batch * w.heads * w.seq)
        nbytes = 2.0 * e * (2 * w.d_qk + 2 * w.d_v) if chunked else 4.0 * e
        if w.backward:
            nbytes += 2.0 * e * (3 * w.d_v + 6 * w.d_qk)
        extra_ms = ms_step - ms_plain

        def recipe_step():
            qa, ka, va = (t.detach().requires_grad_(w.backward) for t in (q, k, v))
            op = LinearAttentionSmallVHD if w.small_v else LinearAttention
            num = op.apply(qa, ka, va)
            den = (qa * ka.cumsum(-2)).sum(dim=-1, keepdim=True) + 1e-5
            out = num / den
            if w.backward:
                out.backward(do)

        from flashy_linear_attention_amd import LinearAttention, LinearAttentionSmallVHD

        for _ in range(10):
            recipe_step()
        ms_recipe = _time_region(torch, recipe_step, max(10, args.steps // 5)) / max(10, args.steps // 5)
        # the dominant kernel is still the product kernel: its per-launch figures come from the plain step
        if not chunked:
            plain_flops = flops_product * (4 if w.backward else 1)
            result["roofline"]["kernel"] = ("fla::tri_xyt_z_fast_kernel / _batch_kernel "
                                            "(all product launches of the plain step)")
            result["roofline"]["avg_launch_ms"] = round(ms_plain / launches, 4)
            result["roofline"]["flops_per_launch"] = plain_flops / launches
            result["roofline"]["achieved"] = round(plain_flops / (ms_plain * 1e-3) / 1e12, 2)
            result["roofline"]["frac"] = round(result["roofline"]["achieved"] / peak, 4)
        result["metric"] = result["metric"].replace("causal linear attention", "normalised causal linear attention")
        result["config"]["workload"] += "; fused normaliser out / (q . cumsum(k) + 1e-5)"
        result["config"]["normaliser"] = {
            "plain_step_ms": round(ms_plain, 4),
            "extra_ms": round(extra_ms, 4),
            "algorithmic_bytes": nbytes,
            "gbps": round(nbytes / (extra_ms * 1e-3) / 1e9, 1) if extra_ms > 0 else None,
            "frac_of_hbm_peak": round(nbytes / (extra_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if extra_ms > 0 else None,
            "pytorch_recipe_step_ms": round(ms_recipe, 4),
            "speedup_vs_pytorch_recipe": round(ms_recipe / ms_step, 2),
        }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = _cpu_baseline(torch, w, args.cpu_seconds)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
