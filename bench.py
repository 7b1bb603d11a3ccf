#!/usr/bin/env python3
"""Benchmark of the causal-linear-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3]

One step = one forward (``linear_flash_wrapper_fwd``) plus one backward
(``linear_flash_wrapper_bwd``) over one synthetic batch of the workload, through
the C ABI of libfla_gfx950.so, inputs resident in HBM.  The default workload is
the one the headline metric is quoted on: bf16, B=4 H=32 N=4096 D_qk=D_v=128.

Before the W warm-up steps the same step runs untimed for ``--settle-seconds``
(default 0.3 s) so that the shader clock has left its idle state; the timed
region is exactly K steps between two synchronisations (``ms_per_step``,
``value``).  After it, forward, backward, the step and the step through autograd
(``LinearAttention.apply`` + ``torch.autograd.grad``) are each timed once more
with one HIP event pair per iteration; ``config.median_ms`` holds the medians.

Prints ONE JSON line.  ``value`` is causal-counted algorithmic TFLOP/s of the
whole step, N^2 (4 D_qk + 3 D_v) per (b, h): five products in backward (S, dS,
dV, dK, dQ), two in forward.  ``roofline`` describes the dominant kernel.  With
equal head dims up to 128 that is the batched backward kernel (dQ, dV and dK in
one launch): ``achieved`` = the backward's algorithmic FLOPs, N^2 (3 D_qk + 2
D_v) B H, over the average duration of the backward-only region timed here with
HIP events on the launch stream; ``frac`` = that over the dense bf16 MFMA peak.
The kernel executes six product-units for those five (dO V^T is formed for dQ
and again for dK): ``executed_tflops`` / ``executed_frac`` price what it issues.
``cpu_baseline`` times the oracle's naive PyTorch formula on the host cores
over a bounded sample, in the same unit.  ``config.other_workloads`` holds
short runs of the other benchmark workloads (default run only).
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0}  # MI355X dense MFMA, published
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of a workload's dominant kernel, from rocprofv3 --pmc FETCH_SIZE and
# --pmc WRITE_SIZE runs (each scaled by what the same counter reads for a device copy of known
# size): (workload, algo) -> (bytes, the summary under profiles/ that holds the readings).
# Workloads without an entry report `traffic: null`.
PROFILED_TRAFFIC = {
    ("C3", "quadratic"): (2.426e9, "profiles/tri_xyt_z_fast_kernels_C3_pmc.md"),
    # chunk-wise: all kernels of a step
    ("C3", "chunked"): (1.847e9, "profiles/chunked_C3_C5_kernel_trace_pmc.md"),
    ("C4", "chunked"): (1.310e9, "profiles/chunked_C4_kernel_trace_pmc.md"),
    ("C5", "chunked"): (1.074e9, "profiles/chunked_C3_C5_kernel_trace_pmc.md"),
}
# MFMA operations the dominant kernel issues over those of its product-units (rocprofv3
# SQ_INSTS_VALU_MFMA_MOPS_BF16 x 512 FLOPs; the excess is the 32 x 32 blocks on the diagonal)
PROFILED_MFMA_RATIO = {("C3", "quadratic"): (1.008, "profiles/tri_xyt_z_fast_kernels_C3_pmc.md")}

ALGOS = ["quadratic", "chunked", "normalised", "normalised-chunked", "poly", "feature"]
# how the quadratic backward is evaluated: "products" = dQ, dV, dK as three products in one launch (the
# library's choice); "fused-dkdv" = dV and dK by one kernel from one stream of (Q, dO) tiles plus dQ's
# product (fla_linear_attn_bwd_fused_dkdv, the measured alternative)
BWD_PLAN = "products"


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
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the short runs of the other workloads that the default run appends")
    ap.add_argument("--other-steps", type=int, default=50, help="timed iterations per entry of other_workloads")
    ap.add_argument("--bwd-plan", choices=["products", "fused-dkdv"], default="products",
                    help="evaluation of the quadratic backward (see BWD_PLAN); the default is what the library's "
                         "operators use")
    ap.add_argument("--algo", default="quadratic", choices=ALGOS,
                    help="quadratic: the tiled O(N^2 D) kernels the headline metric is defined on (default); "
                         "chunked: the O(N) chunk-state path, reported with its own FLOP count and an HBM roofline; "
                         "normalised: the quadratic kernels plus the fused normaliser (out / (q . cumsum(k) + eps)), "
                         "with the normaliser's own time, bytes and the PyTorch recipe's time beside it; "
                         "normalised-chunked: the same with the chunk-wise product; "
                         "poly (workload C4 only): the same function as C4 computed from the 16-wide x behind its "
                         "Taylor features with the polynomial score map, priced in its own FLOPs; "
                         "feature: the chunk-wise operator on raw xq, xk with elu(x) + 1 applied as the kernels load "
                         "them, next to 'PyTorch elu pass + chunk-wise operator' through autograd in the same run")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of one workload: forward + backward of the quadratic kernels over a grid of "
                         "(B*H, N, D_qk, D_v) off the benchmark shapes, one JSON line with a `sweep` list (what the "
                         "fixed launch rules give where nobody tuned them)")
    ap.add_argument("--crossover", action="store_true",
                    help="instead of the benchmark: time the quadratic and the chunk-wise forward + backward over a grid "
                         "of shapes and print one JSON line with a `crossover` list (what the library's selection table, "
                         "fla_linear_attn_prefers_chunked, is read off)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain device copy of 256 MiB (a known-size reference for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


def _time_region(torch, fn, steps):
    """Milliseconds for `steps` back-to-back calls of fn: one HIP event pair on the current stream
    around the whole region, a synchronisation on either side."""
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1)


def _time_each(torch, fn, steps):
    """Milliseconds of each of `steps` back-to-back calls of fn: an event between every two calls
    (the GPU stays busy throughout, so the clock does not drop between iterations)."""
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    return [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]


def _median_ms(torch, fn, steps):
    return statistics.median(_time_each(torch, fn, steps))


def _host_side(torch, fn, calls=200):
    """What a caller sees per call of fn (a launch wrapper): host time to enqueue one call
    (perf_counter over `calls` back-to-back calls, no synchronisation inside the loop; when the
    GPU is the slower side this is the GPU's time per call instead) and the wall time of an
    isolated call, synchronised before and after (launch latency + kernel + completion)."""
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(calls):
        fn()
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    iso = []
    for _ in range(50):
        torch.cuda.synchronize()
        a = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        iso.append((time.perf_counter() - a) * 1e6)
    return {"enqueue_loop_us_per_call": round((t1 - t0) / calls * 1e6, 2),
            "isolated_call_us_median": round(statistics.median(iso), 2)}


def _settle(torch, step, seconds):
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            step()
        n += 8
        torch.cuda.synchronize()
    return n


def _pad(d):
    return 32 if d <= 32 else 64 if d <= 64 else 128 if d <= 128 else 256


def _chunk_rows(w):
    """Rows per chunk of the kernels this workload's chunk-wise step runs."""
    if _pad(w.d_qk) == _pad(w.d_v) and _pad(w.d_qk) <= 128:  # the walk kernels
        return 128 if _pad(w.d_qk) <= 64 else 64
    if 128 < w.d_qk <= 256 and w.d_v <= 128:  # two 128-column halves of q, k through the D = 128 walk kernels
        return 64
    return 256 if (w.d_qk // 2 + w.d_v <= 192 and w.d_v // 2 + w.d_qk <= 192) else 128


def _chunked_flops(w):
    """(forward, backward) FLOPs of the chunk-wise algorithm itself: causal-counted diagonal blocks
    plus Y^T Z per chunk and X . S, per product; backward is three products of the same shape."""
    bh, n, chunk = w.batch * w.heads, w.seq, _chunk_rows(w)
    fwd = float(bh) * n * chunk * (w.d_qk + w.d_v) + 4.0 * bh * n * w.d_qk * w.d_v
    return fwd, (3.0 * fwd if w.backward else 0.0)


def _ops(torch, w, algo, dev):
    """Device inputs and the forward / backward / autograd callables of one (workload, algo)."""
    from flashy_linear_attention_amd import LinearAttention, LinearAttentionChunked, LinearAttentionSmallVHD
    from flashy_linear_attention_amd.kernels import (
        linear_flash_wrapper_bwd,
        linear_flash_wrapper_bwd_smallv_hd,
        linear_flash_wrapper_fwd,
        linear_flash_wrapper_fwd_smallv_hd,
    )
    from flashy_linear_attention_amd.synthetic import make_inputs

    q, k, v, do = (t.to(dev) for t in make_inputs(w, seed=0))
    fwd = linear_flash_wrapper_fwd_smallv_hd if w.small_v else linear_flash_wrapper_fwd
    bwd = linear_flash_wrapper_bwd_smallv_hd if w.small_v else linear_flash_wrapper_bwd
    op = LinearAttentionSmallVHD if w.small_v else LinearAttention
    if BWD_PLAN == "fused-dkdv" and algo == "quadratic":
        from flashy_linear_attention_amd.kernels.linear_attn_kernels import linear_flash_wrapper_bwd_fused_dkdv

        bwd = linear_flash_wrapper_bwd_fused_dkdv
    if algo in ("chunked", "normalised-chunked"):
        from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd

        # as under autograd: forward hands its running state to backward
        _, chunk_state = linear_attention_chunked_fwd(q, k, v, want_state=True)

        def fwd(q_, k_, v_):
            return linear_attention_chunked_fwd(q_, k_, v_, want_state=True)

        def bwd(do_, q_, k_, v_):
            return linear_attention_chunked_bwd(do_, q_, k_, v_, chunk_state)

        op = LinearAttentionChunked
    qa, ka, va = (t.detach().clone().requires_grad_(True) for t in (q, k, v))

    def autograd_step():
        out = op.apply(qa, ka, va)
        if w.backward:
            torch.autograd.grad(out, (qa, ka, va), do)

    return {"q": q, "k": k, "v": v, "do": do, "fwd": lambda: fwd(q, k, v), "bwd": lambda: bwd(do, q, k, v),
            "fwd_fn": fwd, "bwd_fn": bwd, "autograd_step": autograd_step, "op": op}


def _other_workload(torch, name, algo, dev, steps):
    """A short run of another workload: medians of per-iteration HIP event pairs."""
    from flashy_linear_attention_amd.synthetic import WORKLOADS

    w = WORKLOADS[name]
    o = _ops(torch, w, algo, dev)

    def step():
        o["fwd"]()
        if w.backward:
            o["bwd"]()

    _settle(torch, step, 0.15)
    for _ in range(10):
        step()
    ms_step = _median_ms(torch, step, steps)
    ms_fwd = _median_ms(torch, o["fwd"], steps)
    ms_bwd = _median_ms(torch, o["bwd"], steps) if w.backward else None
    dt_name = {torch.bfloat16: "bf16", torch.float16: "f16"}[w.dtype]
    host = _host_side(torch, o["fwd"]) if w.seq * w.batch * w.heads <= 1 << 18 else None
    rec = {"workload": name, "algo": algo, "dtype": dt_name, "steps": steps,
           "shape": f"B={w.batch} H={w.heads} N={w.seq} D_qk={w.d_qk} D_v={w.d_v}",
           "median_step_ms": round(ms_step, 4), "median_fwd_ms": round(ms_fwd, 4),
           "median_bwd_ms": None if ms_bwd is None else round(ms_bwd, 4)}
    if host is not None:  # launch-bound sizes: the region mean (no events between launches) and the host's view
        rec["back_to_back_fwd_ms"] = round(_time_region(torch, o["fwd"], 4 * steps) / (4 * steps), 4)
        rec["host_forward_wrapper"] = host
    if algo == "quadratic":
        flops = w.flops_fwd + (w.flops_bwd if w.backward else 0.0)
        tf = flops / (ms_step * 1e-3) / 1e12
        rec.update({"tflops": round(tf, 1), "bound": "mfma", "frac_of_peak": round(tf / PEAK_TFLOPS[dt_name], 4),
                    "flops": "quadratic algorithm, causal-counted"})
    else:
        nbytes = w.bytes_fwd + (w.bytes_bwd if w.backward else 0.0)
        gbs = nbytes / (ms_step * 1e-3) / 1e9
        ff, fb = _chunked_flops(w)
        rec.update({"gbps_algorithmic": round(gbs, 1), "bound": "hbm", "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4),
                    "own_tflops": round((ff + fb) / (ms_step * 1e-3) / 1e12, 1),
                    "bytes": "each operand read once, each result written once",
                    "algorithmic_bytes_per_step": nbytes})
        traffic, src = PROFILED_TRAFFIC.get((name, algo), (None, None))
        if traffic is not None:  # HBM bytes all kernels of a step move (rocprofv3 FETCH_SIZE / WRITE_SIZE, see the file)
            rec.update({"traffic_bytes_per_step": traffic, "traffic_over_algorithmic_bytes": round(traffic / nbytes, 2),
                        "traffic_gbps": round(traffic / (ms_step * 1e-3) / 1e9, 1), "traffic_source": src})
    del o
    torch.cuda.empty_cache()
    return rec


def _other_extension(torch, name, algo, dev, steps):
    """A short run of one of the operators beyond the reference's two (normaliser inside, feature map on
    load, polynomial score map) with the caller-side PyTorch recipe it replaces timed beside it."""
    import argparse

    from flashy_linear_attention_amd.synthetic import WORKLOADS

    w = WORKLOADS[name]
    short = argparse.Namespace(steps=steps, warmup=10, settle_seconds=0.15)
    if algo in ("poly", "feature"):
        full = (_bench_poly if algo == "poly" else _bench_feature)(torch, short, w, dev)
        c, r = full["config"], full["roofline"]
        rec = {"workload": name, "algo": algo, "dtype": "bf16", "steps": steps,
               "shape": f"B={w.batch} H={w.heads} N={w.seq} D_qk={w.d_qk} D_v={w.d_v}", "step_ms": full["ms_per_step"],
               "bound": r["bound"], "frac_of_peak": r["frac"]}
        if algo == "poly":
            rec.update({"own_tflops": full["value"], "flops": "its own causal-counted FLOPs (scores over the 16-wide x)",
                        "materialised_features_step_ms": c["materialised_features_step_ms"],
                        "speedup_vs_materialised_features": c["speedup_vs_materialised_features"]})
        else:
            rec.update({"gbps_algorithmic": full["value"], "algorithmic_bytes_per_step": c["algorithmic_bytes_per_step"],
                        "bytes": "the plain operator's tensors (xq, xk for q, k) plus phi(xq), phi(xk) written once",
                        "autograd_step_ms": c["median_ms"]["autograd_step"],
                        "pytorch_elu_passes_plus_chunked_operator_autograd_step_ms":
                            c["pytorch_elu_passes_plus_chunked_operator_autograd_step_ms"],
                        "speedup_vs_pytorch_elu_passes": c["speedup_vs_pytorch_elu_passes"]})
        torch.cuda.empty_cache()
        return rec
    from flashy_linear_attention_amd import LinearAttention, LinearAttentionSmallVHD
    from flashy_linear_attention_amd.normalised import linear_attention_normalised_bwd, linear_attention_normalised_fwd
    from flashy_linear_attention_amd.synthetic import make_inputs

    chunked = algo == "normalised-chunked"
    q, k, v, do = (t.to(dev) for t in make_inputs(w, seed=0))
    out, denom, state = linear_attention_normalised_fwd(q, k, v, 1e-5, chunked, want_state=True)

    def step():
        linear_attention_normalised_fwd(q, k, v, 1e-5, chunked, want_state=chunked)
        linear_attention_normalised_bwd(do, q, k, v, out, denom, chunked, state)

    def recipe_step():  # README.md:27-30 of the reference around the quadratic operator, through autograd
        qr, kr, vr = (t.detach().requires_grad_(True) for t in (q, k, v))
        num = (LinearAttentionSmallVHD if w.small_v else LinearAttention).apply(qr, kr, vr)
        (num / ((qr * kr.cumsum(-2)).sum(dim=-1, keepdim=True) + 1e-5)).backward(do)

    _settle(torch, step, 0.15)
    for _ in range(10):
        step()
    ms_step = _median_ms(torch, step, steps)
    for _ in range(3):
        recipe_step()
    ms_recipe = _median_ms(torch, recipe_step, max(5, steps // 5))
    rec = {"workload": name, "algo": algo, "dtype": "bf16", "steps": steps,
           "shape": f"B={w.batch} H={w.heads} N={w.seq} D_qk={w.d_qk} D_v={w.d_v}", "step_ms": round(ms_step, 4),
           "pytorch_recipe_step_ms": round(ms_recipe, 4), "speedup_vs_pytorch_recipe": round(ms_recipe / ms_step, 2)}
    if chunked:
        e = float(w.batch * w.heads * w.seq)
        nbytes = w.bytes_fwd + w.bytes_bwd + 4.0 * e + 4.0 * e + 2.0 * e * w.d_v
        gbs = nbytes / (ms_step * 1e-3) / 1e9
        rec.update({"bound": "hbm", "gbps_algorithmic": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4),
                    "algorithmic_bytes_per_step": nbytes,
                    "bytes": "the plain operator's (operands read once, results written once) plus n written and read "
                             "and the saved output read in backward"})
    else:
        tf = (w.flops_fwd + w.flops_bwd) / (ms_step * 1e-3) / 1e12
        rec.update({"bound": "mfma", "tflops": round(tf, 1), "frac_of_peak": round(tf / PEAK_TFLOPS["bf16"], 4),
                    "flops": "quadratic algorithm, causal-counted (the normaliser's passes add time, no counted FLOPs)"})
    del q, k, v, do, out, denom, state
    torch.cuda.empty_cache()
    return rec


def _crossover(torch, dev, steps) -> int:
    """Quadratic against chunk-wise forward + backward (bf16, B = 1, through the Python wrappers, the
    chunk-wise pair with forward's state handed over) over a grid of shapes, next to what the library's
    selection table answers for each.  Medians of per-iteration event pairs."""
    from flashy_linear_attention_amd import _lib
    from flashy_linear_attention_amd.chunked import linear_attention_chunked_bwd, linear_attention_chunked_fwd
    from flashy_linear_attention_amd.kernels import (
        linear_flash_wrapper_bwd,
        linear_flash_wrapper_bwd_smallv_hd,
        linear_flash_wrapper_fwd,
        linear_flash_wrapper_fwd_smallv_hd,
    )

    pick = _lib.load().fla_linear_attn_prefers_chunked
    gen = torch.Generator(device=dev).manual_seed(0)
    out = []
    for d_qk, d_v in ((32, 32), (64, 64), (128, 128), (256, 64), (192, 128), (256, 256)):
        for bh in (16, 64, 128, 256, 512):
            for n in (256, 512, 1024, 2048, 4096, 8192):
                if bh * n * max(d_qk, d_v) > 2 ** 28 or (d_qk != d_v and bh > 256):
                    continue
                q = (torch.rand(1, bh, n, d_qk, device=dev, generator=gen) + 0.5).bfloat16()
                k = (torch.rand(1, bh, n, d_qk, device=dev, generator=gen) + 0.5).bfloat16()
                v = torch.randn(1, bh, n, d_v, device=dev, generator=gen).bfloat16()
                do = torch.randn(1, bh, n, d_v, device=dev, generator=gen).bfloat16()
                small = d_qk != d_v

                def quadratic():
                    if small:
                        linear_flash_wrapper_fwd_smallv_hd(q, k, v)
                        linear_flash_wrapper_bwd_smallv_hd(do, q, k, v)
                    else:
                        linear_flash_wrapper_fwd(q, k, v)
                        linear_flash_wrapper_bwd(do, q, k, v)

                def chunked():
                    _, st = linear_attention_chunked_fwd(q, k, v, want_state=True)
                    linear_attention_chunked_bwd(do, q, k, v, st)

                _settle(torch, chunked, 0.05)
                us_q, us_c = 1e3 * _median_ms(torch, quadratic, steps), 1e3 * _median_ms(torch, chunked, steps)
                out.append({"BH": bh, "N": n, "D_qk": d_qk, "D_v": d_v, "quadratic_us": round(us_q, 1),
                            "chunked_us": round(us_c, 1), "table_says_chunked": int(pick(1, bh, n, d_qk, d_v)),
                            "chunked_is_faster": int(us_c < us_q)})
                del q, k, v, do
    wrong = [r for r in out if r["table_says_chunked"] != r["chunked_is_faster"]]
    worst = max((max(r["quadratic_us"], r["chunked_us"]) / min(r["quadratic_us"], r["chunked_us"]) for r in wrong), default=1.0)
    print(json.dumps({"metric": "quadratic against chunk-wise forward + backward over a grid of shapes, bf16, 1 MI355X",
                      "unit": "us", "steps": steps, "cells": len(out), "cells_where_the_table_picks_the_slower": len(wrong),
                      "worst_loss_factor": round(worst, 2), "crossover": out}))
    return 0


def _sweep(torch, dev, steps) -> int:
    """Quadratic forward + backward over a grid of shapes, bf16, inputs drawn on the GPU (q, k
    uniform in [0.5, 1.5), v and dO normal).  Medians of per-iteration event pairs."""
    from flashy_linear_attention_amd.kernels import (
        linear_flash_wrapper_bwd,
        linear_flash_wrapper_bwd_smallv_hd,
        linear_flash_wrapper_fwd,
        linear_flash_wrapper_fwd_smallv_hd,
    )

    grid = []
    for d_qk, d_v in ((32, 32), (64, 64), (128, 128), (256, 256), (64, 16), (128, 32), (256, 64), (96, 96), (200, 64)):
        for n in (512, 1024, 2048, 4096, 8192, 16384):
            for bh in (8, 32, 128):
                flops = float(bh) * n * n * (4 * d_qk + 3 * d_v)
                if flops < 2e10 or flops > 8e12 or bh * n * max(d_qk, d_v) * 2 * 7 > 6e9:
                    continue
                grid.append((bh, n, d_qk, d_v, flops))
    gen = torch.Generator(device=dev).manual_seed(0)
    out = []
    for bh, n, d_qk, d_v, flops in grid:
        q = (torch.rand(1, bh, n, d_qk, device=dev, generator=gen) + 0.5).bfloat16()
        k = (torch.rand(1, bh, n, d_qk, device=dev, generator=gen) + 0.5).bfloat16()
        v = torch.randn(1, bh, n, d_v, device=dev, generator=gen).bfloat16()
        do = torch.randn(1, bh, n, d_v, device=dev, generator=gen).bfloat16()
        small = d_qk != d_v
        fwd = (lambda: linear_flash_wrapper_fwd_smallv_hd(q, k, v)) if small else (lambda: linear_flash_wrapper_fwd(q, k, v))
        bwd = (lambda: linear_flash_wrapper_bwd_smallv_hd(do, q, k, v)) if small else (lambda: linear_flash_wrapper_bwd(do, q, k, v))

        def step():
            fwd()
            bwd()

        _settle(torch, step, 0.1)
        ms_f, ms_b = _median_ms(torch, fwd, steps), _median_ms(torch, bwd, steps)
        ms_s = _median_ms(torch, step, steps)
        tf = flops / (ms_s * 1e-3) / 1e12
        out.append({"BH": bh, "N": n, "D_qk": d_qk, "D_v": d_v, "fwd_ms": round(ms_f, 4), "bwd_ms": round(ms_b, 4),
                    "step_ms": round(ms_s, 4), "tflops": round(tf, 1), "pct_of_peak": round(100 * tf / PEAK_TFLOPS["bf16"], 1)})
        del q, k, v, do
    print(json.dumps({"metric": "causal linear attention fwd+bwd TFLOP/s (causal-counted) over a grid of shapes, bf16, 1 MI355X",
                      "unit": "TFLOP/s", "steps": steps, "sweep": out}))
    return 0


def _cpu_baseline(torch, w, target_seconds):
    """The oracle's naive formula, fp32, on the host cores: (i) one (b, h) slice of the workload
    at full N and D, forward (+ backward), repeated until ~target_seconds, extrapolated to all
    slices; (ii) the small normalised workload C1 in full (forward + backward through autograd,
    with the denominator), median of 21 runs."""
    from flashy_linear_attention_amd.synthetic import WORKLOADS, make_inputs
    from oracle import naive

    q, k, v, do = (t.float() for t in make_inputs(w, seed=1, batch=1, heads=1))
    slices = w.batch * w.heads
    flops_slice = (w.flops_fwd + (w.flops_bwd if w.backward else 0.0)) / slices

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
        if dt >= target_seconds or n >= 1000:
            break

    c1 = WORKLOADS["C1"]
    q1, k1, v1, g1 = make_inputs(c1, seed=0)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q1, k1, v1))

    def c1_step():
        out = naive.linear_attention_normalised(qa, ka, va, eps=1e-5)
        torch.autograd.grad(out, (qa, ka, va), g1)

    for _ in range(3):
        c1_step()
    c1_ms = []
    for _ in range(21):
        t1 = time.perf_counter()
        c1_step()
        c1_ms.append((time.perf_counter() - t1) * 1e3)
    c1_flops = c1.flops_fwd + c1.flops_bwd
    return {
        "value": round(flops_slice * n / dt / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{n} repeats of one (b,h) slice (of the workload's {slices}) at full N={w.seq}, D_qk={w.d_qk}, "
                  f"D_v={w.d_v}, fp32 naive PyTorch fwd{'+bwd' if w.backward else ''}, {dt:.1f} s; "
                  f"os.cpu_count()={os.cpu_count()}, torch threads={torch.get_num_threads()}",
        "ms_per_step_extrapolated": round(dt / n * slices * 1e3, 1),
        "c1": {
            "what": f"C1 in full: fp32 B={c1.batch} H={c1.heads} N={c1.seq} D={c1.d_qk}, naive tril(QK^T)V / "
                    f"((Q*cumsum(K)).sum(-1)+1e-5), forward + backward by autograd, median of {len(c1_ms)} runs",
            "median_ms": round(statistics.median(c1_ms), 3),
            "tflops_causal_counted": round(c1_flops / (statistics.median(c1_ms) * 1e-3) / 1e12, 4),
        },
    }


def _bench_poly(torch, args, w, dev):
    """C4's function, O = tril(phi(xq) phi(xk)^T) V with phi(x) = flatten(x (x) x) / sqrt 2, evaluated
    from the 16-wide x with the polynomial score map f(u) = u^2 / 2, next to the same step on the
    materialised 256-wide features (LinearAttentionSmallVHD's kernels) in the same run."""
    import math

    from flashy_linear_attention_amd.kernels import linear_flash_wrapper_bwd_smallv_hd, linear_flash_wrapper_fwd_smallv_hd
    from flashy_linear_attention_amd.poly import poly_attention_bwd, poly_attention_fwd

    if w.features != "taylor2":
        print("bench.py: --algo poly needs a workload whose q, k are Taylor features (C4)", file=sys.stderr)
        return None
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

    _settle(torch, step, args.settle_seconds)
    for _ in range(args.warmup):
        step()
    ms_step = _time_region(torch, step, args.steps) / args.steps
    ms_fwd = _median_ms(torch, lambda: poly_attention_fwd(xq, xk, v, coef), args.steps)
    ms_bwd = _median_ms(torch, lambda: poly_attention_bwd(do, xq, xk, v, coef), args.steps)
    for _ in range(20):
        plain_step()
    ms_plain = _median_ms(torch, plain_step, args.steps)
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
    return result


def _bench_feature(torch, args, w, dev):
    """The chunk-wise operator from the raw inputs xq, xk (q = elu(xq) + 1, k = elu(xk) + 1 formed while
    the kernels load them, gradients with respect to xq, xk), against the same function built the
    caller's way: elu passes in PyTorch around LinearAttentionChunked, differentiated by autograd."""
    from flashy_linear_attention_amd import FeatureMapLinearAttention, LinearAttentionChunked
    from flashy_linear_attention_amd.feature import feature_attention_bwd, feature_attention_fwd

    if w.features != "elu1" or not w.backward:
        print("bench.py: --algo feature needs a forward + backward workload with elu(x) + 1 features (C3, C5)", file=sys.stderr)
        return None
    gen = torch.Generator().manual_seed(0)
    xq, xk = (torch.randn(w.batch, w.heads, w.seq, w.d_qk, generator=gen).to(w.dtype).to(dev) for _ in range(2))
    v, do = (torch.randn(w.batch, w.heads, w.seq, w.d_v, generator=gen).to(w.dtype).to(dev) for _ in range(2))
    _, q_map, k_map, state = feature_attention_fwd(xq, xk, v, "elu1", want_state=True)

    def fwd():
        return feature_attention_fwd(xq, xk, v, "elu1", want_state=True)

    def bwd():
        return feature_attention_bwd(do, q_map, k_map, v, "elu1", state)

    def step():
        fwd()
        bwd()

    xa, xb, va = (t.detach().clone().requires_grad_(True) for t in (xq, xk, v))

    def autograd_step():
        torch.autograd.grad(FeatureMapLinearAttention.apply(xa, xb, va, "elu1"), (xa, xb, va), do)

    def recipe_step():
        q = torch.nn.functional.elu(xa) + 1
        k = torch.nn.functional.elu(xb) + 1
        torch.autograd.grad(LinearAttentionChunked.apply(q, k, va), (xa, xb, va), do)

    _settle(torch, step, args.settle_seconds)
    for _ in range(args.warmup):
        step()
    ms_step = _time_region(torch, step, args.steps) / args.steps
    ms_fwd, ms_bwd = _median_ms(torch, fwd, args.steps), _median_ms(torch, bwd, args.steps)
    for _ in range(5):
        autograd_step()
        recipe_step()
    ms_auto, ms_recipe = _median_ms(torch, autograd_step, args.steps), _median_ms(torch, recipe_step, args.steps)
    # the plain operator's tensors (xq, xk in place of q, k) plus the by-product q, k written in forward
    bytes_step = w.bytes_fwd + w.bytes_bwd + 2.0 * 2.0 * w.batch * w.heads * w.seq * w.d_qk
    # what the PyTorch passes move on top: forward reads xq, xk and writes q, k; backward reads dq, dk and
    # xq, xk (or the saved q, k) and writes dxq, dxk
    e = float(w.batch * w.heads * w.seq)
    recipe_extra = 2.0 * e * w.d_qk * (4 + 6)
    gbs = bytes_step / (ms_step * 1e-3) / 1e9
    ff, fb = _chunked_flops(w)
    result = {
        "metric": f"causal linear attention with elu(x)+1 applied on load, chunk-wise, fwd+bwd GB/s of algorithmic bytes, "
                  f"B={w.batch} H={w.heads} N={w.seq} D_qk={w.d_qk} D_v={w.d_v}, 1 MI355X",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"{w.name} from its raw inputs: xq, xk, v, dO randn (seed 0), q = elu(xq) + 1, k = elu(xk) + 1 inside "
                        f"the kernels; {_chunk_rows(w)}-row chunks",
            "algorithmic_bytes_per_step": bytes_step,
            "own_tflops": round((ff + fb) / (ms_step * 1e-3) / 1e12, 1),
            "median_ms": {"fwd": round(ms_fwd, 4), "bwd": round(ms_bwd, 4), "autograd_step": round(ms_auto, 4)},
            "pytorch_elu_passes_plus_chunked_operator_autograd_step_ms": round(ms_recipe, 4),
            "speedup_vs_pytorch_elu_passes": round(ms_recipe / ms_auto, 2),
            "bytes_the_pytorch_passes_move_on_top": recipe_extra,
        },
        "roofline": {"bound": "hbm", "kernel": "all kernels of a chunk-wise step with the feature map applied on load",
                     "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes_per_step": bytes_step},
    }
    return result


def main() -> int:
    global BWD_PLAN
    args = _parse()
    BWD_PLAN = args.bwd_plan
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU only (every (batch, head) slice is independent; "
              "no collective exists on this path). Re-run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from flashy_linear_attention_amd import _lib
    from flashy_linear_attention_amd.synthetic import WORKLOADS

    if not torch.cuda.is_available():
        print("bench.py: no ROCm GPU visible", file=sys.stderr)
        return 2
    _lib.load()  # fails loudly if the HIP library is missing

    w = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    if args.sweep:
        return _sweep(torch, dev, min(args.steps, 30))
    if args.crossover:
        return _crossover(torch, dev, min(args.steps, 30))
    if args.algo in ("poly", "feature"):
        rec = (_bench_poly if args.algo == "poly" else _bench_feature)(torch, args, w, dev)
        if rec is None:
            return 2
        print(json.dumps(rec))
        return 0
    normalised = args.algo.startswith("normalised")
    chunked = args.algo in ("chunked", "normalised-chunked")
    o = _ops(torch, w, "chunked" if chunked else "quadratic", dev)
    q, k, v, do = o["q"], o["k"], o["v"], o["do"]
    fwd, bwd = o["fwd_fn"], o["bwd_fn"]
    plain_fwd, plain_bwd = fwd, bwd
    autograd_step = o["autograd_step"]
    if normalised:
        from flashy_linear_attention_amd import LinearAttentionNormalised
        from flashy_linear_attention_amd.normalised import (
            linear_attention_normalised_bwd,
            linear_attention_normalised_fwd,
        )

        # (chunk-wise: forward hands its running state to backward, as the autograd Function does)
        norm_out, norm_denom, norm_state = linear_attention_normalised_fwd(q, k, v, 1e-5, chunked, want_state=True)

        def fwd(q_, k_, v_):
            return linear_attention_normalised_fwd(q_, k_, v_, 1e-5, chunked, want_state=chunked)

        def bwd(do_, q_, k_, v_):
            return linear_attention_normalised_bwd(do_, q_, k_, v_, norm_out, norm_denom, chunked, norm_state)

        qa, ka, va = (t.detach().clone().requires_grad_(True) for t in (q, k, v))

        def autograd_step():
            out = LinearAttentionNormalised.apply(qa, ka, va, 1e-5, chunked)
            if w.backward:
                torch.autograd.grad(out, (qa, ka, va), do)

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

    settle_steps = _settle(torch, step, args.settle_seconds)
    for _ in range(args.warmup):
        step()
    # the timed region: exactly K steps between two synchronisations
    ms_total = _time_region(torch, step, args.steps)
    ms_step = ms_total / args.steps

    # each half alone over a region of K launches (the dominant kernel's average launch duration
    # comes from here), then per-iteration event pairs for the medians
    ms_fwd = _time_region(torch, lambda: fwd(q, k, v), args.steps) / args.steps
    ms_bwd = _time_region(torch, lambda: bwd(do, q, k, v), args.steps) / args.steps if w.backward else None
    med_step = _median_ms(torch, step, args.steps)
    med_fwd = _median_ms(torch, lambda: fwd(q, k, v), args.steps)
    med_bwd = _median_ms(torch, lambda: bwd(do, q, k, v), args.steps) if w.backward else None
    for _ in range(5):
        autograd_step()
    med_autograd = _median_ms(torch, autograd_step, args.steps)

    flops_step = w.flops_fwd + (w.flops_bwd if w.backward else 0.0)
    dt_name = {torch.bfloat16: "bf16", torch.float16: "f16"}[w.dtype]
    peak = PEAK_TFLOPS[dt_name]
    tflops = flops_step / (ms_step * 1e-3) / 1e12

    # The dominant kernel.  Every launch evaluates products Out = mask(X Y^T) Z; one product
    # executes N^2 (D_c + D_o) B H FLOPs (causal-counted).  With equal padded widths up to 128 the
    # three backward products go out as ONE launch of fla::tri_xyt_z_fast_batch_kernel, three
    # quarters of the step: its duration is the backward-only region timed above, its algorithmic
    # FLOPs are the backward's five products (it executes six: dO V^T twice).  Otherwise every
    # product is a launch of its own (two when an output wider than 128 columns meets a <= 64- or
    # 256-wide contraction: one per 128-column half) and the figures are means over the launches
    # of a step.
    def n_launches(dc, dout):
        return 2 if dout > 128 and (dc <= 64 or dc > 128) else 1

    flops_product = float(w.batch * w.heads) * w.seq * w.seq * (w.d_qk + w.d_v)
    batched_bwd = w.backward and _pad(w.d_qk) == _pad(w.d_v) and _pad(w.d_qk) <= 128
    if batched_bwd:
        launches = 2
        kernel_name = "fla::tri_xyt_z_fast_batch_kernel (dQ, dV, dK: three products Out = mask(X Y^T) Z in one launch)"
        flops_launch = w.flops_bwd
        executed_launch = 3.0 * flops_product
        ms_launch = ms_bwd
    else:
        launches = n_launches(w.d_qk, w.d_v)
        if w.backward:
            launches += n_launches(w.d_v, w.d_qk) * 2 + n_launches(w.d_qk, w.d_v)
        products = 1 + (3 if w.backward else 0)
        kernel_name = "fla::tri_xyt_z_fast_kernel (Out = mask(X Y^T) Z), mean over the launches of a step"
        flops_launch = flops_step / launches
        executed_launch = flops_product * products / launches
        ms_launch = ms_step / launches
    if BWD_PLAN == "fused-dkdv" and batched_bwd:
        # two launches: the fused dV + dK kernel and dQ's product; figures below are for the pair of them
        launches = 3
        kernel_name = ("fla::tri_pair_upper_kernel (dV and dK from one stream of (Q, dO) tiles) + fla::tri_xyt_z_fast_kernel "
                       "(dQ): the backward's two launches together")
    achieved = flops_launch / (ms_launch * 1e-3) / 1e12
    executed = executed_launch / (ms_launch * 1e-3) / 1e12
    traffic, traffic_src = PROFILED_TRAFFIC.get((w.name, "quadratic" if BWD_PLAN == "products" else BWD_PLAN), (None, None))
    mfma_ratio, mfma_src = PROFILED_MFMA_RATIO.get((w.name, "quadratic"), (None, None))
    alg_bytes_launch = (w.bytes_bwd if batched_bwd else (w.bytes_fwd + (w.bytes_bwd if w.backward else 0.0)) / launches)

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
            "bwd_plan": BWD_PLAN,
            "clock_settle_steps": settle_steps,
            "fwd_ms": round(ms_fwd, 4),
            "bwd_ms": None if ms_bwd is None else round(ms_bwd, 4),
            "fwd_tflops": round(w.flops_fwd / (ms_fwd * 1e-3) / 1e12, 2),
            "bwd_tflops": None if ms_bwd is None else round(w.flops_bwd / (ms_bwd * 1e-3) / 1e12, 2),
            "pct_of_mfma_peak": round(100.0 * tflops / peak, 2),
            "host_forward_wrapper": _host_side(torch, lambda: fwd(q, k, v)),
            "median_ms": {
                "note": f"medians of {args.steps} iterations, one HIP event pair each; autograd_step = "
                        f"{o['op'].__name__ if not normalised else 'LinearAttentionNormalised'}.apply + torch.autograd.grad",
                "step": round(med_step, 4),
                "fwd": round(med_fwd, 4),
                "bwd": None if med_bwd is None else round(med_bwd, 4),
                "autograd_step": round(med_autograd, 4),
            },
        },
        "roofline": {
            "bound": "mfma",
            "kernel": kernel_name,
            "achieved": round(achieved, 2),
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": round(achieved / peak, 4),
            "traffic": traffic,
            "traffic_source": traffic_src,
            "algorithmic_bytes_per_launch": alg_bytes_launch,
            "traffic_over_algorithmic_bytes": None if traffic is None else round(traffic / alg_bytes_launch, 2),
            "launches_per_step": launches,
            "flops_per_launch": flops_launch,
            "avg_launch_ms": round(ms_launch, 4),
            "executed_tflops": round(executed, 2),
            "executed_frac": round(executed / peak, 4),
            "executed_note": "FLOPs of the product-units the kernel executes (backward: six for the five counted, "
                             "dO V^T is formed for dQ and again for dK)"
                             + ("" if mfma_ratio is None else
                                f"; MFMA operations issued / those FLOPs = {mfma_ratio} ({mfma_src})"),
        },
    }
    if chunked:
        # The chunked path does different (far less) arithmetic, so it is never priced in the
        # quadratic algorithm's FLOPs: its own count, and the HBM roofline that bounds it.
        flops_fwd, flops_bwd = _chunked_flops(w)
        bytes_step = w.bytes_fwd + (w.bytes_bwd if w.backward else 0.0)
        traffic, traffic_src = PROFILED_TRAFFIC.get((w.name, "chunked"), (None, None))
        result["metric"] = result["metric"].replace("TFLOP/s (causal-counted)", "TFLOP/s (chunked algorithm's own FLOPs)")
        result["value"] = round((flops_fwd + flops_bwd) / (ms_step * 1e-3) / 1e12, 2)
        result["config"]["workload"] += f"; chunk-wise evaluation, {_chunk_rows(w)}-row chunks"
        result["config"]["flops_per_step"] = flops_fwd + flops_bwd
        result["config"]["fwd_tflops"] = round(flops_fwd / (ms_fwd * 1e-3) / 1e12, 2)
        result["config"]["bwd_tflops"] = None if ms_bwd is None else round(flops_bwd / (ms_bwd * 1e-3) / 1e12, 2)
        result["config"]["pct_of_mfma_peak"] = round(100.0 * result["value"] / peak, 2)
        gbs = bytes_step / (ms_step * 1e-3) / 1e9
        result["roofline"] = {
            "bound": "hbm",
            "kernel": "all kernels of a chunk-wise step (segment totals and their running sums, the walks over the chunks)",
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_src,
            "algorithmic_bytes_per_step": bytes_step,
            "traffic_over_algorithmic_bytes": None if traffic is None else round(traffic / bytes_step, 2),
        }
    if normalised:
        # What is new are the memory-bound passes around the product kernels.  Their time is the
        # difference to the plain step in this same run, their algorithmic bytes: forward (separate pass)
        # reads q, k, O and writes out (+ n); backward reads g, out (pre-pass, writes dO) and
        # q, k, dq, dk (post-pass, writes dq, dk); 2 bytes per element, fp32 vectors of length N aside.
        from flashy_linear_attention_amd import LinearAttention, LinearAttentionSmallVHD

        def plain_step():
            plain_fwd(q, k, v)
            if w.backward:
                plain_bwd(do, q, k, v)

        ms_plain = _time_region(torch, plain_step, args.steps) / args.steps
        # (with the quadratic product the forward normaliser lives inside the product kernel -- row sums
        # of the scores -- and moves no extra bytes; only the chunk-wise product needs the forward pass)
        e = float(w.batch * w.heads * w.seq)
        # chunk-wise with equal padded head dims up to 128: the walk kernels form n and its gradient terms
        # themselves; what the normaliser must move beyond the plain operator is n (written, read again)
        # and, in backward, the saved output
        in_walk = chunked and _pad(w.d_qk) == _pad(w.d_v) and _pad(w.d_qk) <= 128
        if in_walk:
            nbytes = 4.0 * e + ((4.0 * e + 2.0 * e * w.d_v) if w.backward else 0.0)
        else:
            nbytes = 2.0 * e * (2 * w.d_qk + 2 * w.d_v) if chunked else 4.0 * e
            if w.backward:
                nbytes += 2.0 * e * (3 * w.d_v + 6 * w.d_qk)
        extra_ms = ms_step - ms_plain

        def recipe_step():
            qr, kr, vr = (t.detach().requires_grad_(w.backward) for t in (q, k, v))
            op = LinearAttentionSmallVHD if w.small_v else LinearAttention
            num = op.apply(qr, kr, vr)
            den = (qr * kr.cumsum(-2)).sum(dim=-1, keepdim=True) + 1e-5
            out = num / den
            if w.backward:
                out.backward(do)

        for _ in range(10):
            recipe_step()
        ms_recipe = _time_region(torch, recipe_step, max(10, args.steps // 5)) / max(10, args.steps // 5)
        # the dominant kernel is still the product kernel: its per-launch figures come from the plain step
        if not chunked:
            result["roofline"]["kernel"] = ("fla::tri_xyt_z_fast_kernel / _batch_kernel "
                                            "(all product launches of the plain step)")
            result["roofline"]["avg_launch_ms"] = round(ms_plain / launches, 4)
            result["roofline"]["flops_per_launch"] = flops_step / launches
            result["roofline"]["achieved"] = round(flops_step / (ms_plain * 1e-3) / 1e12, 2)
            result["roofline"]["frac"] = round(result["roofline"]["achieved"] / peak, 4)
            for key in ("executed_tflops", "executed_frac", "executed_note", "traffic", "traffic_source",
                        "algorithmic_bytes_per_launch", "traffic_over_algorithmic_bytes"):
                result["roofline"].pop(key, None)
            result["roofline"]["traffic"] = None
        if in_walk:
            # one fused operator: the whole step against the HBM roofline, in the normalised operator's bytes
            bytes_norm = result["roofline"]["algorithmic_bytes_per_step"] + nbytes
            gbs_norm = bytes_norm / (ms_step * 1e-3) / 1e9
            result["roofline"].update({
                "kernel": "all kernels of a normalised chunk-wise step (dO = g / n and dn, running vectors of k and "
                          "dn q, segment totals, the walks over the chunks)",
                "achieved": round(gbs_norm, 1), "frac": round(gbs_norm / HBM_PEAK_GBS, 4),
                "algorithmic_bytes_per_step": bytes_norm, "traffic": None, "traffic_source": None,
                "traffic_over_algorithmic_bytes": None})
        result["metric"] = result["metric"].replace("causal linear attention", "normalised causal linear attention")
        result["config"]["workload"] += "; fused normaliser out / (q . cumsum(k) + 1e-5)"
        result["config"]["normaliser"] = {
            "plain_step_ms": round(ms_plain, 4),
            "extra_ms": round(extra_ms, 4),
            "algorithmic_bytes": nbytes,
            "gbps": round(nbytes / (extra_ms * 1e-3) / 1e9, 1) if extra_ms > 0 else None,
            "frac_of_hbm_peak": round(nbytes / (extra_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if extra_ms > 0 else None,
            "fused_into_the_product_kernels": bool(in_walk) or not chunked,
            "pytorch_recipe_step_ms": round(ms_recipe, 4),
            "speedup_vs_pytorch_recipe": round(ms_recipe / ms_step, 2),
        }
    if args.workload == "C3" and args.algo == "quadratic" and not args.no_other_workloads:
        # the other benchmark workloads, briefly, so that one run of this script times them all
        del o, q, k, v, do
        torch.cuda.empty_cache()
        result["config"]["other_workloads"] = [
            _other_workload(torch, name, algo, dev, args.other_steps)
            for name, algo in (("C2", "quadratic"), ("C4", "quadratic"), ("C5", "quadratic"),
                               ("C2", "chunked"), ("C3", "chunked"), ("C4", "chunked"), ("C5", "chunked"))
        ] + [
            # the operators beyond the reference's two, each beside the PyTorch recipe it replaces
            _other_extension(torch, name, algo, dev, min(args.other_steps, 30))
            for name, algo in (("C3", "normalised"), ("C3", "normalised-chunked"), ("C5", "normalised-chunked"),
                               ("C3", "feature"), ("C4", "poly"))
        ]
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = _cpu_baseline(torch, w, args.cpu_seconds)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
