#!/usr/bin/env python3
"""Benchmark of the HSTU jagged attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2|C3|C4|C5] [--no-cpu]
                    [--forward-only | --backward --ln-mul --in-linear-silu]

A "step" is one forward over one synthetic jagged batch whose inputs already sit in HBM.
The default workload is the configuration the headline metric is quoted on (C2: bf16, batch 32,
heads 4, head dim 128, lengths uniform in [256, 1024], max_seq_len 1024, alpha 128^-0.5,
silu_scale 1/1024, causal, no rab).

Prints ONE JSON line.  ``value`` is causal-effective TFLOP/s of the whole job
(FLOPs = 2 (d_qk + d_v) N_q sum_b nnz(mask_b); SiLU / bias / mask work is not counted);
``ms_per_step`` is the ms/batch half of the metric.  Launches go through the C ABI
(``hstu_jagged_fwd``, the drop-in boundary) back-to-back on torch's current stream and are
timed with events on that same stream; the cost of one call through the Python entry point
(``ops_rec.ascendc.attention.hstu_jagged``) is reported next to it as ``ms_per_step_python_entry``.

``roofline``     -- dominant (only) kernel against the bf16 dense MFMA peak; ``hbm_*`` fields give the
                    same launch against the HBM bound on compulsory bytes.
``cpu_baseline`` -- the oracle's dense-padded fp32 restatement of the reference's PyTorch golden path,
                    timed on this host's cores on the same batch (a reported baseline, not a target).

After the timed forward steps the same line also carries, each with its own roofline and measured outside the timed
region of the headline: ``backward`` (hstu_jagged_backward on the same workload), ``ln_mul`` (the operator that
consumes the attention output) and ``in_linear_silu`` (the operator that produces U, V, Q, K).  Naming any of
--backward / --ln-mul / --in-linear-silu runs only those; --forward-only runs none.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

_ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(_ROOT, "ops-rec_amd"))
sys.path.insert(0, _ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak (published)
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 MFMA peak (published)
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E bandwidth (published)

INFINITY_CACHE_BYTES = 256 << 20  # MI355X memory-side cache; a working set below it replays out of the cache

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), scaled by the same counters' reading
# of a plain copy kernel of known size: workload -> (bytes, the summary under profiles/ it was read from, sha256 of
# the forward kernel's source at the time).  A figure whose hash no longer matches the source in the tree is stale
# and is reported as null.
MEASURED_TRAFFIC = {
    "C2": (98_400_000, "profiles/hstu_fwd_bf16_d128_C2_trace_and_counters.md", "e5fd7490210191fc"),
    "C3": (301_300_000, "profiles/hstu_fwd_bf16_d128_rab_C3_trace_and_counters.md", "53b56a23cf722f67"),
    "C4": (1_498_000_000, "profiles/hstu_fwd_bf16_d128_rab_C4_trace_and_counters.md", "53b56a23cf722f67"),
    "C5": (846_100_000, "profiles/hstu_fwd_f8e4m3_d128_C5_trace_and_counters.md", "53b56a23cf722f67"),
}
_CSRC = os.path.join(_ROOT, "ops-rec_amd", "csrc")
KERNEL_SOURCE = os.path.join(_CSRC, "hstu_fwd_kernel.hip.h")  # the persistent kernel (and the helpers the others share)
SHORT_KERNEL_SOURCE = os.path.join(_CSRC, "hstu_fwd_short_kernel.hip.h")  # the kernel for short lists


def kernel_source_hash(kernel_name: str = "") -> str:
    """sha256[:16] of the code of the forward kernel that ran (by its name: the kernel for short lists includes the
    persistent kernel's file for its helpers, so both files count for it): the sources with // comments, trailing
    blanks and empty lines removed, so that a figure stays valid when only the comments change."""
    import hashlib
    import re

    code = []
    for path in (KERNEL_SOURCE, SHORT_KERNEL_SOURCE) if kernel_name.endswith("_short") else (KERNEL_SOURCE,):
        with open(path, "r", encoding="utf-8") as f:
            lines = [re.sub(r"\s*//.*$", "", line.rstrip()) for line in f]
        code.append("\n".join(line for line in lines if line.strip()))
    return hashlib.sha256("\n".join(code).encode()).hexdigest()[:16]


def measured_traffic(workload: str, kernel_name: str = ""):
    """(bytes or None, where the figure comes from)."""
    if workload not in MEASURED_TRAFFIC:
        return None, "not measured"
    nbytes, source, sha = MEASURED_TRAFFIC[workload]
    now = kernel_source_hash(kernel_name)
    if sha != now:
        return None, f"stale: {source} was taken with kernel source {sha or '?'}, the tree has {now}"
    return nbytes, f"{source} (kernel source {sha})"


def algorithmic_bytes(w, out_element_size: int) -> int:
    """Compulsory HBM traffic: Q, K, V read once, O written once, visible rab elements read once."""
    es = w.q.element_size()
    n = w.q.numel() * es + w.k.numel() * es + w.v.numel() * es
    n += w.q.shape[0] * w.q.shape[1] * w.v.shape[2] * out_element_size
    n += w.seq_offset.numel() * w.seq_offset.element_size()
    return n


# HBM bytes per ln_mul launch by rows (cols 512, bf16), from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a plain
# copy of known size (profiles/ln_mul_bf16_c512_trace_and_counters.md)
# (m, n, k) -> bytes, same method (profiles/in_linear_silu_bf16_trace_and_counters.md)
IN_LINEAR_SILU_MEASURED_TRAFFIC_BYTES = {(16384, 9216, 64): 622_400_000, (20292, 2048, 512): 204_000_000}


LN_MUL_MEASURED_TRAFFIC_BYTES = {20292: 62_457_000, 324672: 997_512_000}


def bench_ln_mul(attn_out, stream, args):
    """ln_mul through ``ln_mul_fwd`` of the C ABI, events on the launch stream.  Algorithmic bytes per launch:
    x and u read once, out written once = 3 * rows * cols * element size (gamma / beta stay in cache)."""
    import ctypes

    import numpy as np
    import torch

    from ops_rec import _native
    from oracle import ln_mul_oracle

    lib = _native.load()
    dev = attn_out.device
    tokens, cols = attn_out.shape[0], attn_out.shape[1] * attn_out.shape[2]
    cases = []
    for rows in (tokens, 16 * tokens):
        x = attn_out.reshape(tokens, cols).repeat(rows // tokens, 1).contiguous()
        u = torch.randn(rows, cols, device=dev).to(x.dtype)
        gamma, beta = torch.randn(cols, device=dev), torch.randn(cols, device=dev)
        out = torch.empty_like(x)
        p = _native.new_ln_mul_params()
        p.x, p.u, p.gamma, p.beta, p.out = (t.data_ptr() for t in (x, u, gamma, beta, out))
        p.rows, p.cols = rows, cols
        p.dtype = _native.DT_BF16 if x.dtype == torch.bfloat16 else _native.DT_FP16
        p.affine_dtype = _native.DT_FP32
        p.epsilon = ln_mul_oracle.EPSILON
        raw = ctypes.c_void_p(stream.cuda_stream)
        n = max(50, args.steps)
        settle(lambda: lib.ln_mul_fwd(ctypes.byref(p), raw), args.settle_ms)
        for _ in range(10):
            assert lib.ln_mul_fwd(ctypes.byref(p), raw) == 0, _native.last_error()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n):
            lib.ln_mul_fwd(ctypes.byref(p), raw)
        e1.record(stream)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / n * 1e3
        nbytes = 3 * rows * cols * x.element_size()
        case = {
            "rows": rows,
            "cols": cols,
            "kernel": lib.ln_mul_fwd_kernel_name(ctypes.byref(p)).decode(),
            "avg_launch_us": round(us, 3),
            "algorithmic_bytes": nbytes,
            "roofline": {"bound": "hbm", "achieved": round(nbytes / us / 1e3, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4),
                         "traffic": LN_MUL_MEASURED_TRAFFIC_BYTES.get(rows) if cols == 512 else None},
        }  # fmt: skip
        if rows == tokens and not args.no_cpu:
            # CPU: the numpy oracle (float64) on a sample of rows, single-threaded numpy
            sample = min(rows, 4096)
            f = lambda t: t[:sample].float().cpu().numpy()  # noqa: E731
            xs, us_, gs, bs = f(x), f(u), gamma.cpu().numpy(), beta.cpu().numpy()
            t0 = time.perf_counter()
            want = ln_mul_oracle.ln_mul(xs, us_, gs, bs)
            cpu_s = time.perf_counter() - t0
            np.testing.assert_allclose(out[:sample].double().cpu().numpy(), want, rtol=2.0**-8, atol=2e-3)
            case["cpu_baseline"] = {"value": round(3 * sample * cols * x.element_size() / cpu_s / 1e9, 3),
                                    "unit": "GB/s", "cores": 1, "kind": "port",
                                    "sample": f"first {sample} rows, numpy float64 oracle"}  # fmt: skip
        cases.append(case)
        del x, u, out
    return {"note": "ln_mul_fwd of the C ABI back-to-back on one stream; x = the attention output as [tokens, heads * dim]",
            "cases": cases}  # fmt: skip


def settle(launch, ms):
    """Keeps the device busy with `launch` for about `ms` milliseconds (untimed), so that what is timed next starts with
    the clocks where sustained work holds them."""
    import torch

    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(32):
            launch()
        torch.cuda.synchronize()


def bench_in_linear_silu(tokens, width, stream, args):
    """in_linear_silu through ``in_linear_silu_fwd`` of the C ABI, events on the launch stream.  Algorithmic bytes per
    launch: x, weight and bias read once, linear_output and the four splits written once =
    2 (m k + n k) + 4 n + 4 m n; flops 2 m n k."""
    import ctypes

    import torch

    from ops_rec import _native
    from oracle import in_linear_silu_oracle

    lib = _native.load()
    dev = torch.device("cuda", 0)
    cases = []
    # (m, n, k): a shape of the reference's own test (test_in_linear_silu.py:127-130), store-bound; and the layer of
    # this workload: its tokens, embedding `width` = heads x dim of the attention workload -> U, V, Q, K of `width` each
    for m, n, k, what in ((16384, 9216, 64, "reference test shape"), (tokens, 4 * width, width, "layer of this workload")):
        x = torch.randn(m, k, device=dev).to(torch.bfloat16)
        wt = (torch.randn(n, k, device=dev) / k**0.5).to(torch.bfloat16)
        bias = torch.randn(n, device=dev)
        split = [n // 4] * 4
        outs = [torch.empty(m, s, dtype=torch.bfloat16, device=dev) for s in split + [n]]
        p = _native.new_in_linear_silu_params()
        p.x, p.weight, p.bias = x.data_ptr(), wt.data_ptr(), bias.data_ptr()
        p.user, p.value, p.query, p.key, p.linear_output = (t.data_ptr() for t in outs)
        p.m, p.n, p.k = m, n, k
        for i, s_ in enumerate(split):
            p.split[i] = s_
        p.dtype = _native.DT_BF16
        raw = ctypes.c_void_p(stream.cuda_stream)
        # (at least 100 launches behind 20 untimed ones: the layer shape is bound by the core clock, which takes a few
        # milliseconds of work to settle after the host-side gaps between the legs -- 25 launches show 86-90 us, 100 show 70-72)
        n_it = max(100, args.steps // 2)
        settle(lambda: lib.in_linear_silu_fwd(ctypes.byref(p), raw), args.settle_ms)
        for _ in range(20):
            assert lib.in_linear_silu_fwd(ctypes.byref(p), raw) == 0, _native.last_error()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n_it):
            lib.in_linear_silu_fwd(ctypes.byref(p), raw)
        e1.record(stream)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / n_it * 1e3
        nbytes = 2 * (m * k + n * k) + 4 * n + 4 * m * n
        flops = 2 * m * n * k
        hbm_bound = nbytes / PEAK_HBM_GBS / 1e3 > flops / PEAK_BF16_TFLOPS / 1e6  # the longer of the two floors, in us
        roof = ({"bound": "hbm", "achieved": round(nbytes / us / 1e3, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                 "frac": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4)} if hbm_bound else
                {"bound": "mfma", "achieved": round(flops / us / 1e6, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                 "frac": round(flops / us / 1e6 / PEAK_BF16_TFLOPS, 4)})  # fmt: skip
        roof["traffic"] = IN_LINEAR_SILU_MEASURED_TRAFFIC_BYTES.get((m, n, k))
        case = {"m": m, "n": n, "k": k, "shape": what,
                "kernel": lib.in_linear_silu_fwd_kernel_name(ctypes.byref(p)).decode(), "avg_launch_us": round(us, 3),
                "algorithmic_bytes": nbytes, "flops": flops, "GBs": round(nbytes / us / 1e3, 1),
                "tflops": round(flops / us / 1e6, 1), "roofline": roof}  # fmt: skip
        if not args.no_cpu:
            sample = 256
            xs, ws, bs = x[:sample].cpu(), wt.cpu(), bias.cpu()
            t0 = time.perf_counter()
            want = in_linear_silu_oracle.in_linear_silu(xs, ws, bs, split, round_to=torch.bfloat16)
            cpu_s = time.perf_counter() - t0
            torch.testing.assert_close(outs[4][:sample].double().cpu(), want[4], rtol=2.0**-7, atol=1e-2)
            torch.testing.assert_close(outs[2][:sample].double().cpu(), want[2], rtol=2.0**-6, atol=1e-2)
            case["cpu_baseline"] = {"value": round(2 * sample * n * k / cpu_s / 1e12, 5), "unit": "TFLOP/s",
                                    "cores": torch.get_num_threads(), "kind": "port",
                                    "sample": f"first {sample} rows, float64 torch oracle"}  # fmt: skip
        cases.append(case)
        del x, wt, outs
    return {"note": "in_linear_silu_fwd of the C ABI back-to-back on one stream, bf16", "cases": cases}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C2", choices=["C2", "C3", "C4", "C5"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--ln-mul", action="store_true",
                    help="also time ln_mul (LayerNorm(x) * u, the operator that consumes the attention output) on the "
                    "output of this workload viewed as [tokens, heads * dim] and on a matrix 16 times as tall, and add "
                    "an 'ln_mul' object with its HBM roofline to the line")  # fmt: skip
    ap.add_argument("--in-linear-silu", action="store_true",
                    help="also time in_linear_silu (the linear + SiLU + split that produces U, V, Q, K in front of "
                    "attention) on one of the reference's test shapes and on the layer shape of this workload, and "
                    "add an 'in_linear_silu' object with its rooflines to the line")  # fmt: skip
    ap.add_argument("--backward", action="store_true",
                    help="also time hstu_jagged_backward (the HIP backward kernels) on the same workload and add a "
                    "'backward' object to the line (bf16 workloads only)")  # fmt: skip
    ap.add_argument("--forward-only", action="store_true",
                    help="time the attention forward only; by default (none of --backward / --ln-mul / --in-linear-silu "
                    "given) the line also carries the 'backward', 'ln_mul' and 'in_linear_silu' objects")
    ap.add_argument("--settle-ms", type=float, default=30.0,
                    help="milliseconds of untimed launches ahead of each leg's warm-up launches (0: none)")
    ap.add_argument("--no-cold", action="store_true",
                    help="skip the cold-cache loop (profiler runs: every traced launch is then one of the timed loop's)")
    ap.add_argument("--drop-rab", action="store_true",
                    help="run the workload without its attn_bias (C3, C4): the difference of a counter run with and "
                    "one without is the HBM traffic that the bias stream alone causes")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="after the timed steps also run 5 plain device-to-device copies of this many MiB, so that a "
                    "counter run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) can be scaled by a kernel of known traffic")  # fmt: skip
    args = ap.parse_args()
    if args.gpus != 1:
        print(
            "bench.py: this build runs on one GPU only (sequences and heads are independent, so the "
            "path shards with no communication; nothing here uses a second GPU). Use --gpus 1.",
            file=sys.stderr,
        )
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the operator has no CPU path", file=sys.stderr)
        return 1

    import ops_rec
    from ops_rec import _ops, workloads
    from oracle import hstu_oracle as oracle  # FLOP model + cpu_baseline leg only

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    heavy = args.workload != "C2"
    w_cpu = None if heavy else workloads.config(args.workload)
    w = workloads.config(args.workload, device=dev) if heavy else w_cpu.to(dev)
    if args.drop_rab:
        w.attn_bias = None
    n_q, d_qk, d_v = w.q.shape[1], w.q.shape[2], w.v.shape[2]
    ctx = None if w.num_context is None else w.num_context.cpu()
    tgt = None if w.num_target is None else w.num_target.cpu()
    flops = oracle.causal_effective_flops(w.seq_offset.cpu(), None, n_q, d_qk, d_v, w.mask_type, ctx, tgt,
                                          w.target_group_size)  # fmt: skip
    nnz = flops // (2 * (d_qk + d_v) * n_q)
    fp8 = args.workload == "C5"  # fp8-e4m3 inputs with per-head scales, bf16 output
    extra = {}
    if fp8:
        (q8, qs), (k8, ks), (v8, vs) = (workloads.quantize_fp8(t) for t in (w.q, w.k, w.v))
        w.q, w.k, w.v = q8, k8, v8
        extra = dict(out_dtype=torch.bfloat16, q_descale=qs, k_descale=ks, v_descale=vs)
    prepared = _ops.prepare_forward(
        w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, w.max_seq_len, w.silu_scale, w.seq_offset,
        w.seq_offset, w.num_context, w.num_target, w.target_group_size, w.alpha, **extra,
    )  # fmt: skip
    alg_bytes = algorithmic_bytes(w, prepared.out.element_size())
    rab_bytes = 0
    if w.attn_bias is not None:
        rab_bytes = nnz * n_q * w.attn_bias.element_size()
    alg_bytes += rab_bytes
    kernel_name = prepared.kernel_name()
    stream = torch.cuda.current_stream(dev)
    raw_stream = stream.cuda_stream

    # ---- GPU: K launches through the C ABI, events on the launch stream ----
    # (ahead of the W warm-up launches the device is kept busy for --settle-ms: the first millisecond or two of work
    # after an idle period runs 4-5 % slower than the launches behind it, and K = 20 launches last under a millisecond)
    settle(lambda: prepared.launch(raw_stream), args.settle_ms)
    for _ in range(args.warmup):
        prepared.launch(raw_stream)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(args.steps):
        prepared.launch(raw_stream)
    e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = e0.elapsed_time(e1) / args.steps
    ms_per_step = max(wall_ms, ev_ms)  # the slower clock: host-bound launches cannot hide

    # ---- the same with cold caches: the timed loop above replays one set of buffers, and a working set below the
    # 256 MiB memory-side cache is then served out of that cache, not out of HBM.  Here independent copies of the
    # inputs (own outputs, own workspaces), together more than twice the cache, take turns, so that every launch
    # finds its rows in HBM only.
    cold_ms, cold_sets = None, 0
    if alg_bytes <= INFINITY_CACHE_BYTES and not args.no_cold:
        cold_sets = max(4, -(-(5 * INFINITY_CACHE_BYTES // 2) // alg_bytes))
        clones = []
        for _ in range(cold_sets):
            wc = w.to(dev)  # (.to() on the same device returns the same storage: clone what the kernel reads)
            wc.q, wc.k, wc.v = wc.q.clone(), wc.k.clone(), wc.v.clone()
            if wc.attn_bias is not None:
                wc.attn_bias = wc.attn_bias.clone()
            clones.append(_ops.prepare_forward(
                wc.q, wc.k, wc.v, wc.mask, wc.attn_bias, wc.mask_type, wc.max_seq_len, wc.max_seq_len, wc.silu_scale,
                wc.seq_offset, wc.seq_offset, wc.num_context, wc.num_target, wc.target_group_size, wc.alpha, **extra,
            ))  # fmt: skip
        for i in range(max(cold_sets, args.warmup)):
            clones[i % cold_sets].launch(raw_stream)
        torch.cuda.synchronize()
        e0.record(stream)
        for i in range(args.steps):
            clones[i % cold_sets].launch(raw_stream)
        e1.record(stream)
        torch.cuda.synchronize()
        cold_ms = e0.elapsed_time(e1) / args.steps
        del clones

    if args.calibration_copy_mib > 0:
        src = torch.empty(args.calibration_copy_mib << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- the same through the Python entry point ----
    if fp8:
        def op(*_):
            return ops_rec.hstu_jagged_fp8(w.q, w.k, w.v, qs, ks, vs, mask_type=w.mask_type, max_seq_len=w.max_seq_len,
                                           silu_scale=w.silu_scale, seq_offset=w.seq_offset, alpha=w.alpha)  # fmt: skip
        op_args = ()
    else:
        op = ops_rec.ascendc.attention.hstu_jagged
        op_args = w.op_args()
    for _ in range(5):
        op(*op_args)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_py = max(50, args.steps // 4)
    for _ in range(n_py):
        op(*op_args)
    torch.cuda.synchronize()
    py_ms = (time.perf_counter() - t0) * 1e3 / n_py

    peak = PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    kernel_tflops = flops / (ev_ms * 1e-3) / 1e12
    result = {
        "metric": "HSTU attn fwd ms/batch + causal TFLOPS (% MFMA peak), B32 H4 d128 L1024 bf16",
        "value": round(tflops, 3),
        "unit": "TFLOP/s (causal-effective)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3" if fp8 else "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: jagged causal HSTU attention fwd, B{len(w.lengths)} H{n_q} d{d_qk}, "
            f"lengths {min(w.lengths)}..{max(w.lengths)} (T={sum(w.lengths)}), max_seq_len {w.max_seq_len}, "
            f"rab={'yes' if w.attn_bias is not None else 'no'}, seed 0",
            "flops_per_step": flops,
            "algorithmic_bytes_per_step": alg_bytes,
            "launch_path": "C ABI hstu_jagged_fwd, back-to-back on one stream",
        },
        "ms_per_step_cold": None if cold_ms is None else round(cold_ms, 6),
        "value_cold": None if cold_ms is None else round(flops / (cold_ms * 1e-3) / 1e12, 3),
        "cold_note": (f"{cold_sets} independent input / output sets of {alg_bytes / 1e6:.0f} MB take turns "
                      f"({cold_sets * alg_bytes / 1e6:.0f} MB against a 256 MiB memory-side cache); 'value' and "
                      "'ms_per_step' replay one set" if cold_ms is not None else
                      "skipped (--no-cold)" if args.no_cold else
                      "one set already exceeds the 256 MiB memory-side cache: the timed loop is cold as it is"),
        "ms_per_step_events": round(ev_ms, 6),
        "ms_per_step_wall": round(wall_ms, 6),
        "ms_per_step_python_entry": round(py_ms, 6),
        "roofline": {
            "bound": "mfma",
            "kernel": kernel_name,
            "achieved": round(kernel_tflops, 3),
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": round(kernel_tflops / peak, 4),
            "traffic": None if args.drop_rab else measured_traffic(args.workload, kernel_name)[0],
            "traffic_source": "not measured" if args.drop_rab else measured_traffic(args.workload, kernel_name)[1],
            "kernel_source_hash": kernel_source_hash(kernel_name),
            "clock": "HIP events on the launch stream around the timed launches (the fraction of the peak is quoted "
                     "on this clock only; 'value' and 'ms_per_step' are the host's clock around the same launches)",
            "avg_launch_us": round(ev_ms * 1e3, 3),
            "hbm_achieved_GBs": round(alg_bytes / (ev_ms * 1e-3) / 1e9, 1),
            "hbm_peak_GBs": PEAK_HBM_GBS,
            "hbm_frac": round(alg_bytes / (ev_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "rab_read_GBs": round(rab_bytes / (ev_ms * 1e-3) / 1e9, 1) if rab_bytes else None,
        },
    }

    # The operators either side of the forward: the ones asked for, or all of them when none is named.  The headline
    # numbers above are complete at this point; a leg that fails reports its error instead of its figures.
    asked = args.backward or args.ln_mul or args.in_linear_silu
    legs = {name: (getattr(args, name) if asked else not args.forward_only) for name in ("backward", "ln_mul", "in_linear_silu")}

    def guarded(name, fn):
        try:
            result[name] = fn()
        except Exception as exc:  # noqa: BLE001
            result[name] = {"error": f"{type(exc).__name__}: {exc}"[:300]}

    # ---- backward: d q, d k, d v (and d attn_bias) through the operator ----
    def bench_backward():
        grad = torch.randn(prepared.out.shape, device=dev).to(prepared.out.dtype)
        zeros = None if w.num_context is None and w.num_target is None else torch.zeros(len(w.lengths), dtype=w.seq_offset.dtype, device=dev)
        bwd_args = (grad, w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, w.silu_scale, w.seq_offset,
                    w.num_context if w.num_context is not None else zeros, w.num_target if w.num_target is not None else zeros,
                    w.target_group_size, w.alpha)  # fmt: skip
        bwd = ops_rec.ascendc.attention.hstu_jagged_backward
        n_bwd = max(50, args.steps // 4)
        settle(lambda: bwd(*bwd_args), args.settle_ms)
        for _ in range(10):
            bwd(*bwd_args)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(n_bwd):
            bwd(*bwd_args)
        e1.record(stream)
        torch.cuda.synchronize()
        bwd_ms = e0.elapsed_time(e1) / n_bwd
        bwd_flops = flops * 5 // 2  # five products (S, dP, dV, dK, dQ) against the forward's two
        return {
            "ms_per_step": round(bwd_ms, 6),
            "steps": n_bwd,
            "flops_per_step": bwd_flops,
            "tflops": round(bwd_flops / (bwd_ms * 1e-3) / 1e12, 3),
            "pct_of_bf16_mfma_peak": round(100.0 * bwd_flops / (bwd_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 2),
            "note": "through torch.ops.ops_rec.hstu_jagged_backward, in the order the library picks for the shape: on this "
            "workload hstu_bwd_dq_kernel storing dS and P, then hstu_bwd_dkv_kernel with a dV and a dK workgroup per key "
            "tile that read them back (the five products of the formula issued once each); with an attn_bias gradient, "
            "head dims up to 64 or long rows two or three launches that recompute S (and dP)",
        }

    if legs["backward"] and not fp8:
        guarded("backward", bench_backward)
    # ---- ln_mul: the operator that takes the attention output next in an HSTU layer ----
    if legs["ln_mul"] and not fp8:
        guarded("ln_mul", lambda: bench_ln_mul(prepared.out, stream, args))
    # ---- in_linear_silu: the operator that produces U, V, Q, K in front of attention ----
    if legs["in_linear_silu"] and not fp8:
        guarded("in_linear_silu", lambda: bench_in_linear_silu(sum(w.lengths), n_q * d_v, stream, args))

    # ---- CPU baseline: dense-padded fp32 golden path on this host's cores ----
    if not args.no_cpu and w_cpu is not None:
        cores = os.cpu_count() or 1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            pass
        cores_available = cores
        cores = min(cores, 16)  # the share of the host a one-GPU box gives a job
        torch.set_num_threads(cores)
        kw = w_cpu.oracle_kwargs()
        args_cpu = (w_cpu.q.float(), w_cpu.k.float(), w_cpu.v.float())
        oracle.hstu_jagged_forward_dense(*args_cpu, **kw)  # warm-up
        times = []
        budget_end = time.perf_counter() + 25.0
        while len(times) < 5 and time.perf_counter() < budget_end:
            t0 = time.perf_counter()
            oracle.hstu_jagged_forward_dense(*args_cpu, **kw)
            times.append(time.perf_counter() - t0)
        times.sort()
        med = times[len(times) // 2]
        t0 = time.perf_counter()
        oracle.hstu_jagged_forward(*args_cpu, **kw)
        per_seq = time.perf_counter() - t0
        result["cpu_baseline"] = {
            "value": round(flops / med / 1e12, 5),
            "unit": "TFLOP/s (causal-effective)",
            "cores": cores,
            "cores_available": cores_available,
            "cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": f"the full {args.workload} batch, dense-padded fp32 torch path, median of {len(times)} runs "
            "after 1 warm-up",
            "ms_per_batch": round(med * 1e3, 2),
            "ms_per_batch_per_sequence_variant": round(per_seq * 1e3, 2),
        }
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
