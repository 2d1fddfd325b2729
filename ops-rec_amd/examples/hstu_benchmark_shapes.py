#!/usr/bin/env python3
"""Forward and backward of ``hstu_jagged`` on the shapes of the reference's own operator benchmark
(ascendc/attention/hstu_v2/test/pytest/test_backward_op_benchmark.py:183-197 "user case 1", :244-258 "user case 2":
every sequence at the full length, causal mask, no context / targets), one JSON line per shape:

    python hstu_benchmark_shapes.py [--case 1|2|all] [--only INDEX[,INDEX...]] [--budget-ms 300]

The reference runs these under msprof and extracts the task duration per operator
(hstu_v2/test/pytest/run_benchmark.sh:17-31, utils/perf_stats.py); here each operator call is timed with events on
the stream, repeated until ``--budget-ms`` of GPU time has been spent (at least twice).  TFLOP/s are causal-effective:
2 (d_qk + d_v) per visible (query, key) pair for the forward, 2.5 times that for the backward.
"""

import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import ops_rec  # noqa: E402

CASE_1 = [  # batch, heads, (d_qk, d_v), (S_q, S_k), rab, dtype
    (2048, 4, (64, 64), (52, 1000), False, torch.float16),
    (16, 4, (64, 64), (501, 1000), False, torch.float16),
    (8, 8, (128, 128), (8000, 8000), False, torch.float16),
    (8, 8, (256, 256), (8000, 8000), False, torch.float16),
    (2048, 2, (256, 256), (32, 32), False, torch.float16),
    (96, 2, (256, 256), (512, 3072), False, torch.float16),
    (16, 4, (64, 32), (32, 499), False, torch.float16),
    (4, 4, (128, 48), (1001, 901), False, torch.float16),
    (128, 4, (128, 128), (7621, 7621), False, torch.bfloat16),
    (96, 3, (256, 256), (674, 674), False, torch.bfloat16),
]
CASE_2 = [(32, 8, (d, d), (s, s), rab, dt) for s in (512, 1024, 2048, 4096) for d in (32, 64, 128, 256)
          for rab in (False, True) for dt in (torch.float16, torch.bfloat16)]  # fmt: skip


def visible_pairs(s_q, s_k):
    # row i sees keys 0 .. i + (s_k - s_q), clipped to [0, s_k]
    delta = s_k - s_q
    return sum(min(max(i + delta + 1, 0), s_k) for i in range(s_q))


def timed(fn, budget_ms):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    fn()
    e1.record()
    torch.cuda.synchronize()
    once = max(e0.elapsed_time(e1), 1e-3)
    n = max(2, min(200, int(budget_ms / once)))
    e0.record()
    for _ in range(n):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n, n


def run(batch, heads, dims, lens, rab, dtype, budget_ms):
    dev = torch.device("cuda", 0)
    (d_qk, d_v), (s_q, s_k) = dims, lens
    g = torch.Generator(device=dev).manual_seed(123)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device=dev) * 0.3).to(dtype)  # noqa: E731
    q, k, v = rnd(batch * s_q, heads, d_qk), rnd(batch * s_k, heads, d_qk), rnd(batch * s_k, heads, d_v)
    offs_q = torch.arange(0, (batch + 1) * s_q, s_q, dtype=torch.int32, device=dev)
    offs_k = torch.arange(0, (batch + 1) * s_k, s_k, dtype=torch.int32, device=dev)
    bias = (torch.randn(batch, heads, s_q, s_k, generator=g, device=dev) * 0.1).to(dtype) if rab else None
    att = ops_rec.ascendc.attention
    scale, alpha = 1.0 / s_q, d_qk**-0.5
    if s_q == s_k:
        fwd = lambda: att.hstu_jagged(q, k, v, None, bias, 0, s_q, scale, offs_q, None, None, 0, alpha)  # noqa: E731
    else:
        fwd = lambda: att.hstu_jagged(q, k, v, None, bias, 0, s_q, s_k, scale, offs_q, offs_k, None, None, 0, alpha)  # noqa: E731
    out = fwd()
    grad = torch.randn(out.shape, generator=g, device=dev).to(dtype)
    if s_q == s_k:
        bwd = lambda: att.hstu_jagged_backward(grad, q, k, v, None, bias, 0, s_q, scale, offs_q, None, None, 0, alpha)  # noqa: E731
    else:
        bwd = lambda: att.hstu_jagged_backward(grad, q, k, v, None, bias, 0, s_q, s_k, scale, offs_q, offs_k, None, None, 0, alpha)  # noqa: E731
    flops = 2 * (d_qk + d_v) * heads * batch * visible_pairs(s_q, s_k)
    f_ms, f_n = timed(fwd, budget_ms)
    b_ms, b_n = timed(bwd, budget_ms)
    return {"batch": batch, "heads": heads, "d_qk": d_qk, "d_v": d_v, "s_q": s_q, "s_k": s_k, "rab": rab,
            "dtype": str(dtype)[6:], "fwd_ms": round(f_ms, 4), "fwd_tflops": round(flops / f_ms / 1e9, 1), "fwd_calls": f_n,
            "bwd_ms": round(b_ms, 4), "bwd_tflops": round(2.5 * flops / b_ms / 1e9, 1), "bwd_calls": b_n}  # fmt: skip


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--case", default="all", choices=["1", "2", "all"])
    ap.add_argument("--only", default="", help="positions in the chosen list, comma-separated (all when empty)")
    ap.add_argument("--budget-ms", type=float, default=300.0)
    args = ap.parse_args()
    shapes = (CASE_1 if args.case in ("1", "all") else []) + (CASE_2 if args.case in ("2", "all") else [])
    if args.only:
        shapes = [shapes[int(i)] for i in args.only.split(",")]
    for shape in shapes:
        try:
            print(json.dumps(run(*shape, args.budget_ms)), flush=True)
        except RuntimeError as exc:  # a shape this build refuses, or one that does not fit the memory
            print(json.dumps({"shape": str(shape), "error": str(exc)[:200]}), flush=True)
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
