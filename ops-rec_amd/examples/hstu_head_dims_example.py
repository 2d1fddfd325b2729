#!/usr/bin/env python3
"""Forward and backward of ``hstu_jagged`` at head dims beyond the tuned kernels' range (the reference takes q/k head
dims in [1, 512] and v head dims in [16, 512] in steps of 16, hstu_forward_v1/op_host/tiling_policy.cpp:68-93), and
the backward of fp32 inputs: one JSON line per case with the kernel that ran, the time per call (events on the stream)
and the causal-effective TFLOP/s (backward = 2.5 x the forward's flops).

    python hstu_head_dims_example.py [--calls 10]
"""

import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import ops_rec  # noqa: E402
from ops_rec import _ops, workloads  # noqa: E402

CASES = [  # name, dtype, batch, heads, head dim, shortest and longest sequence, attn_bias
    ("bf16 d512", torch.bfloat16, 8, 4, 512, 100, 1024, False),
    ("bf16 d384", torch.bfloat16, 8, 4, 384, 2048, 2048, False),
    ("fp16 d512 with attn_bias", torch.float16, 16, 8, 512, 1024, 1024, True),
    ("bf16 d260 / 272 (q/k head dim not a multiple of 8)", torch.bfloat16, 8, 4, (260, 272), 100, 512, False),
    ("fp32 d64", torch.float32, 8, 4, 64, 100, 512, False),
    ("fp32 d128", torch.float32, 16, 4, 128, 100, 1024, False),
]


def timed(fn, calls):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(calls):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / calls


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--calls", type=int, default=10)
    args = ap.parse_args()
    dev = torch.device("cuda", 0)
    for name, dtype, batch, heads, dim, lo, hi, rab in CASES:
        d_qk, d_v = dim if isinstance(dim, tuple) else (dim, dim)
        w = workloads.make("x", dtype=dtype, device=dev, batch=batch, heads=heads, dim=d_qk, dim_v=d_v, lo=lo, hi=hi,
                           std=0.5, rab_std=0.3 if rab else None)  # fmt: skip
        prepared = _ops.prepare_forward(w.q, w.k, w.v, None, w.attn_bias, 0, w.max_seq_len, w.max_seq_len, w.silu_scale,
                                        w.seq_offset, w.seq_offset, None, None, 0, w.alpha)  # fmt: skip
        grad = torch.randn(w.q.shape[0], heads, d_v, device=dev).to(dtype)
        att = ops_rec.ascendc.attention
        bwd = lambda: att.hstu_jagged_backward(grad, w.q, w.k, w.v, None, w.attn_bias, 0, w.max_seq_len, w.silu_scale,
                                               w.seq_offset, None, None, 0, w.alpha)  # noqa: E731  # fmt: skip
        f_ms = timed(prepared.launch, args.calls)
        b_ms = timed(bwd, max(2, args.calls // 2))
        flops = 2 * (d_qk + d_v) * heads * sum(n * (n + 1) // 2 for n in w.lengths)
        print(json.dumps({"case": name, "forward_kernel": prepared.kernel_name(), "fwd_ms": round(f_ms, 4),
                          "fwd_tflops": round(flops / f_ms / 1e9, 2), "bwd_ms": round(b_ms, 4),
                          "bwd_tflops": round(2.5 * flops / b_ms / 1e9, 2)}), flush=True)  # fmt: skip


if __name__ == "__main__":
    main()
