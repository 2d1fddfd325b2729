#!/usr/bin/env python3
"""``hstu_paged`` on one MI355X: the call of the reference's example
(ascendc/attention/hstu_v1/hstu_forward_v1/examples/torch/test_torch_hstu_forward_paged.py:34-100), then a serving-shaped
call that is timed:

    python hstu_paged_example.py [--batch 32] [--cached 4096] [--new 64] [--targets 32] [--page-size 128] [--steps 50]

Per sequence ``cached`` rows already sit in pages of the KV cache, ``new`` history rows and ``targets`` candidate rows
are the queries; the keys are the cached rows, the new rows (appended to the cache by the caller, as in the
reference's flow, so they are in pages too) and the target rows from ``k`` / ``v``.  Prints one JSON line with the time
per call and the K / V bytes streamed per second.
"""

import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import ops_rec  # noqa: E402


def build_case(hist, prev, targets, page_size, heads, dim, dtype, device, seed=0):
    g = torch.Generator(device=device).manual_seed(seed)
    q_lens = [h + t for h, t in zip(hist, targets)]
    k_lens = [p + h + t for p, h, t in zip(prev, hist, targets)]
    total = sum(q_lens)
    rnd = lambda *shape: (torch.randn(*shape, generator=g, device=device) * 0.3).to(dtype)  # noqa: E731
    cached = [p + h for p, h in zip(prev, hist)]
    pages = [(c + page_size - 1) // page_size for c in cached]
    order = torch.randperm(sum(pages), generator=torch.Generator().manual_seed(seed)).tolist()
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int32, device=device)  # noqa: E731
    last = [c % page_size if c % page_size else page_size for c in cached]
    return dict(
        q=rnd(total, heads, dim), k=rnd(total, heads, dim), v=rnd(total, heads, dim),
        kv_cache=rnd(sum(pages), 2, page_size, heads, dim), mask_type=0, max_seq_len=max(q_lens), max_seq_len_k=max(k_lens),
        seq_offset=offs(q_lens), seq_offset_k=offs(k_lens), seq_offset_t=offs(targets), page_offsets=offs(pages),
        page_ids=torch.tensor(order, dtype=torch.int32, device=device),
        last_page_len=torch.tensor(last, dtype=torch.int32, device=device),
        num_target=torch.tensor(targets, dtype=torch.int32, device=device), target_group_size=1,
    )  # fmt: skip


def call(c, **extra):
    kw = {n: t for n, t in c.items() if n not in ("q", "k", "v", "kv_cache")}
    return ops_rec.ascendc.attention.hstu_paged(c["q"], c["k"], c["v"], c["kv_cache"], **kw, **extra)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--cached", type=int, default=4096)
    ap.add_argument("--new", type=int, default=64)
    ap.add_argument("--targets", type=int, default=32)
    ap.add_argument("--page-size", type=int, default=128)
    ap.add_argument("--heads", type=int, default=4)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--steps", type=int, default=50)
    args = ap.parse_args()
    dev = torch.device("cuda:0")

    # the reference example: N 4, D 32, page 32, histories 32 and 48, 4 and 6 targets, fp16
    small = build_case([32, 48], [0, 0], [4, 6], 32, 4, 32, torch.float16, dev)
    y = call(small, silu_scale=1.0 / 54)
    assert y.shape == small["q"].shape and torch.isfinite(y).all()

    b = args.batch
    c = build_case([args.new] * b, [args.cached] * b, [args.targets] * b, args.page_size, args.heads, args.dim,
                   torch.bfloat16, dev)  # fmt: skip
    for _ in range(5):
        call(c, alpha=args.dim**-0.5)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        call(c, alpha=args.dim**-0.5)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / args.steps * 1e3
    kv_bytes = b * (args.cached + args.new + args.targets) * args.heads * args.dim * 2 * 2
    print(json.dumps({
        "op": "hstu_paged", "dtype": "bf16", "batch": b, "heads": args.heads, "head_dim": args.dim, "page_size": args.page_size,
        "cached_rows": args.cached, "new_rows": args.new, "target_rows": args.targets, "us_per_call": round(us, 2),
        "kv_bytes": kv_bytes, "kv_GBs": round(kv_bytes / us / 1e3, 1), "hbm_frac": round(kv_bytes / us / 1e3 / 8000.0, 4),
    }))  # fmt: skip


if __name__ == "__main__":
    main()
