"""Times ``hstu_jagged_backward`` in each of its launch orders over a list of shapes and prints, per shape, the three
times, the order the library's rule takes and how far that is from the best (markdown table on stdout).

    python ops-rec_amd/examples/hstu_bwd_order_sweep.py [--set heldout|fit|bias] [--launches 10]
    python ops-rec_amd/examples/hstu_bwd_order_sweep.py --shape 1,4,4,128,1024,1024,causal [--bias] --only planes   # one shape, one
                                                        # order: what a kernel trace or a counter run of a launch order wants

Orders (forced with HSTU_MI355_BWD_HANDOFF = 0 / 1 / 2, read once per process, hence ``reload_switches``):
  two     key-tile kernel (S, dP, dV, dK) + query-tile kernel (S, dP, dQ): 7 products, no workspace
  three   dV kernel (S, dV) + query-tile kernel storing dS (S, dP, dQ) + dK from dS: 6 products, 2 bytes per pair
          written and read
  planes  query-tile kernel storing dS and P (S, dP, dQ) + dV from P / dK from dS: 5 products, 4 bytes per pair
Shapes are (batch, query heads, K/V heads, head dim, shortest, longest, mask); lengths uniform in [shortest, longest],
max_seq_len = longest rounded up to 8.  The set ``bias`` runs with an attn_bias and asks for its gradient (there the
three-launch order hands dS over through that gradient and needs no workspace).
"""

import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import ops_rec  # noqa: E402
from ops_rec import _native, _ops, workloads  # noqa: E402

# the shapes the rule's constants were fitted on
FIT = [
    (32, 4, 4, 128, 256, 1024, "causal"), (32, 4, 4, 128, 1024, 1024, "causal"), (8, 4, 4, 128, 1024, 1024, "causal"),
    (64, 4, 4, 128, 512, 512, "causal"), (128, 4, 4, 128, 1024, 1024, "causal"), (256, 4, 4, 128, 256, 256, "causal"),
    (16, 4, 4, 128, 512, 2048, "causal"), (8, 4, 4, 128, 2048, 2048, "causal"), (16, 4, 4, 128, 4096, 4096, "causal"),
    (32, 4, 4, 64, 256, 1024, "causal"), (128, 4, 4, 64, 1024, 1024, "causal"), (32, 8, 8, 64, 128, 512, "causal"),
    (32, 4, 4, 256, 256, 1024, "causal"), (64, 2, 2, 256, 1024, 1024, "causal"), (8, 4, 4, 256, 256, 2048, "causal"),
    (32, 4, 4, 128, 256, 1024, "none"), (128, 4, 4, 128, 512, 512, "none"), (4, 4, 4, 128, 1024, 1024, "causal"),
]
# shapes the constants never saw
HELDOUT = [
    (24, 4, 4, 128, 1024, 1024, "causal"), (48, 4, 4, 128, 128, 1024, "causal"), (12, 8, 8, 128, 512, 1536, "causal"),
    (96, 2, 2, 128, 256, 768, "causal"), (200, 4, 4, 128, 64, 384, "causal"), (6, 4, 4, 128, 2048, 2048, "causal"),
    (20, 8, 2, 128, 300, 1200, "causal"), (512, 4, 4, 128, 128, 128, "causal"), (10, 4, 4, 128, 3000, 4096, "causal"),
    (40, 4, 4, 128, 700, 900, "causal"), (16, 16, 16, 128, 256, 512, "causal"), (64, 8, 8, 128, 64, 512, "causal"),
    (3, 4, 4, 128, 1500, 2048, "causal"), (160, 4, 4, 128, 512, 768, "causal"), (28, 4, 4, 96, 256, 1280, "causal"),
    (48, 4, 4, 64, 512, 1024, "causal"), (256, 4, 4, 64, 128, 512, "causal"), (16, 8, 8, 64, 1024, 2048, "causal"),
    (64, 4, 2, 64, 256, 256, "causal"), (12, 4, 4, 64, 2048, 4096, "causal"), (400, 2, 2, 32, 64, 256, "causal"),
    (24, 4, 4, 256, 512, 1024, "causal"), (96, 4, 4, 256, 256, 512, "causal"), (8, 8, 8, 256, 1024, 1024, "causal"),
    (4, 4, 4, 256, 2048, 4096, "causal"), (128, 2, 2, 192, 128, 640, "causal"), (48, 4, 4, 128, 512, 512, "none"),
    (16, 4, 4, 128, 1024, 2048, "none"), (96, 4, 4, 64, 256, 512, "none"), (12, 4, 4, 256, 512, 1024, "none"),
    (32, 4, 4, 128, 900, 1100, "causal"), (72, 4, 4, 128, 256, 640, "causal"), (1, 8, 8, 128, 4096, 4096, "causal"),
    (2, 4, 4, 128, 8192, 8192, "causal"),
]
# with an attn_bias and its gradient
BIAS = [
    (8, 4, 4, 128, 512, 1024, "causal"), (16, 4, 4, 96, 256, 1024, "causal"), (16, 4, 4, 64, 128, 512, "causal"),
    (32, 8, 8, 64, 512, 512, "causal"), (32, 4, 4, 64, 256, 1024, "causal"), (64, 4, 4, 128, 256, 1024, "causal"),
    (32, 4, 4, 128, 278, 1004, "causal"), (8, 4, 4, 256, 512, 1024, "causal"), (32, 4, 4, 192, 256, 1024, "causal"),
    (8, 8, 8, 128, 1024, 2048, "causal"), (32, 4, 4, 64, 100, 1504, "causal"), (128, 4, 4, 64, 64, 512, "causal"),
]
NAMES = {"0": "two", "1": "three", "2": "planes"}


def time_us(fn, launches):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(3):
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / launches)
    return best


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--set", default="heldout", choices=["heldout", "fit", "bias"])
    ap.add_argument("--launches", type=int, default=10)
    ap.add_argument("--shape", action="append", default=[],
                    help="batch,heads,kv_heads,dim,shortest,longest,causal|none (repeatable); instead of --set")
    ap.add_argument("--bias", action="store_true", help="run the shapes of --shape with an attn_bias and its gradient")
    ap.add_argument("--only", choices=sorted(NAMES.values()), help="run this launch order only and print its time")
    args = ap.parse_args()
    bwd = ops_rec.ascendc.attention.hstu_jagged_backward
    asked = []
    new_workspace = _ops._new_workspace
    _ops._new_workspace = lambda n, dev: (asked.append(n), new_workspace(n, dev))[1]
    print("| batch, heads (K/V), head dim, lengths, mask | two us | three us | planes us | rule | rule / best |")
    print("|---|---|---|---|---|---|")
    worst, within = 0.0, 0
    shapes = {"heldout": HELDOUT, "fit": FIT, "bias": BIAS}[args.set]
    if args.shape:
        shapes = [tuple(int(v) for v in t.split(",")[:6]) + (t.split(",")[6],) for t in args.shape]
    for batch, heads, heads_k, dim, lo, hi, mask in shapes:
        max_len = (hi + 7) // 8 * 8
        w = workloads.make("sweep", dtype=torch.bfloat16, device="cuda", batch=batch, heads=heads, heads_k=heads_k, dim=dim,
                           lo=lo, hi=hi, max_seq_len=max_len, seed=batch + hi)  # fmt: skip
        grad = (torch.randn(w.q.shape[0], heads, dim, device="cuda") * 0.1).to(torch.bfloat16)
        rab = None
        if args.bias if args.shape else args.set == "bias":
            rab = (torch.randn(batch, heads, max_len, max_len, device="cuda") * 0.1).to(torch.bfloat16)
        call = (grad, w.q, w.k, w.v, None, rab, 0 if mask == "causal" else 2, max_len, w.silu_scale, w.seq_offset, None, None, 0, w.alpha)
        times = {}
        if args.only:
            os.environ["HSTU_MI355_BWD_HANDOFF"] = {v: k for k, v in NAMES.items()}[args.only]
            _native.reload_switches()
            print(f"| {batch}, {heads} ({heads_k}), {dim}, {lo}..{hi}, {mask} | {args.only} only: "
                  f"{time_us(lambda: bwd(*call), args.launches):.1f} us |", flush=True)  # fmt: skip
            continue
        for order in ("0", "1", "2", None):
            if order is None:
                os.environ.pop("HSTU_MI355_BWD_HANDOFF", None)
            else:
                os.environ["HSTU_MI355_BWD_HANDOFF"] = order
            _native.reload_switches()
            del asked[:]
            times[order] = time_us(lambda: bwd(*call), args.launches)
            if order is None:
                dense = batch * heads * max_len * max_len * 2
                if rab is None:
                    pick = "two" if asked[-1] == 0 else ("three" if asked[-1] == dense else "planes")
                else:  # (two and three both run without a workspace: told apart by their times below)
                    pick = "planes" if asked[-1] else None
        # (a forced order falls back to another when its workspace is over the limit: its time is then that order's)
        best = min(times[o] for o in ("0", "1", "2"))
        if pick is None:
            pick = "two" if abs(times[None] - times["0"]) <= abs(times[None] - times["1"]) else "three"
        picked = times[{v: k for k, v in NAMES.items()}[pick]]
        ratio = picked / best
        worst, within = max(worst, ratio), within + (ratio <= 1.10)
        print(f"| {batch}, {heads} ({heads_k}), {dim}, {lo}..{hi}, {mask} | {times['0']:.1f} | {times['1']:.1f} | {times['2']:.1f} | "
              f"{pick} ({times[None]:.1f}) | {ratio:.2f} |", flush=True)  # fmt: skip
    if args.only:
        return
    print(f"\nrule within 10 % of the best order on {within} of {len(shapes)} shapes; worst {worst:.2f}x")


if __name__ == "__main__":
    main()
