#!/usr/bin/env python3
"""The three operators of an HSTU layer's attention block on one MI355X, chained in bf16 with no cast in between:

    U, V, Q, K, _ = in_linear_silu(x, W, b, [H*D] * 4)          # ops_rec.ascendc.activation
    O = hstu_jagged(Q, K, V as [T, H, D], ..., seq_offset)        # ops_rec.ascendc.attention
    Y = ln_mul(O as [T, H*D], U, gamma, beta)                     # ops_rec.ascendc.activation

(the sequence of the reference's operator list, docs/zh/ops_rec_api.md:41-43, with its HSTU attention in the middle).

    python hstu_layer_example.py [--batch 32] [--heads 4] [--dim 128] [--embed 512] [--lo 256] [--hi 1024] [--steps 50]

Checks the chain against the same chain in fp32 torch operations on the device, then times it; prints one JSON line
with the time of each operator, of the block through the Python entry points, and of the block replayed from a HIP graph.
"""

import argparse
import json
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import ops_rec  # noqa: E402


def block(x, w, b, gamma, beta, offsets, heads, dim, max_len):
    act, att = ops_rec.ascendc.activation, ops_rec.ascendc.attention
    hd = heads * dim
    u, v, q, k, _ = act.distance_in_linear_silu(x, w, b, [hd] * 4)
    t = x.shape[0]
    o = att.hstu_jagged(q.view(t, heads, dim), k.view(t, heads, dim), v.view(t, heads, dim), None, None, 0, max_len,
                        1.0 / max_len, offsets, None, None, 0, dim**-0.5)  # fmt: skip
    return act.ln_mul(o.view(t, hd), u, gamma, beta)


def block_fp32(x, w, b, gamma, beta, offsets, heads, dim, max_len):
    """The same chain in fp32 torch operations, one sequence at a time (rounding to bf16 where the operators do)."""
    hd = heads * dim
    rt = lambda t_: t_.to(torch.bfloat16).float()  # noqa: E731
    mixed = rt(x.float() @ w.float().t() + b)
    u, v, q, k = (rt(t_) for t_ in torch.split(torch.nn.functional.silu(mixed), [hd] * 4, dim=-1))
    out = torch.zeros(x.shape[0], heads, dim, device=x.device)
    for s, e in zip(offsets[:-1].tolist(), offsets[1:].tolist()):
        qs, ks, vs = (t_[s:e].view(e - s, heads, dim).transpose(0, 1) for t_ in (q, k, v))
        p = torch.nn.functional.silu(qs @ ks.transpose(1, 2) * dim**-0.5) / max_len
        out[s:e] = (torch.tril(p) @ vs).transpose(0, 1)
    o = rt(out).view(-1, hd)
    return torch.nn.functional.layer_norm(o, (hd,), gamma, beta, 1e-5) * u


def timed(fn, steps):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps * 1e3


def graph_replay_us(fn, steps):
    """The same calls captured once in a HIP graph and replayed: what a serving loop pays per block."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return timed(graph.replay, steps)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--heads", type=int, default=4)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--embed", type=int, default=512)
    ap.add_argument("--lo", type=int, default=256)
    ap.add_argument("--hi", type=int, default=1024)
    ap.add_argument("--steps", type=int, default=50)
    args = ap.parse_args()
    dev = torch.device("cuda", 0)
    g = torch.Generator(device=dev).manual_seed(0)
    lengths = torch.randint(args.lo, args.hi + 1, (args.batch,), generator=torch.Generator().manual_seed(0))
    offsets = torch.zeros(args.batch + 1, dtype=torch.int32)
    offsets[1:] = lengths.cumsum(0)
    offsets = offsets.to(dev)
    t, hd = int(lengths.sum()), args.heads * args.dim
    x = torch.randn(t, args.embed, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(4 * hd, args.embed, generator=g, device=dev) / args.embed**0.5).to(torch.bfloat16)
    b = torch.randn(4 * hd, generator=g, device=dev) * 0.1
    gamma = 1.0 + 0.1 * torch.randn(hd, generator=g, device=dev)
    beta = 0.1 * torch.randn(hd, generator=g, device=dev)
    common = (x, w, b, gamma, beta, offsets, args.heads, args.dim, args.hi)

    y = block(*common)
    want = block_fp32(*common)
    err = (y.float() - want).abs().max().item()
    scale = want.abs().max().item()
    # LayerNorm divides by the spread of an attention output row, which is small: a bf16 rounding of O is amplified
    assert err <= 0.05 * scale, (err, scale)

    act, att = ops_rec.ascendc.activation, ops_rec.ascendc.attention
    u, v, q, k, _ = act.distance_in_linear_silu(x, w, b, [hd] * 4)
    q3, k3, v3 = (t_.view(t, args.heads, args.dim) for t_ in (q, k, v))
    o = att.hstu_jagged(q3, k3, v3, None, None, 0, args.hi, 1.0 / args.hi, offsets, None, None, 0, args.dim**-0.5)
    us = {
        "in_linear_silu_us": timed(lambda: act.distance_in_linear_silu(x, w, b, [hd] * 4), args.steps),
        "hstu_jagged_us": timed(lambda: att.hstu_jagged(q3, k3, v3, None, None, 0, args.hi, 1.0 / args.hi, offsets, None,
                                                        None, 0, args.dim**-0.5), args.steps),  # fmt: skip
        "ln_mul_us": timed(lambda: act.ln_mul(o.view(t, hd), u, gamma, beta), args.steps),
        "block_us": timed(lambda: block(*common), args.steps),
        "block_graph_replay_us": graph_replay_us(lambda: block(*common), args.steps),
        "fp32_torch_chain_us": timed(lambda: block_fp32(*common), 2),
    }
    print(json.dumps({"tokens": t, "batch": args.batch, "heads": args.heads, "dim": args.dim, "embed": args.embed,
                      "max_abs_err_vs_fp32_chain": err, "max_abs_value": scale,
                      **{k_: round(v_, 1) for k_, v_ in us.items()}}))  # fmt: skip


if __name__ == "__main__":
    main()
