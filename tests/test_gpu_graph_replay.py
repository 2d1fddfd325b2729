"""The operators under HIP graph capture: a captured chain (in_linear_silu -> hstu_jagged -> ln_mul, a short-list
forward that takes the split variant with its device-side counters, and the backward in each of its launch orders) is
replayed several times, with eager work and
synchronisations of the program's own between the replays, and every replay is compared with the eager result bit for
bit.  Nothing in these entry points allocates device memory behind torch's back or clears memory with a memset node:
outputs and workspaces come from torch's allocator (its graph-private pool during capture), and the counter block at
the head of a workspace is cleared by a small kernel on the launch stream ahead of the forward."""

import pytest
import torch

import ops_rec
from ops_rec import workloads
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def layer_inputs(lengths, heads, dim, embed, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    offsets = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32, device=DEV)
    t, hd = sum(lengths), heads * dim
    x = torch.randn(t, embed, generator=g, device=DEV).to(torch.bfloat16)
    w = (torch.randn(4 * hd, embed, generator=g, device=DEV) / embed**0.5).to(torch.bfloat16)
    b = torch.randn(4 * hd, generator=g, device=DEV) * 0.1
    gamma = 1.0 + 0.1 * torch.randn(hd, generator=g, device=DEV)
    beta = 0.1 * torch.randn(hd, generator=g, device=DEV)
    return x, w, b, gamma, beta, offsets


def block(x, w, b, gamma, beta, offsets, heads, dim, max_len):
    act, att = ops_rec.ascendc.activation, ops_rec.ascendc.attention
    hd, t = heads * dim, x.shape[0]
    u, v, q, k, _ = act.distance_in_linear_silu(x, w, b, [hd] * 4)
    o = att.hstu_jagged(q.view(t, heads, dim), k.view(t, heads, dim), v.view(t, heads, dim), None, None, 0, max_len,
                        1.0 / max_len, offsets, None, None, 0, dim**-0.5)  # fmt: skip
    return act.ln_mul(o.view(t, hd), u, gamma, beta)


def replay_and_compare(fn, static_inputs, fresh_inputs):
    """Captures fn(*static_inputs), then for each set of fresh values copies them into the static tensors, replays,
    and compares with an eager call on the same values."""
    s = torch.cuda.Stream(device=DEV)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):  # warm-up outside capture (library load, allocator)
            fn(*static_inputs)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = fn(*static_inputs)
    for values in fresh_inputs:
        for dst, src in zip(static_inputs, values):
            if torch.is_tensor(dst):
                dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = captured.clone()
        want = fn(*values)  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want)


def test_layer_chain_replays():
    heads, dim, embed, lengths = 4, 128, 256, [300, 77, 512, 129, 1]
    sets = [layer_inputs(lengths, heads, dim, embed, seed) for seed in range(4)]
    static = tuple(t.clone() for t in sets[0]) + (heads, dim, max(lengths))
    fresh = [tuple(s) + (heads, dim, max(lengths)) for s in sets[1:]] + [tuple(sets[0]) + (heads, dim, max(lengths))]
    replay_and_compare(block, static, fresh)


def test_split_variant_replays():
    # one long sequence: the forward cuts its items into parts, with arrival counters at the head of its workspace
    # that a fill kernel ahead of it clears -- at every replay as at the capture
    def make(seed):
        w = workloads.make("long", dtype=torch.bfloat16, device=DEV, seed=seed, batch=1, heads=2, dim=128, lo=3000, hi=3000)
        return w

    ws = [make(s) for s in range(3)]

    def fwd(q, k, v, offsets):
        return ops_rec.ascendc.attention.hstu_jagged(q, k, v, None, None, 0, 3000, 1.0 / 3000, offsets, None, None, 0, 128**-0.5)

    static = (ws[0].q.clone(), ws[0].k.clone(), ws[0].v.clone(), ws[0].seq_offset.clone())
    fresh = [(w.q, w.k, w.v, w.seq_offset) for w in ws[1:]] + [(ws[0].q, ws[0].k, ws[0].v, ws[0].seq_offset)]
    replay_and_compare(fwd, static, fresh)


@pytest.mark.parametrize("order", ["0", "1", "2"], ids=["two_launches", "three_launches", "planes"])
@pytest.mark.parametrize("rab", [False, True], ids=["norab", "rab"])
def test_backward_replays_in_every_launch_order(order, rab, monkeypatch):
    # the backward's launch orders under capture: fills are kernels, the workspace through which the query-tile kernel
    # hands dS (and P) on comes from torch's graph-private pool and is never cleared; the gradients of every replay are
    # compared with eager calls on the same values
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
    max_len = 520

    def make(seed):
        return workloads.make("bwd", dtype=torch.bfloat16, device=DEV, seed=seed, batch=3, heads=2, dim=128, lo=100, hi=max_len,
                              max_seq_len=max_len, std=0.5, silu_scale=1.0, rab_std=0.5 if rab else None)  # fmt: skip

    ws = [make(s) for s in range(3)]
    rows = max(w.q.shape[0] for w in ws)

    def padded(t):  # (the same number of rows in every set: lengths differ between the seeds)
        return torch.cat([t, torch.zeros(rows - t.shape[0], *t.shape[1:], dtype=t.dtype, device=DEV)])

    def bwd(grad, q, k, v, bias, offsets):
        got = ops_rec.ascendc.attention.hstu_jagged_backward(grad, q, k, v, None, bias, 0, max_len, max_len, 1.0, offsets,
                                                             offsets, None, None, 0, 128**-0.5)  # fmt: skip
        return torch.cat([g.float().flatten() for g in got if g is not None])

    def inputs(w, seed):
        g = torch.Generator(device=DEV).manual_seed(100 + seed)
        grad = torch.randn(rows, 2, 128, generator=g, device=DEV).to(torch.bfloat16)
        return (grad, padded(w.q), padded(w.k), padded(w.v), w.attn_bias, w.seq_offset)

    sets = [inputs(w, i) for i, w in enumerate(ws)]
    static = tuple(t.clone() if torch.is_tensor(t) else t for t in sets[0])
    replay_and_compare(bwd, static, sets[1:] + [sets[0]])
