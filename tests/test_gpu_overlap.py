"""Forward launches that overlap on one GPU.  The variants that pull work items from device counters (per-XCD
queues for long lists, split items for short ones) keep the counters in the caller's workspace, cleared on the launch
stream ahead of the kernel, and the plain variant has none: launches in flight at the same time, on several streams or
as replays of captured graphs on different streams, must each give bit for bit what the same call gives alone.
Every kernel in these tests runs to its normal end."""

import pytest
import torch

import ops_rec
import helpers
from ops_rec import _ops, workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def prepared(w):
    return _ops.prepare_forward(w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, w.max_seq_len,
                                w.silu_scale, w.seq_offset, w.seq_offset, w.num_context, w.num_target,
                                w.target_group_size, w.alpha)  # fmt: skip


def cases():
    mk = workloads.make
    bf = torch.bfloat16
    return {
        # long jagged list: the variant with per-XCD queues
        "queues": lambda s: mk("q", dtype=bf, device=DEV, seed=s, batch=48, heads=4, dim=128, lo=200, hi=2000),
        # two long sequences: split items (arrival counters and partial outputs in the workspace)
        "split": lambda s: mk("s", dtype=bf, device=DEV, seed=s, batch=2, heads=2, dim=128, lo=2500, hi=3000),
        # a list in between: the plain variant, no counters (with the kernel for short lists switched off), and the
        # same list on that kernel
        "plain": lambda s: mk("p", dtype=bf, device=DEV, seed=s, batch=24, heads=4, dim=128, lo=100, hi=900),
        "short": lambda s: mk("p", dtype=bf, device=DEV, seed=s, batch=24, heads=4, dim=128, lo=100, hi=900),
    }


@pytest.mark.parametrize("name", ["queues", "split", "plain", "short"])
def test_many_launches_in_flight_on_several_streams(name, monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None if name == "short" else "0")
    make = cases()[name]
    n_calls, n_streams = 72, 6  # more launches in flight than the 64 counter sets an earlier design shared
    inputs = [make(seed) for seed in range(4)]
    serial = []
    for w in inputs:
        p = prepared(w)
        assert name in ("plain",) or name in p.kernel_name()
        assert name != "plain" or not p.kernel_name().endswith(("_queues", "_short"))
        serial.append(p.launch().clone())
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=DEV) for _ in range(n_streams)]
    calls = [prepared(inputs[i % len(inputs)]) for i in range(n_calls)]  # own output and workspace each
    torch.cuda.synchronize()
    for i, p in enumerate(calls):
        with torch.cuda.stream(streams[i % n_streams]):
            p.launch()
    torch.cuda.synchronize()
    for i, p in enumerate(calls):
        assert torch.equal(p.out, serial[i % len(inputs)]), f"{name}: call {i} differs from the serial result"


@pytest.mark.parametrize("name", ["queues", "split"])
def test_two_captured_forwards_replayed_at_once(name):
    make = cases()[name]
    w_a, w_b = make(11), make(12)
    want_a, want_b = prepared(w_a).launch().clone(), prepared(w_b).launch().clone()
    torch.cuda.synchronize()
    p_a, p_b = prepared(w_a), prepared(w_b)
    graphs = []
    for p in (p_a, p_b):
        s = torch.cuda.Stream(device=DEV)
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            p.launch()  # warm-up outside capture
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            p.launch()
        graphs.append(g)
    s_a, s_b = torch.cuda.Stream(device=DEV), torch.cuda.Stream(device=DEV)
    for _ in range(4):
        p_a.out.zero_()
        p_b.out.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(s_a):
            graphs[0].replay()
        with torch.cuda.stream(s_b):
            graphs[1].replay()
        eager = prepared(w_a).launch()  # the program's own eager work beside the replays
        torch.cuda.synchronize()
        assert torch.equal(p_a.out, want_a) and torch.equal(p_b.out, want_b) and torch.equal(eager, want_a)
