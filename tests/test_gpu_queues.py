"""Launches large enough for the kernel variant with per-XCD work queues (host rule: the upper bound on the
number of (query tile, sequence, head) items is at least four per resident workgroup), in both of its item
orders and with queues that start out empty.

A schedule must not change a single bit of any output row: every sequence of the big launch is also run on its
own (a short list, served by the variant without queues) and compared exactly; the shortest sequence is
compared with the CPU oracle as well.
"""

import pytest
import torch

import ops_rec
from ops_rec import workloads
from oracle import hstu_oracle as O
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(w):
    out = ops_rec.ascendc.attention.hstu_jagged(*w.op_args())
    torch.cuda.synchronize()
    return out


def alone(w, b):
    """Sequence b of (device) workload w as a one-sequence workload."""
    offs = w.seq_offset.cpu().tolist()
    r0, r1 = offs[b], offs[b + 1]
    pick = lambda t: None if t is None else t[b : b + 1]  # noqa: E731
    return workloads.Workload(
        name="one", q=w.q[r0:r1], k=w.k[r0:r1], v=w.v[r0:r1],
        seq_offset=torch.tensor([0, r1 - r0], dtype=w.seq_offset.dtype, device=w.q.device), max_seq_len=w.max_seq_len,
        silu_scale=w.silu_scale, alpha=w.alpha, attn_bias=pick(w.attn_bias), mask=pick(w.mask), mask_type=w.mask_type,
        num_context=pick(w.num_context), num_target=pick(w.num_target), target_group_size=w.target_group_size,
        lengths=[r1 - r0],
    ), (r0, r1)  # fmt: skip


CASES = {
    # jagged, many pairs, grouped K/V heads: per-pair order, every queue busy
    "jagged_gqa": dict(batch=64, heads=8, heads_k=2, dim=64, lo=1, hi=2048, max_seq_len=2048),
    # all sequences equally long: per-tile order (one shared queue) inside the queue variant
    "uniform": dict(batch=32, heads=8, heads_k=8, dim=128, lo=1024, hi=1024, max_seq_len=1024),
    # four pairs only (one K/V head): queues 4..7 are empty from the start, their workgroups go and help
    "few_pairs": dict(heads=16, heads_k=1, dim=128, lengths=[8192, 1024, 4096, 3072], max_seq_len=8192, batch=4, lo=0, hi=0),
    # context rows and grouped targets with the per-pair order
    "jagged_targets": dict(batch=48, heads=8, heads_k=8, dim=128, lo=64, hi=2048, max_seq_len=2048, num_context=6,
                           max_target=40, target_group_size=3),
    # all sequences equally long and six items per workgroup: per-pair order all the same
    "uniform_many": dict(batch=48, heads=8, heads_k=8, dim=128, lo=1024, hi=1024, max_seq_len=1024),
    # the head-dim slot 32 (four workgroups per CU)
    "jagged_d32": dict(batch=64, heads=8, heads_k=4, dim=32, lo=1, hi=2048, max_seq_len=2048),
    # the head-dim slot 256 (one workgroup per CU): jagged with a bias, and equally long sequences
    "jagged_d256_rab": dict(batch=40, heads=4, heads_k=2, dim=256, lo=1, hi=2048, max_seq_len=2048, rab_std=0.2),
    "uniform_d256": dict(batch=32, heads=8, heads_k=8, dim=256, lo=1024, hi=1024, max_seq_len=1024),
    # context rows with the per-tile order: the first tile of every pair stands ahead of the top tiles
    "uniform_contexts": dict(batch=32, heads=8, heads_k=8, dim=128, lo=1024, hi=1024, max_seq_len=1024, num_context=9),
}  # fmt: skip


@pytest.mark.parametrize("name", list(CASES))
def test_schedule_does_not_change_results(name, monkeypatch):
    # (a sequence run on its own is a short list; without this, its long items would be split over workgroups,
    # which changes the order of the fp32 sums and with it the last bit of some outputs)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")  # (keys up to 1024 would go to the kernel for short lists)
    w = workloads.make(name, dtype=torch.bfloat16, device=DEV, seed=5, **CASES[name])
    out = run(w)
    assert torch.isfinite(out.float()).all()
    order = sorted(range(len(w.lengths)), key=lambda b: w.lengths[b])
    picks = sorted(set(order[:2] + order[-2:] + order[len(order) // 2 : len(order) // 2 + 1]))
    for b in picks:
        one, (r0, r1) = alone(w, b)
        if r1 == r0:
            continue
        assert torch.equal(run(one), out[r0:r1]), (name, b, w.lengths[b])
    # the shortest non-empty sequence against the oracle
    b = next(b for b in order if w.lengths[b] > 0)
    one, (r0, r1) = alone(w, b)
    c = one.to("cpu")
    ref = O.hstu_jagged_forward(c.q, c.k, c.v, out_dtype=torch.float32, **c.oracle_kwargs())
    torch.testing.assert_close(out[r0:r1].float().cpu(), ref, atol=1e-2, rtol=1e-2)
    assert torch.equal(run(w), out)  # and the same bits again


@pytest.mark.parametrize("dim", [128, 256])
def test_fp8_long_list_matches_sequences_run_alone(dim, monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")
    w = workloads.make("f8", dtype=torch.bfloat16, device=DEV, seed=7, batch=64, heads=8, heads_k=2, dim=dim, lo=1,
                       hi=2048, max_seq_len=2048)  # fmt: skip
    (q8, qs), (k8, ks), (v8, vs) = (workloads.quantize_fp8(t) for t in (w.q, w.k, w.v))
    kw = dict(mask_type=0, max_seq_len=w.max_seq_len, silu_scale=w.silu_scale, alpha=w.alpha)
    out = ops_rec.hstu_jagged_fp8(q8, k8, v8, qs, ks, vs, seq_offset=w.seq_offset, **kw)
    offs = w.seq_offset.cpu().tolist()
    order = sorted(range(len(w.lengths)), key=lambda b: w.lengths[b])
    for b in order[:2] + order[-2:]:
        r0, r1 = offs[b], offs[b + 1]
        one = torch.tensor([0, r1 - r0], dtype=w.seq_offset.dtype, device=DEV)
        got = ops_rec.hstu_jagged_fp8(q8[r0:r1], k8[r0:r1], v8[r0:r1], qs, ks, vs, seq_offset=one, **kw)
        assert torch.equal(got, out[r0:r1])
