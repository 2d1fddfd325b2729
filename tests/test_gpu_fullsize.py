"""Full-size configurations (C2, C3, C4) on the GPU.

The CPU oracle cannot finish these sizes in seconds, so they are checked through
  * the oracle on a sub-batch: a few sequences cut out of the batch must reproduce exactly the rows the
    full launch wrote for them (sequences are independent), and those rows are compared with the oracle;
  * size-independent properties: linearity in V, zero bias == no bias, bitwise reproducibility,
    invariance to a permutation of the sequences, every row written exactly once (NaN-prefilled output).
"""

import pytest
import torch

import ops_rec
from ops_rec import workloads
from oracle import hstu_oracle as O
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def launch(w):
    out = ops_rec.ascendc.attention.hstu_jagged(*w.op_args())
    torch.cuda.synchronize()
    return out


def sub_batch(w, seqs):
    """The sequences ``seqs`` of workload ``w`` (device tensors) as a CPU workload of their own."""
    offs = w.seq_offset.cpu().tolist()
    rows = torch.cat([torch.arange(offs[b], offs[b + 1]) for b in seqs])
    lens = [offs[b + 1] - offs[b] for b in seqs]
    new_offs = [0]
    for n in lens:
        new_offs.append(new_offs[-1] + n)
    pick = lambda t: None if t is None else t[torch.tensor(seqs, device=t.device)].cpu()  # noqa: E731
    sub = workloads.Workload(
        name="sub", q=w.q[rows.to(w.q.device)].cpu(), k=w.k[rows.to(w.q.device)].cpu(), v=w.v[rows.to(w.q.device)].cpu(),
        seq_offset=torch.tensor(new_offs, dtype=w.seq_offset.dtype), max_seq_len=w.max_seq_len, silu_scale=w.silu_scale,
        alpha=w.alpha, attn_bias=pick(w.attn_bias), mask=pick(w.mask), mask_type=w.mask_type,
        num_context=pick(w.num_context), num_target=pick(w.num_target), target_group_size=w.target_group_size,
        lengths=lens,
    )  # fmt: skip
    return sub, rows


@pytest.fixture(scope="module", params=["C2", "C3", "C4"])
def config(request):
    heavy = request.param != "C2"
    w = workloads.config(request.param, device=DEV) if heavy else workloads.config(request.param).to(DEV)
    out = launch(w)
    yield request.param, w, out
    del w, out
    torch.cuda.empty_cache()


def test_subbatch_matches_oracle(config, monkeypatch):
    name, w, out = config
    # the cut-out sequences make a list shorter than the machine; with splitting on, the fp32 sums of their long
    # items would be taken in another order than in the full batch
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")
    order = sorted(range(len(w.lengths)), key=lambda b: w.lengths[b])
    seqs = sorted(order[:2] + order[-1:]) if name == "C2" else sorted(order[:2])
    sub, rows = sub_batch(w, seqs)
    full_rows = out[rows.to(DEV)].float().cpu()
    # independence: running the cut-out sequences alone gives bit-identical rows
    alone = launch(sub.to(DEV)).float().cpu()
    assert torch.equal(alone, full_rows)
    ref = O.hstu_jagged_forward(sub.q, sub.k, sub.v, out_dtype=torch.float32, **sub.oracle_kwargs())
    torch.testing.assert_close(full_rows, ref, atol=1e-2, rtol=1e-2)
    lo = O.hstu_jagged_forward(sub.q, sub.k, sub.v, out_dtype=torch.bfloat16, emulate_lowp=torch.bfloat16,
                               **sub.oracle_kwargs()).float()  # fmt: skip
    assert O.mismatch_fraction(full_rows, lo, 5e-3) < 5e-3
    assert O.double_benchmark_ok(full_rows, lo, ref)[0]


def test_reproducible_and_every_row_written(config):
    _, w, out = config
    again = launch(w)
    assert torch.equal(out, again)
    assert torch.isfinite(out.float()).all()
    # rows of non-empty sequences are not all zero (each row sees at least its own key)
    assert (out.float().abs().amax(dim=(1, 2)) > 0).all()


def test_linear_in_v(config):
    _, w, out = config
    w2 = workloads.Workload(**{**w.__dict__})
    w2.v = w.v * 2  # exact in bf16
    out2 = launch(w2)
    torch.testing.assert_close(out2.float(), out.float() * 2, atol=1e-6, rtol=1e-2)


def test_zero_bias_equals_no_bias(config, monkeypatch):
    name, w, out = config
    # (bit for bit on one kernel: with a bias the call runs on the persistent kernel, without one a list of C2's shape
    # would take the kernel for short lists, whose fp32 sums are taken in pieces of another size)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    bare = workloads.Workload(**{**w.__dict__})
    bare.attn_bias = None
    expected = launch(bare)
    zeroed = workloads.Workload(**{**w.__dict__})
    zeroed.attn_bias = torch.zeros(len(w.lengths), w.q.shape[1], w.max_seq_len, w.max_seq_len, dtype=w.q.dtype, device=DEV)
    got = launch(zeroed)
    del zeroed
    torch.cuda.empty_cache()
    assert torch.equal(got, expected)
    if w.attn_bias is not None:
        # and the configuration's own bias does change the rows (the comparison above is not between two calls that ignore it)
        assert not torch.equal(out, expected)


def test_sequence_permutation(config):
    name, w, out = config
    offs = w.seq_offset.cpu().tolist()
    order = list(reversed(range(len(w.lengths))))
    rows = torch.cat([torch.arange(offs[b], offs[b + 1]) for b in order]).to(DEV)
    idx = torch.tensor(order, device=DEV)
    new_offs = [0]
    for b in order:
        new_offs.append(new_offs[-1] + w.lengths[b])
    w2 = workloads.Workload(**{**w.__dict__})
    w2.q, w2.k, w2.v = w.q[rows], w.k[rows], w.v[rows]
    w2.seq_offset = torch.tensor(new_offs, dtype=w.seq_offset.dtype, device=DEV)
    w2.attn_bias = None if w.attn_bias is None else w.attn_bias[idx]
    w2.num_context = None if w.num_context is None else w.num_context[idx]
    w2.num_target = None if w.num_target is None else w.num_target[idx]
    got = launch(w2)
    del w2  # (C4: the permuted copy of the bias is 4 GiB)
    torch.cuda.empty_cache()
    assert torch.equal(got, out[rows])


def test_flop_model_matches_expectation():
    # C2: expectation of the length distribution is about 15 GFLOP; the seeded sample must be near it
    w = workloads.config("C2")
    f = O.causal_effective_flops(w.seq_offset, None, 4, 128, 128)
    assert 12e9 < f < 18e9
