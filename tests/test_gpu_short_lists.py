"""The forward kernel for short work lists (16-bit inputs, head-dim slot 128, no custom mask): one
workgroup of eight 16-row wavefronts per (query tile, sequence, head) slot, no work list.

Checked against the CPU oracle on the mask, layout and index variants it accepts (forced with HSTU_MI355_SHORT=1 so
that the small cases reach it whatever the host's rule says), against the persistent kernel on the same inputs, for
independence of the rows of a sequence from the rest of the batch (bit for bit), and for the host's rule itself.
"""

import pytest
import torch

import ops_rec
from ops_rec import _ops, workloads
from oracle import hstu_oracle as O
import helpers
from helpers import small_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(w):
    out = ops_rec.ascendc.attention.hstu_jagged(*w.op_args())
    torch.cuda.synchronize()
    return out


def kernel_name(w):
    k_offs = w.seq_offset_k if w.seq_offset_k is not None else w.seq_offset
    p = _ops.prepare_forward(w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len,
                             w.max_seq_len_k or w.max_seq_len, w.silu_scale, w.seq_offset, k_offs, w.num_context,
                             w.num_target, w.target_group_size, w.alpha)  # fmt: skip
    return p.kernel_name()


CASES = {
    "plain": dict(batch=5, heads=2, dim=128, lo=1, hi=300),
    "context_targets_groups": dict(batch=4, heads=2, dim=128, lo=20, hi=400, ctx=5, max_target=17, group=3),
    "targets_group_of_one": dict(batch=3, heads=1, dim=128, lo=130, hi=260, ctx=0, max_target=40, group=1),
    "grouped_heads_more_keys": dict(batch=4, heads=4, heads_k=2, dim=128, lo=1, hi=200, delta=True),
    "padded_head_dims": dict(batch=3, heads=2, dim=96, dim_v=112, lo=1, hi=260),
    "int64_offsets": dict(batch=3, heads=3, dim=128, lo=100, hi=700, index_dtype=torch.int64),
    "nine_pairs": dict(batch=9, heads=1, dim=128, lo=1, hi=140),  # pairs padded to 16 per level
    "sixty_four_sequences": dict(batch=64, heads=2, dim=128, lo=1, hi=140),
}


@pytest.mark.parametrize("kernel", ["short", "persistent"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(CASES))
def test_against_the_oracle(name, dtype, kernel, monkeypatch):
    # (the same cases on the persistent kernel: small lists at head dim 128 reach it only with the switch off)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1" if kernel == "short" else "0")
    for seed in range(2):
        w = small_case(seed=seed, dtype=dtype, std=0.5, **CASES[name])
        wd = w.to(DEV)
        assert kernel_name(wd).endswith("_d128_short") == (kernel == "short"), kernel_name(wd)
        got = run(wd).float().cpu()
        ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
        torch.testing.assert_close(got, ref, atol=1e-2, rtol=1e-2)
        lo = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=dtype, emulate_lowp=dtype, **w.oracle_kwargs()).float()
        assert O.mismatch_fraction(got, lo, 5e-3) < 5e-3


BIAS_CASES = {
    "plain": dict(batch=5, heads=2, dim=128, lo=1, hi=300, max_seq_len=304),
    "context_targets_groups": dict(batch=4, heads=2, dim=128, lo=20, hi=400, max_seq_len=420, num_context=5, max_target=17,
                                   target_group_size=3),
    "grouped_heads_padded_dims": dict(batch=4, heads=4, heads_k=2, dim=96, dim_v=112, lo=1, hi=200, max_seq_len=200),
    "long_rows": dict(batch=2, heads=1, dim=128, lo=900, hi=1500, max_seq_len=1500),
    "one_sub_tile": dict(batch=6, heads=2, dim=128, lo=1, hi=31, max_seq_len=32),
}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(BIAS_CASES))
def test_attn_bias_against_the_oracle(name, dtype, monkeypatch):
    """With an attn_bias (rows of 8-byte pieces: max_seq_len_k a multiple of 4) the kernel adds it to the fp32 scores
    ahead of the SiLU, like the persistent kernel; no-mask calls and rows whose last sub-tile runs past the row included."""
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1")
    for seed, mask_type in ((0, 0), (1, 0), (2, 2)):
        w = workloads.make("bias", dtype=dtype, std=0.5, rab_std=0.5, seed=seed, **BIAS_CASES[name])
        if mask_type == 2:
            w.mask_type, w.num_context, w.num_target, w.target_group_size = 2, None, None, 0
        wd = w.to(DEV)
        assert kernel_name(wd).endswith("_d128_rab_short"), kernel_name(wd)
        got = run(wd).float().cpu()
        ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
        torch.testing.assert_close(got, ref, atol=1e-2, rtol=1e-2)
        lo = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=dtype, emulate_lowp=dtype, **w.oracle_kwargs()).float()
        assert O.mismatch_fraction(got, lo, 5e-3) < 5e-3
        # the persistent kernel on the same inputs: the same sums in another order
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
        assert not kernel_name(wd).endswith("_short")
        torch.testing.assert_close(run(wd).float().cpu(), got, atol=1e-2, rtol=1e-2)
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1")


TINY_CASES = {
    "dim256": dict(batch=40, heads=2, dim=256, lo=1, hi=32),
    "dim128": dict(batch=40, heads=2, dim=128, lo=1, hi=32),
    "all_32_rows": dict(batch=16, heads=3, dim=256, lo=32, hi=32),
    "context_targets_groups": dict(batch=12, heads=2, dim=256, lo=12, hi=32, ctx=3, max_target=9, group=2),
    "grouped_heads_more_keys": dict(batch=10, heads=4, heads_k=2, dim=256, lo=1, hi=24, delta=True),
    "padded_head_dims": dict(batch=9, heads=2, dim=208, dim_v=144, lo=1, hi=30),
    "padded_head_dims_128": dict(batch=9, heads=2, dim=80, dim_v=112, lo=1, hi=30),
    "int64_offsets": dict(batch=7, heads=1, dim=256, lo=5, hi=20, index_dtype=torch.int64),
    "dim64": dict(batch=40, heads=3, dim=64, lo=1, hi=32),
    "dims_8_16": dict(batch=12, heads=2, dim=8, dim_v=16, lo=1, hi=30),
    "up_to_64_rows_dim64": dict(batch=40, heads=2, dim=64, lo=1, hi=64),
    "up_to_64_rows_dim128": dict(batch=30, heads=2, dim=128, lo=20, hi=64),
    "up_to_64_rows_dim256": dict(batch=20, heads=2, dim=256, lo=33, hi=64),
    "all_64_rows": dict(batch=9, heads=3, dim=128, lo=64, hi=64),
    "64_rows_context_targets_groups": dict(batch=12, heads=2, dim=64, dim_v=48, lo=24, hi=64, ctx=5, max_target=20, group=3),
    "64_rows_grouped_heads_more_keys": dict(batch=10, heads=4, heads_k=2, dim=128, lo=1, hi=55, delta=True),
    "64_rows_padded_head_dims": dict(batch=9, heads=2, dim=208, dim_v=144, lo=1, hi=60),
}


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(TINY_CASES))
def test_tiny_sequences_against_the_oracle(name, dtype, monkeypatch):
    """Batches whose sequences are all at most 32 rows and keys long take the kernel with one two-wavefront workgroup
    per (sequence, head); the same inputs on the persistent kernel (switch off) agree with it."""
    for seed in range(2):
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
        w = small_case(seed=seed, dtype=dtype, std=0.5, **TINY_CASES[name])
        if seed == 1 and "ctx" not in TINY_CASES[name]:
            w.mask_type = 2  # every key visible
        wd = w.to(DEV)
        longest = max(wd.max_seq_len, wd.max_seq_len_k or 0)
        assert kernel_name(wd).endswith("_tiny32" if longest <= 32 else "_tiny64"), kernel_name(wd)
        got = run(wd).float().cpu()
        ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
        torch.testing.assert_close(got, ref, atol=1e-2, rtol=1e-2)
        lo = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=dtype, emulate_lowp=dtype, **w.oracle_kwargs()).float()
        assert O.mismatch_fraction(got, lo, 5e-3) < 5e-3
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
        assert "_tiny" not in kernel_name(wd) and "_short" not in kernel_name(wd)
        torch.testing.assert_close(run(wd).float().cpu(), got, atol=1e-2, rtol=1e-2)


def test_tiny_sequences_gaps_and_rows_past_the_last_offset():
    lengths = [7, 0, 0, 32, 0, 31, 1]
    w = workloads.make("gaps", batch=len(lengths), heads=2, dim=256, lo=0, hi=0, lengths=lengths, dtype=torch.bfloat16,
                       std=0.5, max_seq_len=32)  # fmt: skip
    extra = 9
    pad = lambda t: torch.cat([t, torch.full((extra, *t.shape[1:]), 3.0, dtype=t.dtype)])  # noqa: E731
    wd = workloads.Workload(**{**w.__dict__})
    wd.q, wd.k, wd.v = pad(w.q), pad(w.k), pad(w.v)
    wd.seq_offset = torch.cat([w.seq_offset, w.seq_offset[-1:]])
    wd = wd.to(DEV)
    assert kernel_name(wd).endswith("_d256_tiny32")
    got = run(wd).float().cpu()
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    torch.testing.assert_close(got[: ref.shape[0]], ref, atol=1e-2, rtol=1e-2)
    assert (got[ref.shape[0] :] == 0).all()
    # one more key than the kernel for 32 rows takes: the one for 64; one more than that takes: the other kernels
    w33 = workloads.make("n", batch=4, heads=2, dim=256, lo=1, hi=33, dtype=torch.bfloat16, max_seq_len=33, device=DEV)
    assert kernel_name(w33).endswith("_d256_tiny64")
    w65 = workloads.make("n", batch=4, heads=2, dim=256, lo=1, hi=65, dtype=torch.bfloat16, max_seq_len=65, device=DEV)
    assert "_tiny" not in kernel_name(w65)


def test_attn_bias_rows_that_are_not_8_byte_pieces_stay_on_the_persistent_kernel(monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1")
    w = workloads.make("bias", dtype=torch.bfloat16, std=0.5, rab_std=0.5, batch=3, heads=2, dim=128, lo=1, hi=90, max_seq_len=90)
    wd = w.to(DEV)
    assert "_short" not in kernel_name(wd)
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    torch.testing.assert_close(run(wd).float().cpu(), ref, atol=1e-2, rtol=1e-2)


def test_no_mask_and_empty_sequences_and_rows_past_the_last_offset(monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1")
    w = small_case(seed=5, batch=3, heads=2, dim=128, lo=50, hi=300, dtype=torch.bfloat16, std=0.5)
    w.mask_type = 2  # every key visible
    got = run(w.to(DEV)).float().cpu()
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    torch.testing.assert_close(got, ref, atol=1e-2, rtol=1e-2)
    # empty sequences inside the batch, a repeated last offset, and rows behind the last offset (zero-filled)
    lengths = [70, 0, 0, 129, 0, 31]
    w = workloads.make("gaps", batch=len(lengths), heads=2, dim=128, lo=0, hi=0, lengths=lengths, dtype=torch.bfloat16,
                       std=0.5, max_seq_len=200)  # fmt: skip
    extra = 9
    pad = lambda t: torch.cat([t, torch.full((extra, *t.shape[1:]), 3.0, dtype=t.dtype)])  # noqa: E731
    wd = workloads.Workload(**{**w.__dict__})
    wd.q, wd.k, wd.v = pad(w.q), pad(w.k), pad(w.v)
    wd.seq_offset = torch.cat([w.seq_offset, w.seq_offset[-1:]])
    wd = wd.to(DEV)
    assert kernel_name(wd).endswith("_short")
    got = run(wd).float().cpu()
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    torch.testing.assert_close(got[: w.q.shape[0]], ref, atol=1e-2, rtol=1e-2)
    assert (got[w.q.shape[0] :] == 0).all()


def test_rows_do_not_depend_on_the_rest_of_the_batch_or_on_the_launch(monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1")
    w = workloads.make("j", batch=24, heads=4, dim=128, lo=1, hi=1024, dtype=torch.bfloat16, device=DEV, seed=3,
                       num_context=3, max_target=20, target_group_size=2)  # fmt: skip
    out = run(w)
    assert torch.equal(run(w), out)
    offs = w.seq_offset.cpu().tolist()
    for b in (0, 7, 23):
        r0, r1 = offs[b], offs[b + 1]
        one = workloads.Workload(
            name="one", q=w.q[r0:r1], k=w.k[r0:r1], v=w.v[r0:r1],
            seq_offset=torch.tensor([0, r1 - r0], dtype=w.seq_offset.dtype, device=DEV), max_seq_len=w.max_seq_len,
            silu_scale=w.silu_scale, alpha=w.alpha, num_context=w.num_context[b : b + 1],
            num_target=w.num_target[b : b + 1], target_group_size=w.target_group_size, lengths=[r1 - r0],
        )  # fmt: skip
        assert torch.equal(run(one), out[r0:r1]), b


def test_agrees_with_the_persistent_kernel(monkeypatch):
    w = workloads.config("C2").to(DEV)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1")
    assert kernel_name(w).endswith("_short")
    short = run(w).float()
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    assert not kernel_name(w).endswith("_short")
    persistent = run(w).float()
    # the two kernels contract the head dim in different piece sizes (32 against 16 per matrix instruction): the
    # fp32 sums, and with them a rounded output here and there, differ in the last place
    torch.testing.assert_close(short, persistent, atol=2e-5, rtol=8e-3)
    assert (short != persistent).float().mean().item() < 0.25


def test_the_hosts_rule(monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", None)

    def name(**kw):
        base = dict(batch=32, heads=4, dim=128, lo=8, hi=8, dtype=torch.bfloat16, device=DEV)
        base.update(kw)
        return kernel_name(workloads.make("r", **base))

    assert name(max_seq_len=1024).endswith("_short")  # the headline shape: keys up to 1024
    assert name(max_seq_len=1024, dtype=torch.float16).endswith("_short")
    assert name(max_seq_len=1024, batch=512).endswith("_short")  # long list, short keys
    # long lists over more K / V rows than the caches hold: the queues (pair after pair on one XCD each)
    assert name(max_seq_len=1024, batch=384, lo=700, hi=700).endswith("_queues")
    assert name(max_seq_len=1024, batch=128, lo=700, hi=700).endswith("_short")  # under six items per resident workgroup
    assert name(max_seq_len=256, batch=2048, lo=136, hi=136).endswith("_short")  # sequences of a tile or two share nothing
    assert name(max_seq_len=2048, batch=8).endswith("_short")  # keys up to 2048, one slot per resident workgroup
    assert not name(max_seq_len=2048, batch=32).endswith("_short")  # four per resident workgroup
    assert not name(max_seq_len=2048, batch=2).endswith("_short")  # fewer than workgroups: split items
    assert not name(max_seq_len=4096, batch=4).endswith("_short")
    assert name(max_seq_len=1024, batch=8, rab_std=0.1).endswith("_rab_short")  # with a bias: up to a slot per workgroup
    assert not name(max_seq_len=1024, batch=32, rab_std=0.1).endswith("_short")
    assert not name(max_seq_len=1024, dim=64).endswith("_short")  # other head-dim slots
    assert not name(max_seq_len=1024, dim=256).endswith("_short")
    w = workloads.make("m", batch=4, heads=2, dim=128, lo=8, hi=8, max_seq_len=64, dtype=torch.bfloat16, device=DEV)
    w.mask = torch.ones(4, 2, 64, 64, dtype=torch.bfloat16, device=DEV)
    w.mask_type = 3
    assert not kernel_name(w).endswith("_short")  # custom mask
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    assert not name(max_seq_len=1024).endswith("_short")
