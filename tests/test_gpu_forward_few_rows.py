"""The forward kernel for small launches of sequences with few query rows (hstu_fwd_few_rows_kernel.hip.h: one workgroup per
(sequence, head) whose eight wavefronts are dealt over the 16-row groups and over the keys; taken when no sequence has more
than 64 query rows, some sequence has more than 64 keys (else the kernel for tiny sequences runs), head dims are at most 128
and there is at most one item per compute unit): against the CPU oracle, and
against the persistent kernel on the same inputs (HSTU_MI355_SHORT=0).
"""

import pytest
import torch

import helpers
import ops_rec
from ops_rec import _ops, workloads
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def case(lq, lk, heads=2, heads_k=None, dim=64, dim_v=None, dtype=torch.bfloat16, seed=8, index_dtype=torch.int32, **kw):
    g = torch.Generator().manual_seed(seed)
    mk = lambda n, h, d: (torch.randn(n, h, d, generator=g) * 0.5).to(dtype)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=index_dtype)  # noqa: E731
    hk = heads_k or heads
    return workloads.Workload(name="few_rows", q=mk(sum(lq), heads, dim), k=mk(sum(lk), hk, dim), v=mk(sum(lk), hk, dim_v or dim),
                              seq_offset=offs(lq), max_seq_len=max(max(lq), 1), silu_scale=0.0, alpha=dim**-0.5,
                              seq_offset_k=offs(lk), max_seq_len_k=max(max(lk), 1), lengths=lq, **kw)  # fmt: skip


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


def check(w, monkeypatch, dtype, kernel="_few_rows"):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    wd = w.to(DEV)
    assert kernel_name(wd).endswith(kernel), kernel_name(wd)
    got = run(wd).float().cpu()
    assert torch.equal(run(wd).float().cpu(), got)  # the partial outputs are added in a fixed order
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    torch.testing.assert_close(got, ref, atol=1e-2, rtol=1e-2)
    lo = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=dtype, emulate_lowp=dtype, **w.oracle_kwargs()).float()
    assert O.mismatch_fraction(got, lo, 5e-3) < 5e-3
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    assert not kernel_name(wd).endswith(kernel)
    torch.testing.assert_close(run(wd).float().cpu(), got, atol=1e-2, rtol=1e-2)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)


CASES = {
    "candidates_on_a_history": dict(lq=[32] * 6, lk=[499] * 6, heads=4, dim=64, dim_v=32),
    "one_row_group": dict(lq=[7, 16, 1, 12], lk=[300, 1000, 33, 257]),
    "two_row_groups": dict(lq=[17, 32, 20], lk=[300, 64, 700]),
    "three_and_four_row_groups": dict(lq=[33, 48, 49, 64, 40], lk=[519, 48, 1001, 64, 130]),
    "fewer_keys_than_rows": dict(lq=[40, 64, 10, 33, 20], lk=[12, 40, 10, 1, 70]),
    "sequences_without_rows_or_keys": dict(lq=[0, 30, 5, 0, 64, 9], lk=[40, 0, 77, 0, 200, 9]),
    "dims_32_16": dict(lq=[52, 3, 64, 17], lk=[499, 130, 64, 401], dim=32, dim_v=16),
    "dims_8_64": dict(lq=[52, 3, 64, 17], lk=[499, 130, 64, 401], dim=8, dim_v=64),
    "dim_128": dict(lq=[52, 7, 64, 33, 1], lk=[500, 300, 64, 419, 77], dim=128),
    "dims_72_128": dict(lq=[52, 3, 64, 17], lk=[499, 130, 64, 401], dim=72, dim_v=128),
    "dims_128_96": dict(lq=[40, 64, 10, 0, 33], lk=[12, 200, 10, 50, 1], dim=128, dim_v=96, heads=3),
    "grouped_heads": dict(lq=[50, 21, 64, 9], lk=[257, 96, 65, 800], heads=6, heads_k=2),
    "int64_offsets": dict(lq=[20, 64, 3], lk=[90, 64, 640], index_dtype=torch.int64),
    "long_history": dict(lq=[10, 16], lk=[4000, 4096], heads=1),
}  # fmt: skip


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(CASES))
def test_few_query_rows_against_the_oracle(name, dtype, monkeypatch):
    for mask_type in (0, 2):
        w = case(dtype=dtype, seed=len(name), **CASES[name])
        w.mask_type = mask_type
        check(w, monkeypatch, dtype)


def test_few_query_rows_context_rows_and_targets(monkeypatch):
    lq, lk = [40, 64, 12, 33], [400, 64, 300, 133]
    for group in (0, 1, 3):
        for dim in (64, 128):  # (400 keys: 7 sub-tiles per wavefront)
            w = case(lq, lk, dim=dim, num_context=torch.tensor([5, 0, 12, 3], dtype=torch.int32),
                     num_target=torch.tensor([7, 20, 1, 33], dtype=torch.int32), target_group_size=group)  # fmt: skip
            check(w, monkeypatch, torch.bfloat16)


def test_few_query_rows_and_rows_past_the_last_offset(monkeypatch):
    w = case([7, 0, 64, 31], [100, 40, 64, 500])
    check(w, monkeypatch, torch.bfloat16)
    extra = 9
    pad = lambda t: torch.cat([t, torch.full((extra, *t.shape[1:]), 3.0, dtype=t.dtype)])  # noqa: E731
    wd = workloads.Workload(**{**w.__dict__})
    wd.q, wd.k, wd.v = pad(w.q), pad(w.k), pad(w.v)
    wd.seq_offset = torch.cat([w.seq_offset, w.seq_offset[-1:]])
    wd.seq_offset_k = torch.cat([w.seq_offset_k, w.seq_offset_k[-1:]])
    wd = wd.to(DEV)
    assert kernel_name(wd).endswith("_few_rows")
    got = run(wd).float().cpu()
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    torch.testing.assert_close(got[: ref.shape[0]], ref, atol=1e-2, rtol=1e-2)
    assert (got[ref.shape[0] :] == 0).all()


def test_the_hosts_rule_for_few_query_rows(monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ok = case([30] * 8, [200] * 8).to(DEV)
    assert kernel_name(ok).endswith("_d64_few_rows")
    assert kernel_name(case([30] * 8, [200] * 8, dim=96).to(DEV)).endswith("_d128_few_rows")
    assert "_few_rows" not in kernel_name(case([65] + [30] * 7, [200] * 8).to(DEV))  # 65 query rows
    assert "_few_rows" not in kernel_name(case([30] * 8, [200] * 8, dim=136, dim_v=144).to(DEV))  # head dims above 128
    many = case([8] * (cus // 2 + 1), [100] * (cus // 2 + 1), heads=2).to(DEV)  # more items than compute units
    assert "_few_rows" not in kernel_name(many)
    assert "_few_rows" not in kernel_name(case([30] * 8, [2100] * 8).to(DEV))  # 17 sub-tiles per wavefront
    assert kernel_name(case([16] * 8, [4096] * 8).to(DEV)).endswith("_few_rows")  # 16 rows: eight wavefronts over the keys
    bias = case([30] * 8, [200] * 8)
    bias.attn_bias = torch.zeros(8, 2, 30, 200, dtype=torch.bfloat16)
    assert "_few_rows" not in kernel_name(bias.to(DEV))
