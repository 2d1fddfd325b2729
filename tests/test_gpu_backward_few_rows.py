"""The backward for sequences of few query rows (hstu_bwd_few_rows_kernel.hip.h: one launch, a four-wavefront workgroup per
(sequence, head) that keeps Q and dO in LDS, streams K and V once and finishes 32 keys per step; taken when no sequence
has more than 64 query rows, head dims are at most 128 and every query head has its own K/V head): against torch autograd
on the CPU oracle and the library's generic kernels (the bars of test_gpu_backward.py), and against the tuned kernels on
the same inputs (HSTU_MI355_SHORT=0).  Which calls take the kernel is the host's rule: test_host_boundary.py.
"""

import dataclasses

import pytest
import torch

import helpers
from ops_rec import workloads
from test_gpu_backward import DEV, check, device_grads, make

pytestmark = pytest.mark.gpu


def delta_case(lq, lk, heads=2, dim=64, dim_v=None, dtype=torch.bfloat16, seed=8, max_q=None, max_k=None, **kw):
    g = torch.Generator(device=DEV).manual_seed(seed)
    mk = lambda n, d: (torch.randn(n, heads, d, generator=g, device=DEV) * 0.5).to(dtype)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int64, device=DEV)  # noqa: E731
    return workloads.Workload(name="few_rows", q=mk(sum(lq), dim), k=mk(sum(lk), dim), v=mk(sum(lk), dim_v or dim),
                              seq_offset=offs(lq), max_seq_len=max_q or max(lq), silu_scale=1.0, alpha=dim**-0.5,
                              seq_offset_k=offs(lk), max_seq_len_k=max_k or max(lk), lengths=lq, **kw)  # fmt: skip


def against_tuned(w, monkeypatch, seed=5):
    g = torch.Generator(device=DEV).manual_seed(seed)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    got = device_grads(w, grad_out)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    tuned = device_grads(w, grad_out)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    tol = 1e-2 if w.q.dtype == torch.bfloat16 else 2e-3
    for a, b in zip(got[:3], tuned[:3]):
        torch.testing.assert_close(a.float(), b.float(), atol=tol * b.float().abs().max().item(), rtol=tol)


DELTA_CASES = {
    "candidates_on_a_history": dict(lq=[52, 52, 52, 52, 52, 52], lk=[1000, 1000, 1000, 1000, 1000, 1000], heads=4),
    "jagged": dict(lq=[7, 64, 1, 33, 20, 48, 64], lk=[300, 64, 700, 33, 519, 48, 1001]),
    "fewer_keys_than_rows": dict(lq=[40, 64, 10, 33], lk=[12, 40, 10, 1]),
    "sequences_without_rows_or_keys": dict(lq=[0, 30, 5, 0, 64, 9], lk=[40, 0, 77, 0, 200, 9]),
    "dims_32_16": dict(lq=[52, 3, 64, 17], lk=[499, 130, 64, 401], dim=32, dim_v=16),
    "dims_8_64": dict(lq=[52, 3, 64, 17], lk=[499, 130, 64, 401], dim=8, dim_v=64),
    "dims_48_32": dict(lq=[32, 32, 32, 32, 32], lk=[499, 499, 499, 499, 499], dim=48, dim_v=32, heads=4),
    "three_heads": dict(lq=[50, 21, 64], lk=[257, 96, 65], heads=3),
    "dim_128": dict(lq=[52, 7, 64, 33, 1], lk=[1000, 300, 64, 519, 77], dim=128),
    "dims_72_128": dict(lq=[52, 3, 64, 17], lk=[499, 130, 64, 401], dim=72, dim_v=128),
    "dims_128_96": dict(lq=[40, 64, 10, 0, 33], lk=[12, 200, 10, 50, 1], dim=128, dim_v=96, heads=3),
}  # fmt: skip


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(DELTA_CASES))
def test_few_query_rows_on_longer_key_ranges(name, dtype, monkeypatch):
    for mask_type in (0, 2):
        w = delta_case(dtype=dtype, seed=len(name), **DELTA_CASES[name])
        w = dataclasses.replace(w, mask_type=mask_type)
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
        check(w, monkeypatch)
        against_tuned(w, monkeypatch)


SELF_CASES = {
    "up_to_64_rows": dict(batch=30, heads=2, dim=64, lo=1, hi=64, max_seq_len=64),
    "context_targets_groups": dict(batch=12, heads=2, dim=64, lo=20, hi=64, max_seq_len=64, num_context=3, max_target=9,
                                   target_group_size=2),
    "targets": dict(batch=12, heads=3, dim=32, lo=34, hi=60, max_seq_len=60, max_target=30, target_group_size=1),
    "context_rows": dict(batch=9, heads=2, dim=64, dim_v=48, lo=33, hi=64, max_seq_len=64, num_context=40),
    "int64_offsets": dict(batch=7, heads=1, dim=64, lo=5, hi=50, max_seq_len=50, index_dtype=torch.int64),
    "dim_128_up_to_64_rows": dict(batch=30, heads=2, dim=128, lo=1, hi=64, max_seq_len=64),
    "dim_128_context_targets_groups": dict(batch=12, heads=2, dim=128, dim_v=112, lo=20, hi=64, max_seq_len=64, num_context=3,
                                           max_target=9, target_group_size=2),
}  # fmt: skip


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(SELF_CASES))
def test_few_query_rows_over_equal_offsets(name, dtype, monkeypatch):
    w = make(seed=len(name) + 60, dtype=dtype, **SELF_CASES[name])
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    check(w, monkeypatch)
    against_tuned(w, monkeypatch)


def test_few_query_rows_context_rows_and_targets_on_longer_key_ranges(monkeypatch):
    lq, lk = [40, 64, 12, 33], [400, 64, 300, 133]
    ctx = torch.tensor([5, 0, 12, 3], dtype=torch.int64, device=DEV)
    tgt = torch.tensor([7, 20, 1, 33], dtype=torch.int64, device=DEV)
    for group in (0, 1, 3):
        w = delta_case(lq, lk, num_context=ctx, num_target=tgt, target_group_size=group)
        check(w, monkeypatch)
        against_tuned(w, monkeypatch)


def test_few_query_rows_and_rows_past_the_last_offset(monkeypatch):
    w = delta_case([7, 0, 64, 31], [100, 40, 64, 500])
    extra = 9
    pad = lambda t: torch.cat([t, torch.full((extra, *t.shape[1:]), 3.0, dtype=t.dtype, device=t.device)])  # noqa: E731
    wd = dataclasses.replace(w, q=pad(w.q), k=pad(w.k), v=pad(w.v), seq_offset=torch.cat([w.seq_offset, w.seq_offset[-1:]]),
                             seq_offset_k=torch.cat([w.seq_offset_k, w.seq_offset_k[-1:]]))  # fmt: skip
    g = torch.Generator(device=DEV).manual_seed(3)
    grad_out = torch.randn(w.q.shape[0], 2, 64, generator=g, device=DEV).to(w.q.dtype)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    want = device_grads(w, grad_out)
    got = device_grads(wd, pad(grad_out))
    for a, b in zip(got[:3], want[:3]):
        m = b.shape[0]
        assert torch.equal(a[:m], b) and (a[m:] == 0).all()
