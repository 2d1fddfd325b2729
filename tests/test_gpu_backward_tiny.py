"""The backward for batches of tiny sequences (hstu_bwd_tiny_kernel.hip.h: one launch, one two-wavefront workgroup per
(sequence, K/V head), taken when no sequence has more than 32 rows or keys): against torch autograd on the CPU oracle
and the library's generic kernels (the bars of test_gpu_backward.py), and against the tuned kernels on the same inputs
(HSTU_MI355_SHORT=0).  Which calls take the kernel is the host's rule: test_host_boundary.py (no workspace asked for).
"""

import dataclasses

import pytest
import torch

import helpers
from ops_rec import workloads
from test_gpu_backward import DEV, check, device_grads, make

pytestmark = pytest.mark.gpu

CASES = {
    "dim256": dict(batch=40, heads=2, dim=256, lo=1, hi=32),
    "dim128": dict(batch=40, heads=2, dim=128, lo=1, hi=32),
    "dim64": dict(batch=24, heads=3, dim=64, lo=1, hi=32),
    "all_32_rows": dict(batch=16, heads=3, dim=256, lo=32, hi=32),
    "context_targets_groups": dict(batch=12, heads=2, dim=256, lo=12, hi=32, num_context=3, max_target=9, target_group_size=2),
    "targets_128": dict(batch=12, heads=2, dim=128, lo=8, hi=31, max_target=8, target_group_size=1),
    "grouped_heads": dict(batch=10, heads=4, heads_k=2, dim=256, lo=1, hi=24),
    "one_kv_head": dict(batch=10, heads=6, heads_k=1, dim=128, lo=0, hi=32, max_seq_len=32),
    "padded_head_dims": dict(batch=9, heads=2, dim=208, dim_v=144, lo=1, hi=30),
    "padded_head_dims_128": dict(batch=9, heads=2, dim=80, dim_v=112, lo=1, hi=30),
    "small_head_dims": dict(batch=9, heads=2, dim=8, dim_v=16, lo=1, hi=30),
    "int64_offsets": dict(batch=7, heads=1, dim=256, lo=5, hi=20, index_dtype=torch.int64),
}  # fmt: skip


def tuned_and_tiny(w, monkeypatch, seed=5):
    g = torch.Generator(device=DEV).manual_seed(seed)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    tiny = device_grads(w, grad_out)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    tuned = device_grads(w, grad_out)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    return tiny, tuned


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", list(CASES))
def test_tiny_sequences_backward(name, dtype, monkeypatch):
    for seed in range(2):
        w = make(seed=seed + 40, dtype=dtype, **CASES[name])
        if seed == 1 and "max_target" not in CASES[name]:
            w = dataclasses.replace(w, mask_type=2)  # every key visible
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
        check(w, monkeypatch)
        tiny, tuned = tuned_and_tiny(w, monkeypatch)
        tol = 1e-2 if dtype == torch.bfloat16 else 2e-3
        for a, b in zip(tiny[:3], tuned[:3]):
            scale = b.float().abs().max().item()
            torch.testing.assert_close(a.float(), b.float(), atol=tol * scale, rtol=tol)


def test_tiny_sequences_backward_with_more_keys_than_queries(monkeypatch):
    lq, lk = [7, 20, 1, 0, 12, 0], [32, 21, 19, 4, 12, 0]
    g = torch.Generator(device=DEV).manual_seed(8)
    mk = lambda n, h, d: (torch.randn(n, h, d, generator=g, device=DEV) * 0.5).to(torch.bfloat16)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int64, device=DEV)  # noqa: E731
    for dim in (128, 256):
        w = workloads.Workload(name="delta", q=mk(sum(lq), 4, dim), k=mk(sum(lk), 2, dim), v=mk(sum(lk), 2, dim),
                               seq_offset=offs(lq), max_seq_len=20, silu_scale=1.0, alpha=0.09, seq_offset_k=offs(lk),
                               max_seq_len_k=32, lengths=lq)  # fmt: skip
        check(w, monkeypatch)
        tiny, tuned = tuned_and_tiny(w, monkeypatch)
        for a, b in zip(tiny[:3], tuned[:3]):
            torch.testing.assert_close(a.float(), b.float(), atol=1e-2 * b.float().abs().max().item(), rtol=1e-2)


def test_tiny_sequences_backward_gaps_and_rows_past_the_last_offset(monkeypatch):
    lengths = [7, 0, 0, 32, 0, 31, 1]
    w = make(batch=len(lengths), heads=2, dim=256, lo=0, hi=0, lengths=lengths, max_seq_len=32)
    extra = 9
    pad = lambda t: torch.cat([t, torch.full((extra, *t.shape[1:]), 3.0, dtype=t.dtype, device=t.device)])  # noqa: E731
    wd = dataclasses.replace(w, q=pad(w.q), k=pad(w.k), v=pad(w.v), seq_offset=torch.cat([w.seq_offset, w.seq_offset[-1:]]))
    g = torch.Generator(device=DEV).manual_seed(3)
    grad_out = torch.randn(w.q.shape[0], 2, 256, generator=g, device=DEV).to(w.q.dtype)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    want = device_grads(w, grad_out)
    got = device_grads(wd, pad(grad_out))
    n = w.q.shape[0]
    for a, b in zip(got[:3], want[:3]):
        assert torch.equal(a[:n], b) and (a[n:] == 0).all()
