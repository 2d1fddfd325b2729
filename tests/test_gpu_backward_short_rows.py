"""The backward's query-tile kernel with 64-row tiles (hstu_bwd_dq_short_kernel.hip.h; the host takes it for launches
with at most one 128-row slot per compute unit, HSTU_MI355_SHORT=1 forces it) in each of the three launch orders:
against torch autograd on the CPU oracle and the library's generic kernels (the bars of test_gpu_backward.py),
against the kernel with 128-row tiles on the same inputs, and bit for bit against itself across the launch orders.
"""

import dataclasses

import pytest
import torch

import helpers
from test_gpu_backward import DEV, check, device_grads, make

pytestmark = pytest.mark.gpu

CASES = {
    "jagged_gqa": dict(batch=5, heads=4, heads_k=2, dim=128, lo=1, hi=520, max_seq_len=520),
    "targets": dict(batch=3, heads=2, dim=128, lo=200, hi=400, max_seq_len=400, num_context=6, max_target=30, target_group_size=3),
    "context_fp16": dict(batch=3, heads=2, dim=128, lo=0, hi=296, max_seq_len=296, num_context=40, max_target=9,
                         target_group_size=1, dtype=torch.float16),
    "dims_72_128": dict(batch=2, heads=2, dim=72, dim_v=128, lo=300, hi=1200, max_seq_len=1200),
    "dims_128_96": dict(batch=2, heads=3, dim=128, dim_v=96, lo=10, hi=200, max_seq_len=256),
    "one_block": dict(batch=4, heads=2, dim=128, lo=33, hi=33, max_seq_len=72),  # (up to 64 rows: another kernel)
    "long_rows": dict(batch=2, heads=2, dim=128, lo=1500, hi=2300, max_seq_len=2304),
    "tile_edges": dict(batch=6, heads=1, dim=128, lo=63, hi=66, max_seq_len=128),
}  # fmt: skip


@pytest.mark.parametrize("mask", ["causal", "none"])
@pytest.mark.parametrize("name", list(CASES))
def test_short_row_kernel_in_every_order(name, mask, monkeypatch):
    w = make(seed=31, **CASES[name])
    if mask == "none":
        w = dataclasses.replace(w, mask_type=2, num_context=None, num_target=None, target_group_size=0)
    g = torch.Generator(device=DEV).manual_seed(8)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    tol = 1e-2 if w.q.dtype == torch.bfloat16 else 2e-3
    grads = {}
    for short in ("1", "0"):
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", short)
        for order in ("0", "1", "2"):
            helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
            if short == "1":
                check(w, monkeypatch)  # oracle, generic kernels, NaN-filled workspace
                helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
            grads[short, order] = device_grads(w, grad_out)
    for order in ("1", "2"):
        assert torch.equal(grads["1", "0"][0], grads["1", order][0])  # dq: one arithmetic in every order
    for order in ("0", "1", "2"):
        for a, b in zip(grads["1", order][:3], grads["0", order][:3]):
            scale = b.float().abs().max().item()
            torch.testing.assert_close(a.float(), b.float(), atol=tol * scale, rtol=tol)
    # in the two-launch order dk and dv are the key-tile kernel's own work: the query-tile kernel does not touch them
    assert torch.equal(grads["1", "0"][1], grads["0", "0"][1]) and torch.equal(grads["1", "0"][2], grads["0", "0"][2])


def test_rule_follows_the_slot_count(monkeypatch):
    """Without the switch, small launches take the 64-row kernel and large ones the 128-row kernel: the results are
    those of the forced kernel, bit for bit."""
    g = torch.Generator(device=DEV).manual_seed(9)
    for kw, expect in ((dict(batch=4, heads=4, dim=128, lo=900, hi=1024, max_seq_len=1024), "1"),
                       (dict(batch=40, heads=4, dim=128, lo=300, hi=1024, max_seq_len=1024), "0")):  # fmt: skip
        w = make(seed=33, **kw)
        grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
        by_rule = device_grads(w, grad_out)[0]
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", expect)
        assert torch.equal(by_rule, device_grads(w, grad_out)[0])
        helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "1" if expect == "0" else "0")
        assert not torch.equal(by_rule, device_grads(w, grad_out)[0])  # (the other kernel sums in another order)
