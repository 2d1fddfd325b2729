"""The HIP backward kernels (``hstu_jagged_bwd`` of the C ABI, reached through ``hstu_jagged_backward`` and through
``loss.backward()``) against torch autograd on the CPU oracle, on the same seeded inputs.

Tolerance: the kernels round P and dS to the input type before the products that consume them (as the reference's
backward does, hstu_backward_v1/op_kernel/vector_score.h:159-205), so a gradient element carries the rounding of a
sum of up to S products: each gradient tensor must agree with the fp32 oracle within atol = 1e-2 x max|reference|
and rtol = 1e-2 (bf16) / atol = 2e-3 x max|reference|, rtol = 2e-3 (fp16) -- the forward's 1e-2 bar relative to the
tensor's scale -- and must not be further from it than 2 x the rounding to the output type of the library's generic
backward kernels (fp32 arithmetic, P and dS unrounded) plus that bound.  The same cases run through those kernels
(HSTU_MI355_GENERIC_BACKWARD=1) pin that the two device paths agree.
"""

import dataclasses

import pytest
import torch

import ops_rec
from ops_rec import workloads
from oracle import hstu_oracle as O
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def oracle_grads(w, grad_out):
    c = w.to("cpu")
    q, k, v = (t.float().clone().requires_grad_(True) for t in (c.q, c.k, c.v))
    kw = c.oracle_kwargs()
    bias = None
    if c.attn_bias is not None:
        bias = c.attn_bias.float().clone().requires_grad_(True)
        kw["attn_bias"] = bias
    out = O.hstu_jagged_forward(q, k, v, out_dtype=torch.float32, **kw)
    out.backward(grad_out.float().cpu())
    return q.grad, k.grad, v.grad, (bias.grad if bias is not None else None)


def device_grads(w, grad_out):
    k_offs = w.seq_offset if w.seq_offset_k is None else w.seq_offset_k
    max_k = w.max_seq_len if w.max_seq_len_k is None else w.max_seq_len_k
    ctx, tgt = w.num_context, w.num_target
    if (ctx is None) != (tgt is None):  # the backward op wants both or neither (hstu_jagged_plugin.cpp:81-84)
        zeros = torch.zeros_like(ctx if tgt is None else tgt)
        ctx, tgt = (zeros if ctx is None else ctx), (zeros if tgt is None else tgt)
    got = ops_rec.ascendc.attention.hstu_jagged_backward(
        grad_out, w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, max_k, w.silu_scale, w.seq_offset,
        k_offs, ctx, tgt, w.target_group_size, w.alpha)  # fmt: skip
    torch.cuda.synchronize()
    return got


def check(w, monkeypatch, seed=5):
    g = torch.Generator(device=DEV).manual_seed(seed)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    # the workspace in which the query-tile kernel leaves dS for the dK workgroups is not cleared: filled with NaN
    # here, so that a read of an element that was never written would show in dk
    helpers.poison_workspace(monkeypatch)
    got = device_grads(w, grad_out)
    assert torch.equal(device_grads(w, grad_out)[0], got[0])  # reproducible
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "1")
    comp = device_grads(w, grad_out)
    ref = oracle_grads(w, grad_out)
    tol = 1e-2 if w.q.dtype == torch.bfloat16 else 2e-3
    for name, a, c, r in zip(("dq", "dk", "dv", "dbias"), got, comp, ref):
        if r is None:
            assert a is None
            continue
        assert a.dtype == w.q.dtype and a.shape == r.shape, name
        a, c = a.float().cpu(), c.float().cpu()
        assert torch.isfinite(a).all(), name
        scale = r.abs().max().item()
        torch.testing.assert_close(a, r, atol=tol * scale, rtol=tol, msg=lambda m, n=name: f"{n} vs oracle: {m}")
        torch.testing.assert_close(a, c, atol=tol * scale, rtol=tol, msg=lambda m, n=name: f"{n} vs generic kernels: {m}")
        assert (a - r).abs().max() <= 2 * (c - r).abs().max() + tol * scale, name


def make(**kw):
    kw.setdefault("dtype", torch.bfloat16)
    kw.setdefault("std", 0.5)
    kw.setdefault("silu_scale", 1.0)
    return workloads.make("bwd", device=DEV, **kw)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("dim,dim_v", [(64, 64), (128, 128), (96, 64), (32, 16), (8, 128), (256, 256), (136, 192)])
def test_plain_causal(dim, dim_v, dtype, monkeypatch):
    check(make(batch=3, heads=2, dim=dim, dim_v=dim_v, lo=1, hi=300, seed=dim + dim_v, dtype=dtype), monkeypatch)


@pytest.mark.parametrize("ctx,tgt,group", [(0, 30, 1), (0, 30, 3), (6, 0, 0), (6, 30, 3), (200, 40, 7)])
@pytest.mark.parametrize("rab", [False, True], ids=["norab", "rab"])
def test_context_targets_rab(ctx, tgt, group, rab, monkeypatch):
    w = make(batch=3, heads=2, dim=64, lo=260, hi=420, max_seq_len=420, seed=ctx + tgt, num_context=ctx, max_target=tgt,
             target_group_size=group, rab_std=0.5 if rab else None)  # fmt: skip
    check(w, monkeypatch)


@pytest.mark.parametrize("max_len", [300, 301, 303, 304])  # rows of rab / mask / d rab 8-byte, 2-byte, 16-byte aligned
def test_custom_mask_and_rab_alignment(max_len, monkeypatch):
    w = make(batch=2, heads=2, dim=64, lo=150, hi=max_len, max_seq_len=max_len, seed=max_len, rab_std=0.5, dtype=torch.float16)
    g = torch.Generator(device=DEV).manual_seed(1)
    mask = (torch.rand(2, 2, max_len, max_len, generator=g, device=DEV) < 0.6).to(torch.float16)
    check(dataclasses.replace(w, mask=mask, mask_type=3), monkeypatch)


@pytest.mark.parametrize("kw", [
    dict(dim=64, lo=260, hi=424, max_seq_len=424), dict(dim=128, lo=1, hi=520, max_seq_len=520, heads=4, heads_k=2),
    dict(dim=256, lo=100, hi=264, max_seq_len=264), dict(dim=64, lo=200, hi=400, max_seq_len=400, num_context=6, max_target=30, target_group_size=3),
    dict(dim=128, dim_v=64, lo=0, hi=296, max_seq_len=296, dtype=torch.float16), dict(dim=32, lo=300, hi=1200, max_seq_len=1200),
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items() if k != "dtype"))  # fmt: skip
@pytest.mark.parametrize("custom_mask", [False, True], ids=["causal", "custom"])
def test_attn_bias_gradient_handed_to_the_dk_workgroups(kw, custom_mask, monkeypatch):
    """With the attn_bias gradient asked for and 16-byte aligned bias rows the library can hand dS (and P) from the
    query-tile kernel to the workgroups that produce dK (and dV); HSTU_MI355_BWD_HANDOFF=0 keeps the order in which
    they recompute them.  dq and the bias gradient come out bit-identical in every order, dv as well while P is
    recomputed; what is computed from a stored dS or P agrees to rounding."""
    kw = dict(kw)
    w = make(batch=3, heads=kw.pop("heads", 2), seed=len(kw) + 50, rab_std=0.5, **kw)
    assert w.max_seq_len % 8 == 0
    if custom_mask:
        g = torch.Generator(device=DEV).manual_seed(2)
        shape = (3, w.q.shape[1], w.max_seq_len, w.max_seq_len)
        mask = (torch.rand(shape, generator=g, device=DEV) < 0.7).to(w.q.dtype)
        w = dataclasses.replace(w, mask=mask, mask_type=3, num_context=None, num_target=None, target_group_size=0)
    tol = 1e-2 if w.q.dtype == torch.bfloat16 else 2e-3
    g = torch.Generator(device=DEV).manual_seed(6)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    # 1: dV workgroups / query-tile kernel storing dS into the gradient / dK workgroups reading it;  2: query-tile
    # kernel storing dS and P into a workspace and clearing the gradient / dV and dK workgroups reading them, the dK
    # ones writing the gradient
    for order in ("1", "2"):
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        helpers.poison_workspace(monkeypatch)
        check(w, monkeypatch)
        helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
        two = device_grads(w, grad_out)
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        other = device_grads(w, grad_out)
        assert torch.equal(two[0], other[0]) and torch.equal(two[3], other[3])  # dq and the bias gradient: the same bits
        if order == "1":
            assert torch.equal(two[2], other[2])
        for i in (1, 2):
            scale = two[i].float().abs().max().item()
            torch.testing.assert_close(other[i].float(), two[i].float(), atol=tol * scale, rtol=tol)


@pytest.mark.parametrize("kw", [
    dict(dim=128, lo=1, hi=520, max_seq_len=520, heads=4, heads_k=2), dict(dim=256, lo=100, hi=264, max_seq_len=264),
    dict(dim=128, lo=200, hi=400, max_seq_len=400, num_context=6, max_target=30, target_group_size=3),
    dict(dim=128, lo=0, hi=296, max_seq_len=296, num_context=40, max_target=9, target_group_size=1, dtype=torch.float16),
    dict(dim=72, dim_v=128, lo=300, hi=1200, max_seq_len=1200), dict(dim=128, lo=33, hi=33, max_seq_len=40),
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items() if k != "dtype"))  # fmt: skip
@pytest.mark.parametrize("mask", ["causal", "custom", "none"])
def test_ds_handed_to_the_dk_workgroups_through_a_workspace(kw, mask, monkeypatch):
    """Without an attn_bias gradient and with max_seq_len_k a multiple of 8, the query-tile kernel can leave dS -- or
    dS and P -- in a workspace for dK (and dV) workgroups that read them back (hstu_jagged_bwd_workspace_size asks for
    it where that pays; HSTU_MI355_BWD_HANDOFF=1 / 2 force the two orders).  Checked against the oracle and the
    generic kernels with the workspace full of NaN, and against the two-launch order."""
    kw = dict(kw)
    w = make(batch=3, heads=kw.pop("heads", 2), seed=len(kw) + 60, **kw)
    if mask == "custom":
        g = torch.Generator(device=DEV).manual_seed(2)
        shape = (3, w.q.shape[1], w.max_seq_len, w.max_seq_len)
        m = (torch.rand(shape, generator=g, device=DEV) < 0.7).to(w.q.dtype)
        w = dataclasses.replace(w, mask=m, mask_type=3, num_context=None, num_target=None, target_group_size=0)
    elif mask == "none":
        w = dataclasses.replace(w, mask_type=2, num_context=None, num_target=None, target_group_size=0)
    tol = 1e-2 if w.q.dtype == torch.bfloat16 else 2e-3
    g = torch.Generator(device=DEV).manual_seed(6)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    for order in ("1", "2"):  # three launches (dS handed over) and the planes order (dS and P handed over)
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        helpers.poison_workspace(monkeypatch)
        check(w, monkeypatch)  # against the oracle and the generic kernels
        helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
        two = device_grads(w, grad_out)
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        other = device_grads(w, grad_out)
        assert torch.equal(two[0], other[0])  # dq: the same kernel arithmetic in every order
        if order == "1":
            assert torch.equal(two[2], other[2])  # dv as well
        for i in (1, 2):  # dk from the stored dS, dv from the stored P: rounded at the same points
            scale = two[i].float().abs().max().item()
            torch.testing.assert_close(other[i].float(), two[i].float(), atol=tol * scale, rtol=tol)
        # a caller that does not bring the workspace the library asked for gets the two-launch order
        helpers.withhold_workspace(monkeypatch)
        without = device_grads(w, grad_out)
        assert all(torch.equal(x, y) for x, y in zip(two[:3], without[:3]))


@pytest.mark.parametrize("kw", [
    dict(dim=128, lo=200, hi=1004, max_seq_len=1004, heads=4), dict(dim=64, lo=1, hi=331, max_seq_len=331),
    dict(dim=256, lo=100, hi=261, max_seq_len=261), dict(dim=512, lo=60, hi=301, max_seq_len=301),
    dict(dim=384, dim_v=320, lo=1, hi=203, max_seq_len=203, heads=4, heads_k=2),
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))  # fmt: skip
@pytest.mark.parametrize("mask_type", [0, 2], ids=["causal", "none"])
def test_planes_with_a_max_seq_len_that_is_not_a_multiple_of_8(kw, mask_type, monkeypatch):
    """The pair plane has a layout of its own, so a call without attn_bias, custom mask or attn_bias gradient takes the
    planes order (and, above head dim 256, the two windows) whatever max_seq_len_k is: the library asks for the
    workspace, and the gradients come out right with it full of NaN.  (Rows of [max_q][max_k] tensors start at multiples
    of 16 bytes only when max_seq_len_k is a multiple of 8: with such a tensor in the call the same shapes run in two
    launches, or on the generic kernels.)"""
    from ops_rec import _ops

    kw = dict(kw)
    w = dataclasses.replace(make(batch=3, heads=kw.pop("heads", 2), seed=77, **kw), mask_type=mask_type)
    asked = []
    plain = _ops._new_workspace
    monkeypatch.setattr(_ops, "_new_workspace", lambda n, dev: (asked.append(n), plain(n, dev))[1])
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "2")
    g = torch.Generator(device=DEV).manual_seed(6)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    device_grads(w, grad_out)
    assert asked and asked[-1] > 0  # the planes (and, for the windows, the partial scores)
    check(w, monkeypatch)  # with the workspace full of NaN, against the oracle and the generic kernels


@pytest.mark.parametrize("dim,max_len", [(64, 300), (128, 420), (256, 268), (384, 132)])
@pytest.mark.parametrize("custom_mask", [False, True], ids=["builtin", "custom"])
@pytest.mark.parametrize("want_drab", [False, True], ids=["nodrab", "drab"])
def test_rows_of_8_byte_pieces_in_every_order(dim, max_len, custom_mask, want_drab, monkeypatch):
    """max_seq_len_k a multiple of 4 but not of 8: rows of attn_bias, custom mask, the attn_bias gradient and the dense dS
    plane start at multiples of 8 bytes only.  The key-tile kernels then take a piece of 8 keys as two 8-byte accesses, the
    second only when it starts inside the row (the sequence's keys): sequences that end at, one short of and three short
    of max_seq_len_k put the next row right behind such a piece.  Every launch order, the workspace full of NaN, against
    the oracle and the generic kernels."""
    lengths = [max_len, max_len - 1, max_len - 3, max_len // 2, 37]
    w = make(batch=len(lengths), heads=2, dim=dim, lo=0, hi=0, lengths=lengths, max_seq_len=max_len, seed=dim + max_len,
             rab_std=0.5)  # fmt: skip
    if custom_mask:
        g = torch.Generator(device=DEV).manual_seed(1)
        m = (torch.rand(len(lengths), 2, max_len, max_len, generator=g, device=DEV) < 0.6).to(w.q.dtype)
        w = dataclasses.replace(w, mask=m, mask_type=3)
    if not want_drab:
        # (the operator returns the gradient of every attn_bias it is given: the case without one keeps the custom mask
        # or, failing that, runs without bias tensors at all -- the planes order with a layout of its own)
        w = dataclasses.replace(w, attn_bias=None)
    for order in ("0", "1", "2"):
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        check(w, monkeypatch)


def test_no_mask(monkeypatch):
    check(dataclasses.replace(make(batch=2, heads=2, dim=128, lo=100, hi=300, seed=9), mask_type=2), monkeypatch)


@pytest.mark.parametrize("heads,heads_k", [(4, 2), (8, 1), (3, 3)])
def test_grouped_heads(heads, heads_k, monkeypatch):
    check(make(batch=3, heads=heads, heads_k=heads_k, dim=64, lo=50, hi=400, seed=heads, rab_std=0.3), monkeypatch)


def test_more_keys_than_queries(monkeypatch):
    lq, lk = [70, 200, 1], [370, 333, 129]
    g = torch.Generator(device=DEV).manual_seed(8)
    mk = lambda n, h, d: (torch.randn(n, h, d, generator=g, device=DEV) * 0.5).to(torch.bfloat16)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int64, device=DEV)  # noqa: E731
    w = workloads.Workload(name="delta", q=mk(sum(lq), 2, 64), k=mk(sum(lk), 2, 64), v=mk(sum(lk), 2, 64),
                           seq_offset=offs(lq), max_seq_len=200, silu_scale=1.0, alpha=0.125, seq_offset_k=offs(lk),
                           max_seq_len_k=370, lengths=lq)  # fmt: skip
    check(w, monkeypatch)


@pytest.mark.parametrize("n_ctx", [3, 40, 130, 700])
@pytest.mark.parametrize("order", ["0", "1", "2"])
def test_context_rows_with_grouped_heads_and_more_keys_than_queries(n_ctx, order, monkeypatch):
    """Context rows see every history key: the first query tile of a sequence runs ahead of the others, and a key tile's
    workgroup sweeps the sub-tiles of the context rows, skips those that see nothing of it and goes on at the first causal
    row -- for every query head of its group.  Context rows within one sub-tile, over several, past the first query tile
    and longer than a sequence; key ranges longer than the query ranges; every launch order."""
    lq, lk = [600, 333, 64, 1, 190], [900, 333, 264, 129, 200]
    g = torch.Generator(device=DEV).manual_seed(n_ctx)
    mk = lambda n, h, d: (torch.randn(n, h, d, generator=g, device=DEV) * 0.5).to(torch.bfloat16)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int32, device=DEV)  # noqa: E731
    w = workloads.Workload(name="ctx", q=mk(sum(lq), 4, 128), k=mk(sum(lk), 2, 128), v=mk(sum(lk), 2, 128),
                           seq_offset=offs(lq), max_seq_len=600, silu_scale=1.0, alpha=0.09, seq_offset_k=offs(lk),
                           max_seq_len_k=904, lengths=lq,
                           num_context=torch.tensor([n_ctx, n_ctx, 5, 0, n_ctx], dtype=torch.int32, device=DEV),
                           num_target=torch.tensor([30, 0, 7, 1, 64], dtype=torch.int32, device=DEV), target_group_size=3)  # fmt: skip
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
    check(w, monkeypatch)


@pytest.mark.parametrize("order", ["0", "1", "2"])
@pytest.mark.parametrize("rab", [False, True], ids=["plain", "bias_gradient"])
def test_grids_pair_after_pair_give_the_same_bits(order, rab, monkeypatch):
    """Long launches over more rows than the caches hold run their grids pair after pair, the pairs dealt to the XCDs,
    instead of level after level (HSTU_MI355_BWD_PAIR_MAJOR forces either): the same workgroups in another order, so every
    gradient must come out bit for bit the same -- here with 30 (query) and 15 (key) pairs, neither a multiple of 8, so that
    the rounded-up grids have slots without a pair, with empty and one-row sequences, context rows, targets, and more keys
    than queries, in every launch order; the level-after-level result is checked against the oracle as usual."""
    lq, lk = [600, 333, 0, 1, 190], [900, 333, 0, 129, 200]
    g = torch.Generator(device=DEV).manual_seed(77)
    mk = lambda n, h, d: (torch.randn(n, h, d, generator=g, device=DEV) * 0.5).to(torch.bfloat16)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int32, device=DEV)  # noqa: E731
    bias = (torch.randn(5, 6, 600, 904, generator=g, device=DEV) * 0.5).to(torch.bfloat16) if rab else None
    w = workloads.Workload(name="pairs", q=mk(sum(lq), 6, 128), k=mk(sum(lk), 3, 128), v=mk(sum(lk), 3, 128),
                           seq_offset=offs(lq), max_seq_len=600, silu_scale=1.0, alpha=0.09, seq_offset_k=offs(lk),
                           max_seq_len_k=904, attn_bias=bias, lengths=lq,
                           num_context=torch.tensor([3, 40, 0, 0, 5], dtype=torch.int32, device=DEV),
                           num_target=torch.tensor([30, 0, 0, 1, 64], dtype=torch.int32, device=DEV), target_group_size=3)  # fmt: skip
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")  # (the 64-row query-tile kernel has a grid of its own)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_PAIR_MAJOR", "0")
    check(w, monkeypatch)
    grad_out = torch.randn(w.q.shape[0], 6, 128, generator=g, device=DEV).to(torch.bfloat16)
    by_level = device_grads(w, grad_out)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_PAIR_MAJOR", "1")
    by_pair = device_grads(w, grad_out)
    for name, a, b in zip(("dq", "dk", "dv", "d_attn_bias"), by_level, by_pair):
        assert (a is None) == (b is None), name
        if a is not None:
            assert torch.equal(a, b), name


@pytest.mark.parametrize("rab", [False, True], ids=["workspace", "bias_gradient"])
def test_ds_hand_over_with_more_keys_than_queries(rab, monkeypatch):
    # the three-launch order on key ranges longer than the query ranges (delta), grouped heads, 16-byte aligned rows
    lq, lk = [70, 200, 1, 0, 129], [376, 333, 129, 40, 129]
    g = torch.Generator(device=DEV).manual_seed(18)
    mk = lambda n, h, d: (torch.randn(n, h, d, generator=g, device=DEV) * 0.5).to(torch.bfloat16)  # noqa: E731
    offs = lambda ls: torch.tensor([0] + list(torch.tensor(ls).cumsum(0)), dtype=torch.int64, device=DEV)  # noqa: E731
    bias = (torch.randn(5, 4, 200, 376, generator=g, device=DEV) * 0.5).to(torch.bfloat16) if rab else None
    w = workloads.Workload(name="delta", q=mk(sum(lq), 4, 128), k=mk(sum(lk), 2, 128), v=mk(sum(lk), 2, 128),
                           seq_offset=offs(lq), max_seq_len=200, silu_scale=1.0, alpha=0.09, seq_offset_k=offs(lk),
                           max_seq_len_k=376, attn_bias=bias, lengths=lq)  # fmt: skip
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "1")
    check(w, monkeypatch)
    g2 = torch.Generator(device=DEV).manual_seed(6)
    grad_out = torch.randn(w.q.shape[0], 4, 128, generator=g2, device=DEV).to(torch.bfloat16)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
    two = device_grads(w, grad_out)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "1")
    three = device_grads(w, grad_out)
    assert torch.equal(two[0], three[0]) and torch.equal(two[2], three[2])
    if rab:
        assert torch.equal(two[3], three[3])


def test_random_shapes_in_both_launch_orders(monkeypatch):
    """60 seeded random cases (head dims, grouped heads, lengths from empty to 1030, context / targets, every mask
    type, with and without attn_bias, both index types): the three-launch and the planes order, their workspace
    full of NaN, against the two-launch order -- dq and the bias gradient bit for bit, dv as well with three launches,
    what is computed from a stored dS or P to rounding."""
    import random

    rnd = random.Random(5)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    helpers.poison_workspace(monkeypatch)
    for case in range(60):
        d = rnd.choice([32, 64, 64, 128, 128, 128, 256, 80, 96, 48, 208])
        heads_k = rnd.choice([1, 2, 3])
        heads = heads_k * rnd.choice([1, 1, 2, 4])
        hi = rnd.choice([8, 31, 32, 33, 64, 100, 127, 128, 129, 200, 256, 300, 511, 520, 777, 1030])
        max_len = (hi + rnd.choice([0, 0, 5, 40]) + 7) // 8 * 8
        kw = dict(batch=rnd.choice([1, 2, 3, 5, 9]), heads=heads, heads_k=heads_k, dim=d,
                  dim_v=rnd.choice([d, d, max(16, (d // 2 + 15) // 16 * 16)]), lo=rnd.choice([0, 1, hi // 2, hi]), hi=hi,
                  max_seq_len=max_len, dtype=rnd.choice([torch.bfloat16, torch.float16]), silu_scale=rnd.choice([0.0, 1.0]),
                  seed=case, rab_std=rnd.choice([None, 0.5]), index_dtype=rnd.choice([torch.int32, torch.int64]))  # fmt: skip
        if rnd.random() < 0.4:
            kw.update(num_context=rnd.choice([0, 3, 40]), max_target=rnd.choice([0, 5, 60]), target_group_size=rnd.choice([0, 1, 3]))
        mask_type = rnd.choice([0, 0, 0, 2, 3])
        w = make(**kw)
        if mask_type == 3:
            g = torch.Generator(device=DEV).manual_seed(case)
            m = (torch.rand(len(w.lengths), heads, max_len, max_len, generator=g, device=DEV) < 0.7).to(w.q.dtype)
            w = dataclasses.replace(w, mask=m, mask_type=3, num_context=None, num_target=None, target_group_size=0)
        elif mask_type == 2:
            w = dataclasses.replace(w, mask_type=2, num_context=None, num_target=None, target_group_size=0)
        g = torch.Generator(device=DEV).manual_seed(1000 + case)
        grad_out = torch.randn(w.q.shape[0], heads, w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
        two = device_grads(w, grad_out)
        label = f"case {case}: {kw}, mask_type {mask_type}"
        tol = 1e-2 if w.q.dtype == torch.bfloat16 else 2e-3
        for order in ("1", "2"):  # (2: dS and P through the workspace; with an attn_bias gradient it is order 1 again)
            helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
            other = device_grads(w, grad_out)
            assert all(torch.isfinite(t).all() for t in other if t is not None), label
            assert torch.equal(two[0], other[0]), label
            assert two[3] is None or torch.equal(two[3], other[3]), label
            if order == "1":
                assert torch.equal(two[2], other[2]), label
            for i in (1, 2):
                scale = max(two[i].float().abs().max().item(), 1e-6)
                assert (two[i].float() - other[i].float()).abs().max().item() <= tol * scale, label


def test_long_sequences_and_rows_past_the_last_offset(monkeypatch):
    w = make(batch=2, heads=2, dim=128, lo=1500, hi=2500, seed=7, std=0.3)
    # 40 rows that belong to no sequence: their gradients must come back as zeros
    pad = lambda t: torch.cat([t, torch.ones(40, *t.shape[1:], dtype=t.dtype, device=DEV)])  # noqa: E731
    w = dataclasses.replace(w, q=pad(w.q), k=pad(w.k), v=pad(w.v))
    check(w, monkeypatch)
    grad_out = torch.ones(w.q.shape[0], 2, 128, dtype=torch.bfloat16, device=DEV)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    dq, dk, dv, _ = device_grads(w, grad_out)
    assert not dq[-40:].any() and not dk[-40:].any() and not dv[-40:].any()


def test_empty_sequences_and_trailing_repeated_offset(monkeypatch):
    w = make(batch=5, heads=2, dim=64, lo=0, hi=0, lengths=[0, 130, 0, 57, 0], seed=3)
    check(w, monkeypatch)


def test_loss_backward_uses_the_kernels(monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    w = make(batch=2, heads=2, dim=64, lo=100, hi=200, seed=11, rab_std=0.3)
    q, k, v, bias = (t.clone().requires_grad_(True) for t in (w.q, w.k, w.v, w.attn_bias))
    args = list(w.op_args())
    args[0], args[1], args[2], args[4] = q, k, v, bias
    out = ops_rec.ascendc.attention.hstu_jagged(*args)
    grad_out = torch.randn(out.shape, device=DEV).to(out.dtype)
    out.backward(grad_out)
    direct = device_grads(w, grad_out)
    for a, b in zip((q.grad, k.grad, v.grad, bias.grad), direct):
        assert torch.equal(a, b)


@pytest.mark.parametrize("use_bias", [False, True], ids=["nobias", "bias"])
@pytest.mark.parametrize("dtype,dim", [(torch.bfloat16, 64), (torch.float16, 128), (torch.float32, 32)])
def test_dense_layout_backward(dtype, dim, use_bias, monkeypatch):
    # hstu_dense / hstu_dense_backward: [B, S, N, D], alpha 1, every sequence of full length
    # (torch_extension/hstu_dense_plugin.cpp:41-151); loss.backward() through the registered autograd as well
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "0")
    batch, seq, heads = 3, 200, 2
    g = torch.Generator().manual_seed(dim)
    mk = lambda *shape, std=0.5: (torch.randn(*shape, generator=g) * std).to(dtype)  # noqa: E731
    q, k, v, grad = (mk(batch, seq, heads, dim) for _ in range(4))
    bias = mk(batch, heads, seq, seq, std=0.3) if use_bias else None
    d = lambda t: None if t is None else t.to(DEV)  # noqa: E731
    dq, dk, dv, db = ops_rec.ascendc.attention.hstu_dense_backward(d(grad), d(q), d(k), d(v), None, d(bias), 0, seq, 0.0)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    assert tuple(db.shape) == ((batch, heads, seq, seq) if use_bias else (batch, heads, 256, 256))
    # oracle: the jagged forward on the flattened tensors with offsets 0, S, 2S, ...
    qf, kf, vf = (t.float().view(batch * seq, heads, dim).clone().requires_grad_(True) for t in (q, k, v))
    bf = bias.float().clone().requires_grad_(True) if use_bias else None
    offs = torch.arange(0, (batch + 1) * seq, seq, dtype=torch.int32)
    out = O.hstu_jagged_forward(qf, kf, vf, attn_bias=bf, mask_type=0, max_seq_len=seq, seq_offset=offs, alpha=1.0,
                                out_dtype=torch.float32)  # fmt: skip
    out.backward(grad.float().view(batch * seq, heads, dim))
    tol = {torch.bfloat16: 1e-2, torch.float16: 2e-3, torch.float32: 1e-4}[dtype]
    for name, a, r in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        r = r.view(batch, seq, heads, dim)
        torch.testing.assert_close(a.float().cpu(), r, atol=tol * r.abs().max().item(), rtol=tol, msg=lambda m, n=name: f"{n}: {m}")
    if use_bias:
        torch.testing.assert_close(db.float().cpu(), bf.grad, atol=tol * bf.grad.abs().max().item(), rtol=tol)
    else:
        assert not db.any()
    # the same through autograd
    qd, kd, vd = (d(t).clone().requires_grad_(True) for t in (q, k, v))
    y = ops_rec.ascendc.attention.hstu_dense(qd, kd, vd, None, d(bias), 0, seq, 0.0)
    y.backward(d(grad))
    assert torch.equal(qd.grad, dq) and torch.equal(kd.grad, dk) and torch.equal(vd.grad, dv)
