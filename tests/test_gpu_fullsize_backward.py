"""hstu_jagged_backward at the full sizes of C2 and C3 on the GPU.

The oracle (autograd on the fp32 golden path) cannot finish these sizes in seconds, so they are checked through
  * the oracle on a sub-batch: the gradients of a few sequences cut out of the batch, computed from the rows the full
    launch wrote for them, against autograd on the oracle for those sequences alone (sequences are independent);
  * size-independent properties: the gradients are linear in grad_out (doubling it doubles every gradient exactly: a
    power of two commutes with every rounding on the way), bitwise reproducible, finite with the dS workspace
    filled with NaN beforehand, and the launch orders of the library (dK workgroups that recompute dS / that read the
    query-tile kernel's dS back / dV workgroups that read its P back as well) agree: bit for bit in dq and the
    attn_bias gradient, to rounding in what is computed from a stored dS or P.
Tolerances as in tests/test_gpu_backward.py: 1e-2 of the largest reference value (bf16).
"""

import pytest
import torch

import ops_rec
from ops_rec import workloads
from oracle import hstu_oracle as O
from test_gpu_fullsize import sub_batch
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def backward(w, grad_out):
    ctx, tgt = w.num_context, w.num_target
    if (ctx is None) != (tgt is None):  # the backward op wants both or neither (hstu_jagged_plugin.cpp:81-84)
        zeros = torch.zeros_like(ctx if tgt is None else tgt)
        ctx, tgt = (zeros if ctx is None else ctx), (zeros if tgt is None else tgt)
    got = ops_rec.ascendc.attention.hstu_jagged_backward(
        grad_out, w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, w.max_seq_len, w.silu_scale,
        w.seq_offset, w.seq_offset, ctx, tgt, w.target_group_size, w.alpha)  # fmt: skip
    torch.cuda.synchronize()
    return got


@pytest.fixture(scope="module", params=["C2", "C3"])
def config(request):
    w = workloads.config(request.param, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(17)
    grad_out = torch.randn(w.q.shape[0], w.q.shape[1], w.v.shape[2], generator=g, device=DEV).to(w.q.dtype)
    yield request.param, w, grad_out
    del w, grad_out
    torch.cuda.empty_cache()


@pytest.mark.parametrize("order", ["library's choice", "two launches", "three launches", "planes"])
def test_subbatch_matches_autograd_on_the_oracle(config, order, monkeypatch):
    name, w, grad_out = config
    if order != "library's choice":
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", {"two launches": "0", "three launches": "1", "planes": "2"}[order])
    helpers.poison_workspace(monkeypatch)
    dq, dk, dv, dbias = backward(w, grad_out)
    for t in (dq, dk, dv) + ((dbias,) if dbias is not None else ()):
        assert torch.isfinite(t).all()
    by_len = sorted(range(len(w.lengths)), key=lambda b: w.lengths[b])
    seqs = sorted(by_len[:2])  # the two shortest sequences
    sub, rows = sub_batch(w, seqs)
    q, k, v = (t.float().clone().requires_grad_(True) for t in (sub.q, sub.k, sub.v))
    kw = sub.oracle_kwargs()
    bias = None
    if sub.attn_bias is not None:
        bias = sub.attn_bias.float().clone().requires_grad_(True)
        kw["attn_bias"] = bias
    O.hstu_jagged_forward(q, k, v, out_dtype=torch.float32, **kw).backward(grad_out[rows.to(DEV)].float().cpu())
    pairs = [("dq", dq[rows.to(DEV)], q.grad), ("dk", dk[rows.to(DEV)], k.grad), ("dv", dv[rows.to(DEV)], v.grad)]
    if bias is not None:
        pairs.append(("dbias", dbias[torch.tensor(seqs, device=DEV)], bias.grad))
    for label, got, ref in pairs:
        scale = ref.abs().max().item()
        torch.testing.assert_close(got.float().cpu(), ref, atol=1e-2 * scale, rtol=1e-2, msg=lambda m, n=label: f"{n}: {m}")


def test_linear_in_grad_out_and_reproducible(config):
    name, w, grad_out = config
    one = backward(w, grad_out)
    again = backward(w, grad_out)
    two = backward(w, grad_out * 2)
    for a, b, c in zip(one, again, two):
        if a is None:
            continue
        assert torch.equal(a, b)
        assert torch.equal(a * 2, c)


def test_the_launch_orders_agree(config, monkeypatch):
    name, w, grad_out = config
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
    two = backward(w, grad_out)
    helpers.poison_workspace(monkeypatch)
    for order in ("1", "2"):
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        other = backward(w, grad_out)
        assert torch.equal(two[0], other[0])
        if order == "1":
            assert torch.equal(two[2], other[2])
        if two[3] is not None:
            assert torch.equal(two[3], other[3])
        for i in (1, 2):
            scale = two[i].float().abs().max().item()
            torch.testing.assert_close(other[i].float(), two[i].float(), atol=1e-2 * scale, rtol=1e-2)


def test_planes_beyond_4_gib_agree_with_the_two_launch_order(monkeypatch):
    """A call whose pair plane passes 4 GiB (64 sequences x 4 heads of 1024 .. 4096 rows at head dim 256: 5.5 GB, within the
    library's limit of 16 GiB): offsets into the plane are 64-bit sums of 32-bit parts per sequence.  The workspace is
    filled with NaN beforehand; dq must match the two-launch order bit for bit, dk and dv to rounding."""
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_WORKSPACE_MB", None)
    w = workloads.make("big", dtype=torch.bfloat16, device=DEV, seed=21, batch=64, heads=4, dim=256, lo=1024, hi=4096,
                       max_seq_len=4096, std=0.5)  # fmt: skip
    g = torch.Generator(device=DEV).manual_seed(3)
    grad_out = torch.randn(w.q.shape, generator=g, device=DEV).to(torch.bfloat16)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
    two = backward(w, grad_out)
    asked = helpers.poison_workspace(monkeypatch)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "2")
    planes = backward(w, grad_out)
    assert asked and asked[-1] > (4 << 30), asked
    assert torch.equal(two[0], planes[0])
    for i in (1, 2):
        assert torch.isfinite(planes[i].float()).all()
        scale = two[i].float().abs().max().item()
        torch.testing.assert_close(planes[i].float(), two[i].float(), atol=1e-2 * scale, rtol=1e-2)
