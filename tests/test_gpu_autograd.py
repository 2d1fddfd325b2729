"""The autograd wrapper on the GPU: ``loss.backward()`` through ``hstu_jagged`` must give the gradients
of the oracle's formula (torch autograd on the CPU restatement), for the ``equal`` and ``delta``
overloads, with and without attn_bias; and a direct call of ``hstu_jagged_backward`` must agree with the
wrapper (hstu_backward_v1/test/pytest/test_hstu_autograd.py:137-463 checks the same two things)."""

import pytest
import torch

import ops_rec
from helpers import small_case
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _grads_via_op(w, use_bias):
    wd = w.to(DEV)
    q, k, v = (t.clone().requires_grad_(True) for t in (wd.q, wd.k, wd.v))
    bias = wd.attn_bias.clone().requires_grad_(True) if use_bias else None
    args = list(wd.op_args())
    args[0], args[1], args[2], args[4] = q, k, v, bias
    out = ops_rec.ascendc.attention.hstu_jagged(*args)
    g = torch.Generator(device="cpu").manual_seed(3)
    grad_out = torch.randn(out.shape, generator=g).to(out.dtype)
    out.backward(grad_out.to(DEV))
    return grad_out, (q.grad, k.grad, v.grad, bias.grad if use_bias else None), (q, k, v, bias, wd)


def _grads_via_oracle(w, grad_out, use_bias):
    q, k, v = (t.float().clone().requires_grad_(True) for t in (w.q, w.k, w.v))
    kw = w.oracle_kwargs()
    bias = w.attn_bias.float().clone().requires_grad_(True) if use_bias else None
    kw["attn_bias"] = bias
    out = O.hstu_jagged_forward(q, k, v, out_dtype=torch.float32, **kw)
    out.backward(grad_out.float())
    return q.grad, k.grad, v.grad, (bias.grad if use_bias else None)


@pytest.mark.parametrize("use_bias", [False, True])
@pytest.mark.parametrize("variant", [dict(), dict(ctx=3, max_target=6, group=2), dict(delta=True), dict(heads=4, heads_k=2)],
                         ids=["plain", "ctx_tgt", "delta", "gqa"])  # fmt: skip
def test_backward_matches_oracle_autograd(variant, use_bias):
    w = small_case(seed=41, batch=3, dim=32, lo=10, hi=60, dtype=torch.float32, std=0.7, rab=True, alpha=0.5, **variant)
    if not use_bias:
        w.attn_bias = None
    grad_out, got, _ = _grads_via_op(w, use_bias)
    ref = _grads_via_oracle(w, grad_out, use_bias)
    for name, a, b in zip(("dq", "dk", "dv", "dbias"), got, ref):
        if b is None:
            assert a is None
            continue
        torch.testing.assert_close(a.float().cpu(), b, atol=2e-4, rtol=2e-3, msg=lambda m, n=name: f"{n}: {m}")


def test_direct_backward_call_agrees_with_wrapper():
    w = small_case(seed=42, batch=2, dim=64, lo=20, hi=90, dtype=torch.bfloat16, std=0.5, rab=True)
    grad_out, got, (q, k, v, bias, wd) = _grads_via_op(w, True)
    dq, dk, dv, db = ops_rec.ascendc.attention.hstu_jagged_backward(
        grad_out.to(DEV), q.detach(), k.detach(), v.detach(), None, bias.detach(), 0, wd.max_seq_len, wd.max_seq_len,
        wd.silu_scale, wd.seq_offset, wd.seq_offset, None, None, 0, wd.alpha,
    )  # fmt: skip
    for a, b in zip(got, (dq, dk, dv, db)):
        assert torch.equal(a, b)


def test_no_grad_path_and_mask_requires_grad_is_rejected():
    w = small_case(seed=43, batch=2, dim=32, lo=5, hi=30, dtype=torch.float16, custom_mask=True).to(DEV)
    out = ops_rec.ascendc.attention.hstu_jagged(*w.op_args())
    assert not out.requires_grad
    args = list(w.op_args())
    args[0] = w.q.clone().requires_grad_(True)
    args[3] = w.mask.clone().requires_grad_(True)
    with pytest.raises(NotImplementedError, match="non-differentiable"):
        ops_rec.ascendc.attention.hstu_jagged(*args)
