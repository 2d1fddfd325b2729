"""The one-launch kernels at the full sizes of two shapes of the reference's own operator benchmark
(ascendc/attention/hstu_v2/test/pytest/test_backward_op_benchmark.py:183-197): batch 2048 x 4 heads x 52 rows x 1000 keys at
head dim 64 (few query rows) and batch 2048 x 2 heads x 32 rows at head dim 256 (tiny sequences); in bf16, whose exponent
range keeps the doubling below exact (the benchmark's fp16 runs into subnormal dS values).

The oracle cannot finish these sizes in seconds, so they are checked through
  * the oracle on a sub-batch: a few sequences cut out of the batch, forward and (by autograd) backward, against the rows
    the full launch wrote for them (sequences are independent);
  * the tuned kernels on the same inputs (HSTU_MI355_SHORT=0), to rounding;
  * size-independent properties: bitwise reproducible, finite, linear in grad_out (doubling it doubles every gradient
    exactly: a power of two commutes with every rounding on the way).
Tolerances as in tests/test_gpu_backward.py: 1e-2 of the largest reference value (bf16).
"""

import pytest
import torch

import helpers
import ops_rec
from oracle import hstu_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
att = ops_rec.ascendc.attention

SHAPES = {
    "few_query_rows": dict(batch=2048, heads=4, dim=64, s_q=52, s_k=1000),
    "tiny_sequences": dict(batch=2048, heads=2, dim=256, s_q=32, s_k=32),
}


@pytest.fixture(scope="module", params=list(SHAPES))
def shape(request):
    p = SHAPES[request.param]
    b, h, d, s_q, s_k = p["batch"], p["heads"], p["dim"], p["s_q"], p["s_k"]
    g = torch.Generator(device=DEV).manual_seed(5)
    rnd = lambda *s: (torch.randn(*s, generator=g, device=DEV) * 0.5).to(torch.bfloat16)  # noqa: E731
    t = dict(q=rnd(b * s_q, h, d), k=rnd(b * s_k, h, d), v=rnd(b * s_k, h, d), grad=rnd(b * s_q, h, d),
             offs_q=torch.arange(0, (b + 1) * s_q, s_q, dtype=torch.int32, device=DEV),
             offs_k=torch.arange(0, (b + 1) * s_k, s_k, dtype=torch.int32, device=DEV), alpha=d**-0.5, **p)  # fmt: skip
    yield t
    del t
    torch.cuda.empty_cache()


def forward(t, q=None, k=None, v=None, offs_q=None, offs_k=None):
    q, k, v = (t["q"] if q is None else q), (t["k"] if k is None else k), (t["v"] if v is None else v)
    oq, ok = (t["offs_q"] if offs_q is None else offs_q), (t["offs_k"] if offs_k is None else offs_k)
    out = att.hstu_jagged(q, k, v, None, None, 0, t["s_q"], t["s_k"], 0.0, oq, ok, None, None, 0, t["alpha"])
    torch.cuda.synchronize()
    return out


def backward(t, grad=None):
    got = att.hstu_jagged_backward(t["grad"] if grad is None else grad, t["q"], t["k"], t["v"], None, None, 0, t["s_q"],
                                   t["s_k"], 0.0, t["offs_q"], t["offs_k"], None, None, 0, t["alpha"])  # fmt: skip
    torch.cuda.synchronize()
    return got[:3]


def test_subbatch_matches_the_oracle(shape, monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    t = shape
    s_q, s_k = t["s_q"], t["s_k"]
    out = forward(t)
    dq, dk, dv = backward(t)
    for x in (out, dq, dk, dv):
        assert torch.isfinite(x).all()
    seqs = [0, 777, t["batch"] - 1]
    rows_q = torch.cat([torch.arange(b * s_q, (b + 1) * s_q) for b in seqs])
    rows_k = torch.cat([torch.arange(b * s_k, (b + 1) * s_k) for b in seqs])
    q = t["q"][rows_q.to(DEV)].float().cpu().requires_grad_(True)
    k = t["k"][rows_k.to(DEV)].float().cpu().requires_grad_(True)
    v = t["v"][rows_k.to(DEV)].float().cpu().requires_grad_(True)
    offs_q = torch.arange(0, (len(seqs) + 1) * s_q, s_q, dtype=torch.int32)
    offs_k = torch.arange(0, (len(seqs) + 1) * s_k, s_k, dtype=torch.int32)
    ref = O.hstu_jagged_forward(q, k, v, out_dtype=torch.float32, seq_offset=offs_q, seq_offset_k=offs_k, max_seq_len=s_q,
                                max_seq_len_k=s_k, silu_scale=0.0, alpha=t["alpha"], mask_type=0)  # fmt: skip
    ref.backward(t["grad"][rows_q.to(DEV)].float().cpu())
    tol = 1e-2
    pairs = ((out[rows_q.to(DEV)], ref.detach()), (dq[rows_q.to(DEV)], q.grad), (dk[rows_k.to(DEV)], k.grad), (dv[rows_k.to(DEV)], v.grad))
    for got, want in pairs:
        scale = want.abs().max().item()
        torch.testing.assert_close(got.float().cpu(), want, atol=tol * scale, rtol=tol)


def test_agrees_with_the_tuned_kernels_and_is_reproducible_and_linear(shape, monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    t = shape
    out, grads = forward(t), backward(t)
    assert torch.equal(forward(t), out)
    for a, b in zip(backward(t), grads):
        assert torch.equal(a, b)
    for a, b in zip(backward(t, t["grad"] * 2), grads):
        assert torch.equal(a, b * 2)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    tol = 1e-2
    for got, want in zip((out,) + tuple(grads), (forward(t),) + tuple(backward(t))):
        scale = want.float().abs().max().item()
        torch.testing.assert_close(got.float(), want.float(), atol=tol * scale, rtol=tol)
