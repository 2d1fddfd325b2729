"""The operators under torch.compile (the reference's "graph" tests: torch.compile(op, dynamic=True, fullgraph=True),
e.g. ascendc/activation/ln_mul/test/pytest/test_ln_mul.py:69-85, hstu_forward_v1/test/pytest/test_hstu_jagged.py:1202-1338):
tracing needs the schemas, the Meta implementations and the autograd formulas to agree with what the kernels return.
Two backends: the default one, as the reference's tests use it (inductor: it generates the code around the
operators, which stay opaque calls), and "aot_eager", which runs dynamo, fake-tensor propagation and AOT autograd
the same way and then calls everything as it is.  The operators' own outputs must be bit-identical to eager under
both; gradients that pass through arithmetic inductor generates itself (the float losses below) are compared
bit for bit under aot_eager and to rounding under inductor.  torch.library.opcheck repeats the checks per operator."""

import pytest
import torch

import ops_rec
from helpers import small_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


BACKENDS = ["aot_eager", "inductor"]


def compiled(fn, backend):
    graph = torch.compile(fn, backend=backend, fullgraph=True, dynamic=True)
    if backend != "inductor":
        return graph

    def call(*args, **kwargs):
        # a code generator that cannot build its own kernels on this machine (no compiler, no cache directory) says
        # nothing about the operators: that is a skip; anything dynamo or the operators raise is a failure
        try:
            return graph(*args, **kwargs)
        except torch._dynamo.exc.BackendCompilerFailed as err:
            pytest.skip(f"inductor could not generate code here: {str(err)[:200]}")

    return call


def same_grad(got, want, backend):
    if backend == "aot_eager":
        return torch.equal(got, want)
    return torch.allclose(got.float(), want.float(), rtol=2e-2, atol=2e-2 * float(want.float().abs().max()))


@pytest.mark.parametrize("backend", BACKENDS)
def test_ln_mul_compiled_matches_eager(backend):
    op = ops_rec.ascendc.activation.ln_mul
    fn = compiled(op, backend)
    for a, r, dtype in [(8, 64, torch.float32), (33, 512, torch.bfloat16), (5, 100, torch.float32)]:
        x, u = torch.randn(a, r, device=DEV).to(dtype), torch.randn(a, r, device=DEV).to(dtype)
        g, b = torch.randn(r, device=DEV), torch.randn(r, device=DEV)
        assert torch.equal(fn(x=x, u=u, gamma=g, beta=b), op(x, u, g, b))


@pytest.mark.parametrize("backend", BACKENDS)
def test_in_linear_silu_compiled_forward_and_backward(backend):
    op = ops_rec.ascendc.activation.distance_in_linear_silu
    fn = compiled(op, backend)
    for m in (100, 257):
        x = torch.randn(m, 64, device=DEV).to(torch.bfloat16)
        w = (torch.randn(512, 64, device=DEV) / 8).to(torch.bfloat16)
        b = torch.randn(512, device=DEV)
        split = [96, 96, 160, 160]
        got, want = fn(x=x, weight=w, bias=b, attr_dict=split), op(x, w, b, split)
        assert all(torch.equal(g, t) for g, t in zip(got, want))

    def loss(x, w, b):
        u, v, q, k, _ = op(x, w, b, [128] * 4)
        return (u.float() * 0.5).sum() + (v.float() * q.float()).sum() - k.float().sum()

    args = [t.requires_grad_() for t in (torch.randn(130, 64, device=DEV).to(torch.bfloat16),
                                        (torch.randn(512, 64, device=DEV) / 8).to(torch.bfloat16),
                                        torch.randn(512, device=DEV))]  # fmt: skip
    loss(*args).backward()
    eager = [t.grad.clone() for t in args]
    for t in args:
        t.grad = None
    compiled(loss, backend)(*args).backward()
    for t, e in zip(args, eager):
        assert same_grad(t.grad, e, backend)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("kw", [dict(), dict(rab=True, ctx=3, max_target=5, group=1), dict(delta=True)])
def test_hstu_jagged_compiled_forward_and_backward(kw, backend):
    w = small_case(seed=3, batch=3, heads=2, dim=64, lo=10, hi=200, dtype=torch.bfloat16, std=0.5, **kw).to(DEV)
    op = ops_rec.ascendc.attention.hstu_jagged
    args = list(w.op_args())
    want = op(*args)
    got = compiled(lambda *a: op(*a), backend)(*args)
    assert torch.equal(got, want)

    def loss(q, k, v):
        a = list(args)
        a[0], a[1], a[2] = q, k, v
        return op(*a).float().square().sum()

    qkv = [t.clone().requires_grad_() for t in (w.q, w.k, w.v)]
    loss(*qkv).backward()
    eager = [t.grad.clone() for t in qkv]
    for t in qkv:
        t.grad = None
    compiled(loss, backend)(*qkv).backward()
    for t, e in zip(qkv, eager):
        assert same_grad(t.grad, e, backend)


def test_opcheck_of_every_operator():
    checks = ("test_schema", "test_faketensor", "test_aot_dispatch_dynamic")
    x, u = torch.randn(16, 64, device=DEV), torch.randn(16, 64, device=DEV)
    torch.library.opcheck(torch.ops.ops_rec.ln_mul.default, (x, u, torch.randn(64, device=DEV), torch.randn(64, device=DEV)),
                          test_utils=checks)  # fmt: skip
    xb = torch.randn(40, 32, device=DEV).to(torch.float16).requires_grad_()
    wb = (torch.randn(128, 32, device=DEV) / 6).to(torch.float16).requires_grad_()
    bb = torch.randn(128, device=DEV).requires_grad_()
    torch.library.opcheck(torch.ops.ops_rec.distance_in_linear_silu.default, (xb, wb, bb, [32, 32, 32, 32]),
                          test_utils=checks + ("test_autograd_registration",))  # fmt: skip
    w = small_case(seed=5, batch=2, heads=2, dim=32, lo=5, hi=60, dtype=torch.float16, std=0.5).to(DEV)
    args = list(w.op_args())
    args[0], args[1], args[2] = (t.clone().requires_grad_() for t in (w.q, w.k, w.v))
    torch.library.opcheck(torch.ops.ops_rec.hstu_jagged.equal, tuple(args), test_utils=checks + ("test_autograd_registration",))
    q4 = torch.randn(2, 40, 2, 32, device=DEV).to(torch.bfloat16)
    torch.library.opcheck(torch.ops.ops_rec.hstu_dense.default, (q4, q4, q4, None, None, 0, 40, 0.0), test_utils=checks)


def test_opcheck_of_the_backward_and_paged_operators():
    from helpers import paged_case

    checks = ("test_schema", "test_faketensor", "test_aot_dispatch_dynamic")
    w = small_case(seed=8, batch=2, heads=2, dim=64, lo=5, hi=90, dtype=torch.bfloat16, std=0.5).to(DEV)
    out = ops_rec.ascendc.attention.hstu_jagged(*w.op_args())
    grad = torch.randn_like(out)
    torch.library.opcheck(torch.ops.ops_rec.hstu_jagged_backward.equal,
                          (grad, w.q, w.k, w.v, None, None, 0, w.max_seq_len, w.silu_scale, w.seq_offset, None, None, 0, w.alpha),
                          test_utils=checks)  # fmt: skip
    q4 = torch.randn(2, 48, 2, 64, device=DEV).to(torch.bfloat16)
    torch.library.opcheck(torch.ops.ops_rec.hstu_dense_backward.default,
                          (torch.randn_like(q4), q4, q4, q4, None, None, 0, 48, 0.0), test_utils=checks)  # fmt: skip
    c = {n: (t.to(DEV) if torch.is_tensor(t) else t)
         for n, t in paged_case(hist=[32, 48], prev=[0, 70], targets=[4, 6], page_size=32, heads=2, dim=32,
                                dtype=torch.float16, seed=1).items()}  # fmt: skip
    torch.library.opcheck(
        torch.ops.ops_rec.hstu_paged.default,
        (c["q"], c["k"], c["v"], c["kv_cache"], None, None, 0, c["max_seq_len"], c["max_seq_len_k"], 0.0, c["seq_offset"],
         c["seq_offset_k"], c["seq_offset_t"], c["page_offsets"], c["page_ids"], c["last_page_len"], c["num_target"], 1, 1.0),
        test_utils=checks)  # fmt: skip
    x = torch.randn(40, 32, device=DEV).to(torch.float16)
    wt = (torch.randn(128, 32, device=DEV) / 6).to(torch.float16)
    b = torch.randn(128, device=DEV)
    outs = torch.ops.ops_rec.distance_in_linear_silu(x, wt, b, [32] * 4)
    grads = [torch.randn_like(t) for t in outs[:4]]
    torch.library.opcheck(torch.ops.ops_rec.in_linear_silu_backward.default, (x, wt, b, *grads, outs[4], [32] * 4),
                          test_utils=checks)  # fmt: skip
