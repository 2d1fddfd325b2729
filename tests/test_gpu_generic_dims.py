"""Head dims the tuned kernels do not take -- above 256 (the reference goes to 512,
hstu_forward_v1/op_host/tiling_policy.cpp:68-93) or a q/k head dim that is not a multiple of 8 -- run through the
matrix-pipe kernel for head dims up to 512 (16-bit inputs, q/k head dim a multiple of 8) or the kernel written for
coverage.  Same oracle, same tolerances as the parity tests (bf16 / fp16: atol = rtol = 1e-2 of
the largest reference value; fp32: 1e-4)."""

import dataclasses

import pytest
import torch

import ops_rec
from ops_rec import _ops
from oracle import hstu_oracle as O
from helpers import small_case
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def expected_kernel(w):
    """16-bit inputs with a head dim above 256 and a q/k head dim that is a multiple of 8 take the matrix-pipe kernel
    for head dims up to 512; everything else here takes the kernel written for coverage."""
    d_qk, d_v = w.q.shape[2], w.v.shape[2]
    wide = w.q.dtype != torch.float32 and max(d_qk, d_v) > 256 and d_qk % 8 == 0
    return "hstu_fwd_wide_" if wide else "hstu_fwd_generic_"


def check(w, expect_generic=True):
    d = w.to(DEV)
    k_offs = d.seq_offset if d.seq_offset_k is None else d.seq_offset_k
    max_k = d.max_seq_len if d.max_seq_len_k is None else d.max_seq_len_k
    prepared = _ops.prepare_forward(d.q, d.k, d.v, d.mask, d.attn_bias, d.mask_type, d.max_seq_len, max_k, d.silu_scale,
                                    d.seq_offset, k_offs, d.num_context, d.num_target, d.target_group_size, d.alpha)  # fmt: skip
    if expect_generic:
        assert prepared.kernel_name().startswith(expected_kernel(w)), prepared.kernel_name()
    else:
        assert not prepared.kernel_name().startswith(("hstu_fwd_generic_", "hstu_fwd_wide_")), prepared.kernel_name()
    out = ops_rec.ascendc.attention.hstu_jagged(*d.op_args())
    ref = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    assert out.dtype == w.q.dtype and out.shape == ref.shape
    tol = 1e-4 if w.q.dtype == torch.float32 else 1e-2
    scale = max(1.0, float(ref.abs().max()))
    torch.testing.assert_close(out.float().cpu(), ref, rtol=tol, atol=tol * scale)
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("dim,dim_v", [(1, 16), (4, 16), (12, 48), (20, 32), (100, 112), (130, 64), (260, 272), (384, 384),
                                       (512, 512), (64, 512), (512, 16)])  # fmt: skip
def test_head_dims_beyond_the_tuned_kernels(dtype, dim, dim_v):
    check(small_case(seed=dim + dim_v, batch=3, heads=2, dim=dim, dim_v=dim_v, lo=1, hi=150, dtype=dtype, std=0.5))


@pytest.mark.parametrize("kw", [
    dict(rab=True), dict(custom_mask=True), dict(rab=True, custom_mask=True), dict(ctx=5, max_target=7, group=2),
    dict(ctx=3, max_target=4, group=1, rab=True), dict(heads=4, heads_k=2), dict(heads=8, heads_k=1, rab=True),
    dict(delta=True), dict(delta=True, rab=True, index_dtype=torch.int64), dict(alpha=0.3, rab=True),
])  # fmt: skip
def test_all_the_semantics_at_an_odd_head_dim(kw):
    base = dict(seed=len(kw) + 11, batch=4, heads=2, dim=36, dim_v=48, lo=20, hi=160, dtype=torch.bfloat16, std=0.5)
    base.update(kw)
    check(small_case(**base))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("kw", [
    dict(), dict(rab=True), dict(custom_mask=True), dict(rab=True, custom_mask=True), dict(ctx=5, max_target=7, group=2),
    dict(ctx=3, max_target=40, group=3, rab=True), dict(heads=4, heads_k=2), dict(heads=8, heads_k=1, rab=True),
    dict(delta=True), dict(delta=True, rab=True, index_dtype=torch.int64), dict(alpha=0.3, rab=True),
    dict(dim=264, dim_v=512), dict(dim=512, dim_v=272, rab=True), dict(lo=257, hi=257, rab=True, custom_mask=True),
])  # fmt: skip
def test_all_the_semantics_at_head_dims_above_256(kw, dtype):
    # several 32-key sub-tiles and query tiles per sequence, bias rows of every alignment (lengths are random)
    base = dict(seed=len(kw) + 31, batch=3, heads=2, dim=320, dim_v=384, lo=90, hi=330, dtype=dtype, std=0.4)
    base.update(kw)
    w = small_case(**base)
    assert expected_kernel(w) == "hstu_fwd_wide_"
    check(w)


def test_no_mask_and_long_rows_at_head_dim_512():
    w = small_case(seed=5, batch=2, heads=2, dim=512, dim_v=512, lo=200, hi=300, dtype=torch.float16, std=0.3)
    check(dataclasses.replace(w, mask_type=2))


def test_rows_past_the_last_offset_are_zero_and_empty_sequences_cost_nothing():
    w = small_case(seed=6, batch=4, heads=2, dim=20, dim_v=32, lo=1, hi=40, dtype=torch.bfloat16, std=0.5)
    # two more rows than the offsets cover, and a repeated trailing offset (an empty last sequence)
    pad = lambda t: torch.cat([t, torch.ones(2, *t.shape[1:], dtype=t.dtype)])  # noqa: E731
    offs = torch.cat([w.seq_offset, w.seq_offset[-1:]])
    w2 = dataclasses.replace(w, q=pad(w.q), k=pad(w.k), v=pad(w.v), seq_offset=offs, lengths=w.lengths + [0])
    out = check(w2)
    assert torch.count_nonzero(out[-2:]) == 0


def check_backward(w, seed=3):
    """dq, dk, dv (and the attn_bias gradient) of the generic backward kernels, through loss.backward(), against
    autograd on the fp32 oracle: fp32 inputs within 2e-4 of the largest reference value, 16-bit inputs within 1e-2
    (their gradients are rounded to the input type)."""
    d = w.to(DEV)
    q, k, v = (t.clone().requires_grad_() for t in (d.q, d.k, d.v))
    bias = d.attn_bias.clone().requires_grad_() if d.attn_bias is not None else None
    args = list(d.op_args())
    args[0], args[1], args[2], args[4] = q, k, v, bias
    out = ops_rec.ascendc.attention.hstu_jagged(*args)
    g = torch.Generator().manual_seed(seed)
    grad_out = torch.randn(out.shape, generator=g).to(out.dtype)
    out.backward(grad_out.to(DEV))
    qc, kc, vc = (t.float().clone().requires_grad_() for t in (w.q, w.k, w.v))
    kw = w.oracle_kwargs()
    bc = None
    if w.attn_bias is not None:
        bc = w.attn_bias.float().clone().requires_grad_()
        kw["attn_bias"] = bc
    O.hstu_jagged_forward(qc, kc, vc, out_dtype=torch.float32, **kw).backward(grad_out.float())
    tol = 2e-4 if w.q.dtype == torch.float32 else 1e-2
    pairs = [("dq", q.grad, qc.grad), ("dk", k.grad, kc.grad), ("dv", v.grad, vc.grad)]
    if bias is not None:
        pairs.append(("dbias", bias.grad, bc.grad))
    for name, got, ref in pairs:
        assert got.dtype == w.q.dtype and got.shape == ref.shape, name
        assert torch.isfinite(got).all(), name
        torch.testing.assert_close(got.float().cpu(), ref, rtol=tol, atol=tol * max(1e-3, float(ref.abs().max())),
                                   msg=lambda m, n=name: f"{n}: {m}")  # fmt: skip


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("dim,dim_v", [(1, 16), (12, 48), (20, 32), (130, 64), (260, 272), (512, 512), (64, 512), (512, 16)])
def test_backward_at_head_dims_beyond_the_tuned_kernels(dtype, dim, dim_v):
    check_backward(small_case(seed=dim + dim_v, batch=3, heads=2, dim=dim, dim_v=dim_v, lo=1, hi=90, dtype=dtype, std=0.5))


@pytest.mark.parametrize("kw", [
    dict(), dict(rab=True), dict(custom_mask=True), dict(rab=True, custom_mask=True), dict(ctx=5, max_target=7, group=2),
    dict(ctx=3, max_target=4, group=1, rab=True), dict(heads=4, heads_k=2), dict(heads=8, heads_k=1, rab=True),
    dict(delta=True), dict(delta=True, rab=True, index_dtype=torch.int64), dict(alpha=0.3, rab=True),
    dict(dim=64, dim_v=64), dict(dim=128, dim_v=128, rab=True, hi=300),
])  # fmt: skip
@pytest.mark.parametrize("generic", ["0", "1"])
def test_backward_of_fp32_inputs_with_all_the_semantics(kw, generic, monkeypatch):
    # fp32 inputs with head dims up to 128 and a q/k head dim that is a multiple of 8 run on the fp32 matrix-instruction
    # backward kernels; HSTU_MI355_GENERIC_BACKWARD=1 sends the same cases through the generic kernels
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", generic)
    base = dict(seed=len(kw) + 23, batch=4, heads=2, dim=32, dim_v=48, lo=20, hi=160, dtype=torch.float32, std=0.5)
    base.update(kw)
    # the matrix-instruction kernels in both of their orders: everything computed where it is used, and dS and P handed
    # from the query-tile kernel to the key-tile kernel through a workspace (filled with NaN here: nothing in it is
    # cleared, the key-tile kernel reads what was written)
    for order in (("0", "2") if generic == "0" else ("0",)):
        helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
        helpers.poison_workspace(monkeypatch)
        check_backward(small_case(**base))


@pytest.mark.parametrize("kw", [
    dict(dim=32, dim_v=32, lo=1, hi=700), dict(dim=64, dim_v=48, lo=100, hi=520, rab=True, custom_mask=True),
    dict(dim=128, dim_v=128, lo=0, hi=400, ctx=9, max_target=50, group=4), dict(dim=16, dim_v=16, lo=0, hi=260, delta=True, rab=True),
    dict(dim=8, dim_v=128, lo=127, hi=129, heads=6, heads_k=2, rab=True), dict(dim=104, dim_v=80, lo=255, hi=257, custom_mask=True),
], ids=lambda kw: "-".join(f"{k}{v}" for k, v in kw.items()))  # fmt: skip
@pytest.mark.parametrize("order", ["0", "2"], ids=["recompute", "planes"])
def test_backward_of_fp32_inputs_over_several_query_and_key_tiles(kw, order, monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", order)
    helpers.poison_workspace(monkeypatch)
    base = dict(seed=len(kw) + 41, batch=3, heads=2, dtype=torch.float32, std=0.5)
    base.update(kw)
    check_backward(small_case(**base))


def test_backward_without_mask_and_with_rows_past_the_last_offset():
    w = small_case(seed=9, batch=3, heads=2, dim=24, dim_v=32, lo=1, hi=70, dtype=torch.float32, std=0.5)
    pad = lambda t: torch.cat([t, torch.ones(3, *t.shape[1:], dtype=t.dtype)])  # noqa: E731
    w = dataclasses.replace(w, q=pad(w.q), k=pad(w.k), v=pad(w.v), mask_type=2)
    check_backward(w)


def test_backward_runs_on_the_generic_kernels_for_these_dims():
    w = small_case(seed=7, batch=2, heads=2, dim=12, dim_v=16, lo=10, hi=50, dtype=torch.bfloat16, std=0.5).to(DEV)
    q, k, v = (t.clone().requires_grad_() for t in (w.q, w.k, w.v))
    args = list(w.op_args())
    args[0], args[1], args[2] = q, k, v
    out = ops_rec.ascendc.attention.hstu_jagged(*args)
    out.float().sum().backward()
    c = w.to("cpu")
    qc, kc, vc = (t.float().clone().requires_grad_() for t in (c.q, c.k, c.v))
    O.hstu_jagged_forward(qc, kc, vc, out_dtype=torch.float32, **c.oracle_kwargs()).sum().backward()
    for g, r in ((q.grad, qc.grad), (k.grad, kc.grad), (v.grad, vc.grad)):
        torch.testing.assert_close(g.float().cpu(), r, rtol=2e-2, atol=2e-2 * float(r.abs().max()))


WINDOW_CASES = {
    "plain_512": dict(batch=3, heads=2, dim=512, lo=1, hi=328, max_seq_len=328),
    "dims_384_320": dict(batch=3, heads=2, dim=384, dim_v=320, lo=40, hi=200, max_seq_len=200),
    "dims_64_512": dict(batch=2, heads=2, dim=64, dim_v=512, lo=1, hi=130, max_seq_len=136),
    "dims_512_16": dict(batch=2, heads=2, dim=512, dim_v=16, lo=1, hi=130, max_seq_len=136),
    "dims_272": dict(batch=2, heads=3, dim=272, lo=100, hi=300, max_seq_len=304),
    "bias_and_its_gradient": dict(batch=3, heads=2, dim=512, lo=30, hi=264, max_seq_len=264, rab_std=0.5),
    "context_targets_groups_bias": dict(batch=3, heads=2, dim=320, dim_v=384, lo=60, hi=264, max_seq_len=264, rab_std=0.5,
                                        num_context=5, max_target=33, target_group_size=3),
    "grouped_heads": dict(batch=3, heads=4, heads_k=2, dim=512, lo=1, hi=200, max_seq_len=200),
    "one_kv_head_bias": dict(batch=2, heads=6, heads_k=1, dim=288, dim_v=512, lo=90, hi=160, max_seq_len=160, rab_std=0.5),
    "int64_offsets": dict(batch=2, heads=2, dim=512, lo=33, hi=160, max_seq_len=160, index_dtype=torch.int64),
}


# (context and target rows belong to the built-in mask: such cases run with it only)
WINDOW_CASES_BY_MASK = [(name, mask) for name in WINDOW_CASES for mask in ("builtin", "custom", "none")
                        if mask == "builtin" or "num_context" not in WINDOW_CASES[name]]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name,mask", WINDOW_CASES_BY_MASK, ids=[f"{n}-{m}" for n, m in WINDOW_CASES_BY_MASK])
def test_backward_above_head_dim_256_as_two_windows(name, mask, dtype, monkeypatch):
    """16-bit inputs with head dims in (256, 512] that are multiples of 16, rows of 16 bytes in the planes
    (max_seq_len_k a multiple of 8): the kernels of the head-dim slot 256 over two windows per head, with the workspace
    the library asks for -- the pair plane of the planes order plus 256 bytes per (query row, 32-key block, head) of
    fp32 partial scores -- full of NaN.  Without the workspace, and with HSTU_MI355_GENERIC_BACKWARD=1, the generic
    kernels take the call."""
    from ops_rec import _ops, workloads

    kw = dict(WINDOW_CASES[name])
    w = workloads.make("win", dtype=dtype, std=0.4, seed=len(name), **kw)
    if mask == "custom":
        g = torch.Generator().manual_seed(4)
        shape = (len(w.lengths), w.q.shape[1], w.max_seq_len, w.max_seq_len)
        w = dataclasses.replace(w, mask=(torch.rand(shape, generator=g) < 0.7).to(dtype), mask_type=3)
    elif mask == "none":
        w = dataclasses.replace(w, mask_type=2)
    asked = []
    plain = _ops._new_workspace

    def poisoned(n_bytes, device):
        asked.append(n_bytes)
        ws = plain(n_bytes, device)
        if ws is not None:
            ws.fill_(0xFF)
        return ws

    monkeypatch.setattr(_ops, "_new_workspace", poisoned)
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", None)
    check_backward(w)
    rows, heads, blocks = w.q.shape[0], w.q.shape[1], (w.max_seq_len + 31) // 32
    partial = heads * rows * blocks * 256
    assert asked and asked[-1] > partial and (asked[-1] - partial) % (128 * heads) == 0, (asked, partial)
    # the generic kernels on the same inputs: no workspace
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", "1")
    check_backward(w)
    assert asked[-1] == 0
    helpers.set_switch(monkeypatch, "HSTU_MI355_GENERIC_BACKWARD", None)
    helpers.withhold_workspace(monkeypatch)
    check_backward(w)


def test_backward_windows_and_rows_that_are_not_16_byte_pieces(monkeypatch):
    """Rows of [max_q][max_k] tensors are 16-byte pieces only when max_seq_len_k is a multiple of 8: a call with an
    attn_bias at another max_seq_len_k stays on the generic kernels (no workspace), one without such tensors takes the
    windows all the same; a head dim that is not a multiple of 16 stays on the generic kernels either way."""
    from ops_rec import _ops, workloads

    asked = []
    plain = _ops._new_workspace
    monkeypatch.setattr(_ops, "_new_workspace", lambda n, dev: (asked.append(n), plain(n, dev))[1])
    w = workloads.make("win", dtype=torch.bfloat16, std=0.4, batch=2, heads=2, dim=512, lo=1, hi=90, max_seq_len=90, rab_std=0.5)
    check_backward(w)
    assert asked[-1] == 0
    w = workloads.make("win", dtype=torch.bfloat16, std=0.4, batch=2, heads=2, dim=512, lo=1, hi=90, max_seq_len=90)
    check_backward(w)
    assert asked[-1] > 0
    w = workloads.make("win", dtype=torch.bfloat16, std=0.4, batch=2, heads=2, dim=264, dim_v=272, lo=1, hi=88, max_seq_len=88)
    check_backward(w)  # a head dim that is not a multiple of 16
    assert asked[-1] == 0
