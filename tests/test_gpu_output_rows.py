"""The forward writes its output rows 16 bytes per lane when the output pointer allows it and in 8-byte pieces
otherwise; both paths must give the same bits, for whole and ragged query tiles, padded head dims and every 16-bit
output type, and must leave the memory around the output alone."""

import pytest
import torch

import ops_rec  # noqa: F401
from ops_rec import _ops, workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def prepare(w):
    return _ops.prepare_forward(w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, w.max_seq_len,
                                w.silu_scale, w.seq_offset, w.seq_offset, w.num_context, w.num_target,
                                w.target_group_size, w.alpha)  # fmt: skip


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim, heads", [(32, 3), (64, 2), (128, 4), (256, 1), (48, 2), (96, 2)])
def test_misaligned_output_pointer_gives_the_same_bits(dtype, dim, heads):
    w = workloads.make("rows", dtype=dtype, device=DEV, seed=21, batch=5, heads=heads, dim=dim, lo=1, hi=300)
    p = prepare(w)
    want = p.launch().clone()
    torch.cuda.synchronize()
    n_bytes = want.numel() * want.element_size()
    guard = 256
    # the same call with the output 8 bytes off a 16-byte boundary, inside a buffer of a known byte pattern
    raw = torch.full((n_bytes + 2 * guard,), 0x5A, dtype=torch.uint8, device=DEV)
    assert raw.data_ptr() % 16 == 0
    p.params.out = raw.data_ptr() + guard + 8
    p.launch()
    torch.cuda.synchronize()
    got = raw[guard + 8 : guard + 8 + n_bytes].view(dtype).view(want.shape)
    assert torch.equal(got, want)
    assert bool((raw[: guard + 8] == 0x5A).all()) and bool((raw[guard + 8 + n_bytes :] == 0x5A).all())
    # and 16-byte aligned in the same buffer: nothing outside the output is touched by the wide stores either
    raw.fill_(0x5A)
    p.params.out = raw.data_ptr() + guard
    p.launch()
    torch.cuda.synchronize()
    got = raw[guard : guard + n_bytes].view(dtype).view(want.shape)
    assert torch.equal(got, want)
    assert bool((raw[:guard] == 0x5A).all()) and bool((raw[guard + n_bytes :] == 0x5A).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dim, heads, heads_k", [(64, 2, 2), (128, 4, 2), (256, 1, 1)])
def test_misaligned_gradient_pointers_give_the_same_bits(monkeypatch, dtype, dim, heads, heads_k):
    """dq / dk / dv rows are written 16 bytes per lane into 16-byte aligned tensors and in 8-byte pieces otherwise."""
    w = workloads.make("grads", dtype=dtype, device=DEV, seed=22, batch=4, heads=heads, heads_k=heads_k, dim=dim, lo=1, hi=300)
    g = torch.Generator(device=DEV).manual_seed(5)
    grad = (torch.randn(w.q.shape[0], heads, dim, generator=g, device=DEV) * 0.1).to(dtype)
    args = (grad, w.q, w.k, w.v, None, None, 0, w.max_seq_len, w.max_seq_len, w.silu_scale, w.seq_offset, w.seq_offset,
            None, None, 1, w.alpha)  # fmt: skip
    want = _ops._backward_hip(*args)[:3]
    torch.cuda.synchronize()
    assert all(t.data_ptr() % 16 == 0 for t in want)

    def off_by_eight_bytes(like):
        buf = torch.full((like.numel() + 16,), 7.0, dtype=like.dtype, device=like.device)
        view = buf[4 : 4 + like.numel()].view(like.shape)
        assert view.data_ptr() % 16 == 8
        view._keep = buf  # noqa: SLF001  (the guard elements are checked below)
        return view

    monkeypatch.setattr(_ops, "_new_grad", off_by_eight_bytes)
    got = _ops._backward_hip(*args)[:3]
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)
        buf = a._keep
        assert bool((buf[:4] == 7.0).all()) and bool((buf[4 + a.numel() :] == 7.0).all())


@pytest.mark.parametrize("max_len", [203, 208])
@pytest.mark.parametrize("shift", [0, 1, 4, 7])
def test_bias_gradient_is_written_in_full(monkeypatch, shift, max_len):
    """The call clears the attn_bias gradient itself (the key-tile kernel does it beside its work): a tensor full of
    other values, at any 2-byte alignment, comes back equal to the gradient written into a cleared one, and the
    memory around it is left alone."""
    w = workloads.make("dbias", dtype=torch.bfloat16, device=DEV, seed=23, batch=3, heads=2, dim=64, lo=10, hi=200,
                       max_seq_len=max_len, rab_std=0.3)  # fmt: skip
    g = torch.Generator(device=DEV).manual_seed(6)
    grad = (torch.randn(w.q.shape[0], 2, 64, generator=g, device=DEV) * 0.1).to(torch.bfloat16)
    args = (grad, w.q, w.k, w.v, None, w.attn_bias, 0, w.max_seq_len, w.max_seq_len, w.silu_scale, w.seq_offset,
            w.seq_offset, None, None, 1, w.alpha)  # fmt: skip
    monkeypatch.setattr(_ops, "_new_grad", torch.zeros_like)
    want = _ops._backward_hip(*args)
    torch.cuda.synchronize()
    assert float(want[3].float().abs().max()) > 0

    def poisoned(like):
        buf = torch.full((like.numel() + 32,), 7.0, dtype=like.dtype, device=like.device)
        view = buf[8 + shift : 8 + shift + like.numel()].view(like.shape)
        view._keep = buf  # noqa: SLF001
        return view

    monkeypatch.setattr(_ops, "_new_grad", poisoned)
    got = _ops._backward_hip(*args)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert torch.equal(a, b)
        buf = a._keep
        assert bool((buf[: 8 + shift] == 7.0).all()) and bool((buf[8 + shift + a.numel() :] == 7.0).all())


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_fp8_misaligned_output_pointer_gives_the_same_bits(out_dtype, dim):
    """fp8 inputs: a sub-tile slot holds 16 of a wavefront's 32 output rows, so the rows pass through two slots."""
    w = workloads.make("rows8", dtype=torch.bfloat16, device=DEV, seed=24, batch=4, heads=2, dim=dim, lo=1, hi=300)
    (q8, qs), (k8, ks), (v8, vs) = (workloads.quantize_fp8(t) for t in (w.q, w.k, w.v))
    p = _ops.prepare_forward(q8, k8, v8, None, None, 0, w.max_seq_len, w.max_seq_len, w.silu_scale, w.seq_offset,
                             w.seq_offset, None, None, 1, w.alpha, out_dtype=out_dtype, q_descale=qs, k_descale=ks,
                             v_descale=vs)  # fmt: skip
    want = p.launch().clone()
    torch.cuda.synchronize()
    assert want.dtype == out_dtype and float(want.float().abs().max()) > 0
    n_bytes = want.numel() * want.element_size()
    guard = 256
    for shift in (8, 0):
        raw = torch.full((n_bytes + 2 * guard,), 0x5A, dtype=torch.uint8, device=DEV)
        p.params.out = raw.data_ptr() + guard + shift
        p.launch()
        torch.cuda.synchronize()
        got = raw[guard + shift : guard + shift + n_bytes].view(out_dtype).view(want.shape)
        assert torch.equal(got, want)
        assert bool((raw[: guard + shift] == 0x5A).all()) and bool((raw[guard + shift + n_bytes :] == 0x5A).all())


def test_no_keys_at_all_still_clears_every_gradient(monkeypatch):
    """Every sequence without keys: the key-tile kernel has nothing to run on, so the bias gradient is cleared by a
    fill of its own; dq is all zeros."""
    dt, heads, dim, max_q, max_k = torch.bfloat16, 2, 64, 40, 16
    g = torch.Generator(device=DEV).manual_seed(7)
    q = torch.randn(45, heads, dim, generator=g, device=DEV).to(dt)
    k = torch.empty(0, heads, dim, device=DEV, dtype=dt)
    v = torch.empty(0, heads, dim, device=DEV, dtype=dt)
    offs_q = torch.tensor([0, 5, 45], dtype=torch.int32, device=DEV)
    offs_k = torch.zeros(3, dtype=torch.int32, device=DEV)
    bias = torch.randn(2, heads, max_q, max_k, generator=g, device=DEV).to(dt)
    grad = torch.randn(45, heads, dim, generator=g, device=DEV).to(dt)
    monkeypatch.setattr(_ops, "_new_grad", lambda like: torch.full_like(like, 7.0))
    dq, dk, dv, dbias = _ops._backward_hip(grad, q, k, v, None, bias, 0, max_q, max_k, 1.0, offs_q, offs_k, None, None,
                                           1, 0.125)  # fmt: skip
    torch.cuda.synchronize()
    assert dk.numel() == 0 and dv.numel() == 0
    assert float(dq.float().abs().max()) == 0.0 and float(dbias.float().abs().max()) == 0.0


@pytest.mark.parametrize("dim, short", [(64, None), (128, None), (128, "0")])
def test_rows_that_belong_to_no_work_item_are_left_alone(dim, short, monkeypatch):
    """The precondition of the C ABI, pinned: with a non-zero first offset or a sequence longer than ``max_seq_len``
    the rows before the first offset and the rows of that sequence past ``max_seq_len`` are neither read nor written
    (the reference's adapter hands out zeros there, torch_extension/hstu_jagged_plugin.cpp:56-59: a documented
    difference); every other row is written exactly as in the well-formed call, rows past the last offset as zeros."""
    import helpers

    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", short)  # (head dim 128: both forward kernels)
    max_len, lead, trail = 150, 3, 5
    lengths = [40, 190, 150, 7]  # the second one is 40 rows longer than max_seq_len
    w = workloads.make("pre", dtype=torch.bfloat16, device=DEV, seed=31, batch=4, heads=2, dim=dim, lo=0, hi=0,
                       lengths=lengths, max_seq_len=max_len)  # fmt: skip
    total = sum(lengths)
    pad = lambda t: torch.cat([torch.ones(lead, *t.shape[1:], dtype=t.dtype, device=DEV), t,
                               torch.ones(trail, *t.shape[1:], dtype=t.dtype, device=DEV)])  # noqa: E731
    q, k, v = pad(w.q), pad(w.k), pad(w.v)
    offs = (w.seq_offset + lead).contiguous()
    p = _ops.prepare_forward(q, k, v, None, None, 0, max_len, max_len, w.silu_scale, offs, offs, None, None, 0, w.alpha)
    p.out.fill_(float("nan"))
    out = p.launch()
    torch.cuda.synchronize()
    o = offs.cpu().tolist()
    written = torch.zeros(lead + total + trail, dtype=torch.bool)
    for b, n in enumerate(lengths):
        written[o[b] : o[b] + min(n, max_len)] = True
    written[o[-1] :] = True  # rows past the last offset: zero-filled
    nan_rows = torch.isnan(out.float()).all(dim=(1, 2)).cpu()
    finite_rows = torch.isfinite(out.float()).all(dim=(1, 2)).cpu()
    assert torch.equal(nan_rows, ~written) and torch.equal(finite_rows, written)
    assert (out[o[-1] :] == 0).all()
    # the rows that are written equal those of the same sequences in a well-formed call (the long one cut to max_seq_len)
    cut = [min(n, max_len) for n in lengths]
    rows = torch.cat([torch.arange(o[b], o[b] + cut[b]) for b in range(4)]).to(DEV)
    good = workloads.Workload(name="good", q=q[rows], k=k[rows], v=v[rows],
                              seq_offset=torch.tensor([0] + list(torch.tensor(cut).cumsum(0)), dtype=offs.dtype, device=DEV),
                              max_seq_len=max_len, silu_scale=w.silu_scale, alpha=w.alpha, lengths=cut)  # fmt: skip
    want = ops_rec.ascendc.attention.hstu_jagged(*good.op_args())
    assert torch.equal(out[rows], want)
