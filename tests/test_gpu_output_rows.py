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
