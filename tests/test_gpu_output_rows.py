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
