"""The three operators chained as in an HSTU layer (in_linear_silu -> hstu_jagged -> ln_mul), bf16 end to end, against
the same chain in fp32 torch operations: what the second operator reads is exactly what the first wrote (layouts,
dtypes and views compose without a copy or cast in between)."""

import importlib.util
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ops-rec_amd", "examples",
                     "hstu_layer_example.py")  # fmt: skip
_spec = importlib.util.spec_from_file_location("hstu_layer_example", _PATH)
example = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(example)


@pytest.mark.parametrize("heads,dim,embed,lengths", [(2, 64, 32, [5, 130, 77]), (4, 128, 128, [300, 1, 258, 64])])
def test_chain_matches_fp32_chain(heads, dim, embed, lengths):
    dev = torch.device("cuda", 0)
    g = torch.Generator(device=dev).manual_seed(len(lengths))
    offsets = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32, device=dev)
    t, hd = sum(lengths), heads * dim
    x = torch.randn(t, embed, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(4 * hd, embed, generator=g, device=dev) / embed**0.5).to(torch.bfloat16)
    b = torch.randn(4 * hd, generator=g, device=dev) * 0.1
    gamma = 1.0 + 0.1 * torch.randn(hd, generator=g, device=dev)
    beta = 0.1 * torch.randn(hd, generator=g, device=dev)
    args = (x, w, b, gamma, beta, offsets, heads, dim, max(lengths))
    got = example.block(*args)
    want = example.block_fp32(*args)
    assert got.shape == (t, hd) and got.dtype == torch.bfloat16
    # LayerNorm divides by the spread of an attention output row: a bf16 rounding of O (2^-9 relative) comes out
    # amplified, so the bar is relative to the largest value, with most elements far inside it
    scale = want.abs().max().item()
    diff = (got.float() - want).abs()
    assert diff.max().item() <= 0.05 * scale
    assert diff.mean().item() <= 0.004 * scale
