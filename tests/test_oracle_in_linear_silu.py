"""Pins the in_linear_silu oracle by checks that do not repeat its formula."""

import pytest
import torch

from oracle import in_linear_silu_oracle as O


def rnd(m, n, k, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(m, k, generator=g, dtype=torch.float64).to(dtype),
            (torch.randn(n, k, generator=g, dtype=torch.float64) / k**0.5).to(dtype),
            torch.randn(n, generator=g, dtype=torch.float64))  # fmt: skip


@pytest.mark.parametrize("m,n,k,split", [(5, 64, 16, [16, 16, 16, 16]), (33, 256, 64, [48, 48, 80, 80]),
                                         (7, 128, 32, [16, 32, 64, 16])])  # fmt: skip
def test_against_library_calls_of_the_reference_golden(m, n, k, split):
    # test_in_linear_silu.py:36-49: addmm, silu, split
    x, w, b = rnd(m, n, k, m + n + k)
    mixed = torch.addmm(b, x, w.t())
    want = torch.split(torch.nn.functional.silu(mixed), split, dim=-1)
    got = O.in_linear_silu(x, w, b, split)
    for g, t in zip(got[:4], want):
        torch.testing.assert_close(g, t, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(got[4], mixed, rtol=1e-12, atol=1e-13)


def test_every_output_column_names_its_weight_row():
    # x = one-hot rows: mixed[i, j] = weight[j, i]; with weight[j, i] = j + i / 100 each output element tells which weight
    # row and column made it, so a transposed operand, a shifted split boundary or swapped outputs cannot pass
    k, split = 16, [16, 48, 32, 32]
    n = sum(split)
    x = torch.eye(k, dtype=torch.float64)
    w = torch.arange(n, dtype=torch.float64)[:, None] + torch.arange(k, dtype=torch.float64)[None, :] / 100.0
    user, value, query, key, lin = O.in_linear_silu(x, w, None, split)
    assert lin.shape == (k, n) and [t.shape[1] for t in (user, value, query, key)] == split
    for i in range(k):
        for j in (0, 15, 16, 63, 64, 95, 96, 127):
            assert lin[i, j].item() == pytest.approx(j + i / 100.0)
    silu = lambda v: v / (1.0 + torch.exp(-v))  # noqa: E731
    assert value[3, 0].item() == pytest.approx(silu(torch.tensor(16.03, dtype=torch.float64)).item())
    assert query[2, 31].item() == pytest.approx(silu(torch.tensor(95.02, dtype=torch.float64)).item())
    assert key[0, 0].item() == pytest.approx(silu(torch.tensor(96.0, dtype=torch.float64)).item())
    assert user[5, 15].item() == pytest.approx(silu(torch.tensor(15.05, dtype=torch.float64)).item())


def test_bias_only_and_known_silu_values():
    # x = 0: mixed = bias; silu(0) = 0, silu(large) -> identity, silu(-large) -> 0, silu(1) = 1 / (1 + 1/e)
    n, k = 64, 16
    b = torch.zeros(n, dtype=torch.float64)
    b[1], b[2], b[3] = 1.0, 40.0, -40.0
    outs = O.in_linear_silu(torch.zeros(3, k, dtype=torch.float64), torch.ones(n, k, dtype=torch.float64), b, [16] * 4)
    u = outs[0]
    assert u[0, 0].item() == 0.0
    assert u[1, 1].item() == pytest.approx(1.0 / (1.0 + 2.718281828459045**-1))
    assert u[2, 2].item() == pytest.approx(40.0)
    assert abs(u[0, 3].item()) < 1e-15
    torch.testing.assert_close(outs[4], b.expand(3, n))


def test_rounding_points_of_the_kernel():
    # linear_output is rounded once; SiLU is taken of the ROUNDED value and rounded again
    k, n = 16, 64
    x = torch.zeros(1, k, dtype=torch.float64)
    b = torch.full((n,), 1.00390625 + 2.0**-10, dtype=torch.float64)  # between two bf16 values 1.0 and 1.0078125
    outs = O.in_linear_silu(x, torch.zeros(n, k, dtype=torch.float64), b, [16] * 4, round_to=torch.bfloat16)
    assert outs[4][0, 0].item() == 1.0078125
    want = torch.tensor(1.0078125, dtype=torch.float64)
    want = (want / (1.0 + torch.exp(-want))).float().to(torch.bfloat16).double()
    assert outs[0][0, 0].item() == want.item()
    exact = O.in_linear_silu(x, torch.zeros(n, k, dtype=torch.float64), b, [16] * 4)
    assert exact[4][0, 0].item() == b[0].item()


def test_backward_against_autograd_of_the_forward():
    m, n, k, split = 9, 128, 32, [16, 48, 32, 32]
    x, w, b = (t.requires_grad_() for t in rnd(m, n, k, 5))
    outs = O.in_linear_silu(x, w, b, split)
    g = torch.Generator().manual_seed(6)
    grads = [torch.randn(m, s, generator=g, dtype=torch.float64) for s in split]
    loss = sum((o * gr).sum() for o, gr in zip(outs[:4], grads))
    dx, dw, db = torch.autograd.grad(loss, (x, w, b))
    got = O.in_linear_silu_backward(x.detach(), w.detach(), grads, outs[4].detach())
    for a_, b_ in zip(got, (dx, dw, db)):
        torch.testing.assert_close(a_, b_, rtol=1e-10, atol=1e-12)


def test_shape_errors():
    x, w, b = rnd(3, 64, 16, 1)
    with pytest.raises(ValueError):
        O.in_linear_silu(x, w, b, [16, 16, 16])
    with pytest.raises(ValueError):
        O.in_linear_silu(x, w, b, [16, 16, 16, 32])
    with pytest.raises(ValueError):
        O.in_linear_silu(x, w[:, :8], b, [16] * 4)
