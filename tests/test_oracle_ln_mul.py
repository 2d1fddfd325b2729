"""Pins the ln_mul oracle by checks that do not repeat its formula: a library routine, closed forms, invariants,
and the inputs of the reference's own example."""

import numpy as np
import pytest
import torch

from oracle import ln_mul_oracle as L


def rnd(a, r, seed):
    g = np.random.default_rng(seed)
    return (g.standard_normal((a, r)), g.standard_normal((a, r)), g.standard_normal(r), g.standard_normal(r))


@pytest.mark.parametrize("a,r", [(1, 1), (3, 4), (7, 13), (16, 64), (5, 512), (2, 2048), (3, 5000)])
def test_against_library_layer_norm(a, r):
    x, u, gamma, beta = rnd(a, r, a * 1000 + r)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x), (r,), torch.from_numpy(gamma), torch.from_numpy(beta),
                                          eps=1e-5) * torch.from_numpy(u)  # fmt: skip
    np.testing.assert_allclose(L.ln_mul(x, u, gamma, beta), want.numpy(), rtol=1e-11, atol=1e-12)


def test_population_variance_not_sample_variance():
    # ddof = 0 (test_ln_mul.py:43): with two columns x = (-1, 1) the variance is 1, not 2
    x = np.array([[-1.0, 1.0]])
    one, zero = np.ones(2), np.zeros(2)
    got = L.ln_mul(x, np.ones((1, 2)), one, zero, eps=0.0)
    np.testing.assert_allclose(got, [[-1.0, 1.0]], rtol=0, atol=1e-15)


def test_epsilon_is_inside_the_root():
    # var = 1, eps = 3: rstd = 1 / sqrt(4) = 0.5 (outside the root it would be 1 / (1 + 3))
    x = np.array([[-1.0, 1.0]])
    got = L.ln_mul(x, np.ones((1, 2)), np.ones(2), np.zeros(2), eps=3.0)
    np.testing.assert_allclose(got, [[-0.5, 0.5]], rtol=0, atol=1e-15)
    assert L.EPSILON == 1e-5


def test_single_column_and_constant_rows_give_beta_times_u():
    x, u, gamma, beta = rnd(6, 1, 1)
    np.testing.assert_allclose(L.ln_mul(x, u, gamma, beta), beta[None, :] * u, rtol=0, atol=1e-15)
    _, u, gamma, beta = rnd(4, 37, 2)
    x = np.repeat(np.array([[3.5], [-2.0], [0.0], [1e3]]), 37, axis=1)
    np.testing.assert_allclose(L.ln_mul(x, u, gamma, beta), beta[None, :] * u, rtol=0, atol=1e-9)


def test_rows_are_normalised():
    x, _, _, _ = rnd(9, 300, 3)
    y = L.ln_mul(x * 7.0 + 2.0, np.ones_like(x), np.ones(300), np.zeros(300))
    np.testing.assert_allclose(y.mean(axis=1), 0.0, atol=1e-13)
    np.testing.assert_allclose((y * y).mean(axis=1), 1.0, rtol=1e-6)  # eps / var ~ 2e-7


def test_gamma_scales_beta_shifts_u_multiplies_last():
    x, u, gamma, beta = rnd(5, 40, 4)
    norm = L.ln_mul(x, np.ones_like(x), np.ones(40), np.zeros(40))
    np.testing.assert_allclose(L.ln_mul(x, u, gamma, beta), (norm * gamma + beta) * u, rtol=1e-13, atol=1e-14)
    # linear in u; beta is added before the product with u, not after
    np.testing.assert_allclose(L.ln_mul(x, 2 * u, gamma, beta), 2 * L.ln_mul(x, u, gamma, beta), rtol=1e-14)
    np.testing.assert_allclose(L.ln_mul(x, np.zeros_like(u), gamma, beta), 0.0, atol=0)


def test_shift_and_positive_scale_of_a_row_change_nothing():
    x, u, gamma, beta = rnd(5, 128, 5)
    a = L.ln_mul(x, u, gamma, beta, eps=0.0)
    b = L.ln_mul(4.0 * x - 11.0, u, gamma, beta, eps=0.0)
    np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-12)
    c = L.ln_mul(-x, u, gamma, np.zeros(128), eps=0.0)
    np.testing.assert_allclose(c, -L.ln_mul(x, u, gamma, np.zeros(128), eps=0.0), rtol=1e-12, atol=1e-12)


def test_reference_example_inputs():
    # examples/torch/test_torch_ln_mul.py:27-42: A, R = 4, 8, gamma = 1, beta = 0, checked there against
    # (x - mean) / sqrt(var(unbiased=False) + 1e-5) * u; the same with numpy's own mean / var
    g = np.random.default_rng(0)
    x, u = g.standard_normal((4, 8)).astype(np.float32), g.standard_normal((4, 8)).astype(np.float32)
    want = (x - np.mean(x, axis=1, keepdims=True)) / np.sqrt(np.var(x, axis=1, keepdims=True) + 1e-5) * u
    got = L.ln_mul(x, u, np.ones(8, np.float32), np.zeros(8, np.float32))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    # float32 evaluation as in the reference's golden stays within its tolerance of the float64 one
    got32 = L.ln_mul(x, u, np.ones(8, np.float32), np.zeros(8, np.float32), accumulate=np.float32)
    np.testing.assert_allclose(got32, got, rtol=1e-4, atol=1e-4)


def test_shape_errors():
    x, u, gamma, beta = rnd(3, 4, 6)
    with pytest.raises(ValueError):
        L.ln_mul(x, u[:2], gamma, beta)
    with pytest.raises(ValueError):
        L.ln_mul(x, u, gamma[:3], beta)
