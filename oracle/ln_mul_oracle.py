"""CPU oracle for ``ln_mul`` (LayerNorm(x) * u).  TEST INFRASTRUCTURE ONLY.

Nothing under ``oracle/`` is part of the shipped operator: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it, and only as the checker.

Restates the golden of the reference's test (ascendc/activation/ln_mul/test/pytest/test_ln_mul.py:36-49) and the
formula of its documentation (ascendc/activation/ln_mul/docs/torch_ln_mul.md:17-20)::

    mean = mean(x, axis=1);  var = mean((x - mean)^2, axis=1)      (population variance, ddof = 0)
    out  = ((x - mean) / sqrt(var + eps) * gamma + beta) * u        eps = 1e-5

The reference's golden evaluates this in float32 numpy; here it is evaluated in float64 (``accumulate`` below) and
rounded once to the type of ``x``, so that the checker's own rounding stays far below the tolerance of the test
(rtol = atol = 1e-4 in fp32, test_ln_mul.py:64-66).

Pinned (tests/test_oracle_ln_mul.py), not by retyping the formula: against ``torch.nn.functional.layer_norm`` times
``u`` (a library routine); against closed forms (a row of one column or of equal values gives ``beta * u``; with
gamma = 1, beta = 0, u = 1 every row has mean 0 and, for var >> eps, second moment 1; the output is linear in u;
an affine map a*x + c of a row with a > 0 leaves the normalised row unchanged up to the eps term); against the inputs
of the reference's own example (examples/torch/test_torch_ln_mul.py:27-42: gamma = 1, beta = 0) evaluated by
``numpy.var`` / ``numpy.mean``.
"""

from __future__ import annotations

import numpy as np

EPSILON = 1e-5  # ascendc/activation/ln_mul/op_host/ln_mul.cpp:75


def ln_mul(x: np.ndarray, u: np.ndarray, gamma: np.ndarray, beta: np.ndarray, eps: float = EPSILON,
           accumulate=np.float64) -> np.ndarray:  # fmt: skip
    """``x``, ``u``: [A, R]; ``gamma``, ``beta``: [R].  Returns [A, R] in ``accumulate`` precision (the caller rounds
    to the type under test)."""
    if x.ndim != 2 or u.shape != x.shape or gamma.shape != (x.shape[1],) or beta.shape != (x.shape[1],):
        raise ValueError("ln_mul oracle: x, u must be [A, R] and gamma, beta [R]")
    xf, uf = x.astype(accumulate), u.astype(accumulate)
    n = xf.shape[1]
    mean = xf.sum(axis=1, keepdims=True) / n
    centred = xf - mean
    var = (centred * centred).sum(axis=1, keepdims=True) / n
    rstd = 1.0 / np.sqrt(var + accumulate(eps))
    return (centred * rstd * gamma.astype(accumulate) + beta.astype(accumulate)) * uf
