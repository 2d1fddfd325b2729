"""CPU oracle for ``in_linear_silu`` (linear + SiLU + four-way split).  TEST INFRASTRUCTURE ONLY.

Nothing under ``oracle/`` is part of the shipped operator: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it, and only as the checker.

Restates the golden of the reference's test
(ascendc/activation/in_linear_silu/in_linear_silu_forward/test/pytest/test_in_linear_silu.py:36-49) and the formula of
its documentation (in_linear_silu_forward/docs/torch_in_linear_silu.md:17-21)::

    mixed = x @ weight^T + bias;  linear_output = mixed;  (user, value, query, key) = split(silu(mixed), split, -1)

with the rounding points of the reference's kernel (fp32 accumulation + fp32 bias, ONE rounding to the 16-bit type =
linear_output, SiLU in fp32 OF THAT ROUNDED VALUE, rounded to nearest even:
in_linear_silu_forward/op_kernel/block_epilogue_elemwise_split.h:160-183, tile_elemwise_silu.h:36-47) when
``round_to`` names a 16-bit type; with ``round_to=None`` everything stays in float64 (the exact value).

The backward restated: ``in_linear_silu_backward`` below follows the formula of the reference's backward golden
(in_linear_silu_backward/test/pytest/test_in_linear_silu_backward.py:120-164: d mixed = cat(grads) * silu'(linear_output),
d x = d mixed @ W, d W = d mixed^T @ x, d bias = column sums).

Pinned (tests/test_oracle_in_linear_silu.py), not by retyping the formula: against ``torch.addmm`` +
``torch.nn.functional.silu`` + ``torch.split`` (library routines, the reference golden's own calls); by one-hot inputs
that make every output column name its weight row (catches a transposed weight, a shifted split boundary, a swapped
output); by bias-only and identity-weight cases with closed forms; the backward against torch autograd of the forward.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch


def in_linear_silu(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], split: Sequence[int],
                   round_to: Optional[torch.dtype] = None) -> Tuple[torch.Tensor, ...]:  # fmt: skip
    """``x`` [m, k], ``weight`` [n, k], ``bias`` [n] or None, ``split`` four sizes adding up to n.  Returns
    (user, value, query, key, linear_output) in float64 (values already rounded to ``round_to`` if given)."""
    if x.dim() != 2 or weight.dim() != 2 or weight.shape[1] != x.shape[1] or len(split) != 4 or sum(split) != weight.shape[0]:
        raise ValueError("in_linear_silu oracle: x [m, k], weight [n, k], four split sizes adding up to n")
    mixed = x.double() @ weight.double().t()
    if bias is not None:
        mixed = mixed + bias.double()
    if round_to is not None:
        # the kernel accumulates in fp32; products of 16-bit values summed over k <= 8192 terms: the fp32 sum differs from
        # the exact one far below one 16-bit rounding step, so rounding the exact value is the statement of the result
        mixed = mixed.float().to(round_to).double()
    act = mixed / (1.0 + torch.exp(-mixed))
    if round_to is not None:
        act = act.float().to(round_to).double()
    bounds: List[int] = [0]
    for s in split:
        bounds.append(bounds[-1] + int(s))
    parts = tuple(act[:, bounds[i]:bounds[i + 1]] for i in range(4))
    return parts + (mixed,)


def silu_backward_stage(grads: Sequence[torch.Tensor], linear_output):
    """d mixed = cat(grads) * silu'(linear_output) in float64."""
    z = linear_output.double()
    sig = 1.0 / (1.0 + torch.exp(-z))
    return torch.cat([g.double() for g in grads], dim=1) * sig * (1.0 + z * (1.0 - sig))


def in_linear_silu_backward(x, weight, grads: Sequence[torch.Tensor], linear_output):
    """(d x, d weight, d bias) in float64."""
    d_mixed = silu_backward_stage(grads, linear_output)
    return d_mixed @ weight.double(), d_mixed.t() @ x.double(), d_mixed.sum(dim=0)
