"""ops_rec for MI355X: the HSTU jagged attention forward path of ops-rec, rebuilt for gfx950.

Importing the package registers ``torch.ops.ops_rec.hstu_jagged`` (overloads ``.equal`` /
``.delta``) and ``torch.ops.ops_rec.hstu_jagged_backward`` and attaches the autograd formula,
the same sequence as the reference's ``import ops_rec`` (ops_rec/__init__.py:208-236) minus
the SoC detection: there is one target, gfx950.

    import ops_rec
    y = ops_rec.ascendc.attention.hstu_jagged(q, k, v, None, None, 0, S, 1.0 / S, seq_offset)
"""

from __future__ import annotations

import logging

from . import _ops  # noqa: F401  (defines the attention operators)
from . import _activation  # noqa: F401  (defines ln_mul)
from . import ascendc  # noqa: F401
from . import autograd  # noqa: F401  (registers the autograd formulas)
from ._ops import hstu_jagged_fp8  # noqa: F401  (extension: fp8 inputs with per-head scales)

logger = logging.getLogger(__name__)

__version__ = "0.1.0"
__all__ = ["ascendc", "autograd", "hstu_jagged_fp8", "__version__"]
