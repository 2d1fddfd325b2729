"""Operator groups, named as in the reference (``ops_rec.ascendc.<group>.<op>``)."""

from . import activation  # noqa: F401
from . import attention  # noqa: F401

__all__ = ["activation", "attention"]
