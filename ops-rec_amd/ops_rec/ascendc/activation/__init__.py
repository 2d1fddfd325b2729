"""``ops_rec.ascendc.activation`` -- attribute access is forwarded to ``torch.ops.ops_rec``.

Same surface as the reference module (ops_rec/ascendc/activation/__init__.py:30-55): both
``ops_rec.ascendc.activation.ln_mul(...)`` and ``from ops_rec.ascendc.activation import ln_mul`` work, and an
unknown name raises ``AttributeError`` listing what exists.
"""

import torch

_NS = torch.ops.ops_rec
_OPS = ("ln_mul", "distance_in_linear_silu", "in_linear_silu_backward")

__all__ = [name for name in _OPS if hasattr(_NS, name)]
for _name in __all__:
    globals()[_name] = getattr(_NS, _name)
# the name the reference's documentation uses for the differentiable forward (docs/zh/ops_rec_api.md:42); the
# autograd formula is attached to distance_in_linear_silu itself
if hasattr(_NS, "distance_in_linear_silu"):
    in_linear_silu = _NS.distance_in_linear_silu
    __all__.append("in_linear_silu")


def __getattr__(name: str):
    if not name.startswith("_") and hasattr(_NS, name):
        return getattr(_NS, name)
    raise AttributeError(
        f"module '{__name__}' has no attribute '{name}'. Operator '{name}' is not built for gfx950. "
        f"Available ops: {sorted(__all__)}"
    )


def __dir__():
    return sorted(set(globals().keys()) | set(__all__))
