"""Autograd formulas for ``hstu_jagged.equal`` / ``hstu_jagged.delta``.

The forward operators carry no autograd kernel of their own; this module binds
``hstu_jagged_backward`` as their formula with ``torch.library.register_autograd`` so that
``loss.backward()`` works in eager mode and under ``torch.compile``.  Behaviour follows the
reference wrapper (ascendc/attention/hstu_v1/torch_extension/hstu_v1_autograd.py:53-374):

* what is saved: q, k, v, mask, attn_bias, the offsets, num_context, num_target + the scalars;
* a mask that requires grad is rejected (the backward op produces no mask gradient);
* backward always calls the 16-argument (``delta``) form of ``hstu_jagged_backward``;
* gradients are returned for q, k, v and attn_bias only, padded / cut to the number of
  arguments the forward was actually called with;
* registration is idempotent and per-operator failures are recorded in
  ``_registration_errors`` instead of raised.
"""

import logging
import warnings

import torch

logger = logging.getLogger(__name__)

# schema defaults of the forward overloads, used to fill slots the caller did not pass
_EQUAL_DEFAULTS = (None, None, None, None, None, 0, 0, 0.0, None, None, None, 0, 1.0, False)
_DELTA_DEFAULTS = (None, None, None, None, None, 0, 0, 0, 0.0, None, None, None, None, 0, 1.0, False)


def _unpack(inputs, defaults):
    vals = list(inputs)[: len(defaults)]
    vals.extend(defaults[len(vals) :])
    return tuple(vals)


def _fit_grads(grads, ctx):
    n = len(ctx.needs_input_grad)
    grads = tuple(grads) + (None,) * max(0, n - len(grads))
    return grads[:n]


def _reject_mask_grad(mask, op_name):
    if mask is not None and mask.requires_grad:
        raise NotImplementedError(
            f"{op_name}: mask is a non-differentiable input (the backward op returns no mask gradient); "
            "do not pass a mask with requires_grad=True"
        )


def _backward_op():
    return torch.ops.ops_rec.hstu_jagged_backward


def _jagged_equal_setup_context(ctx, inputs, output=None):
    (q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale, seq_offset, num_context, num_target,
     target_group_size, alpha, _det) = _unpack(inputs, _EQUAL_DEFAULTS)  # fmt: skip
    _reject_mask_grad(mask, "hstu_jagged.equal")
    ctx.save_for_backward(q, k, v, mask, attn_bias, seq_offset, num_context, num_target)
    ctx.mask_type = mask_type
    ctx.max_seq_len = max_seq_len
    ctx.silu_scale = silu_scale
    ctx.target_group_size = target_group_size
    ctx.alpha = alpha


def _jagged_equal_backward(ctx, grad):
    q, k, v, mask, attn_bias, seq_offset, num_context, num_target = ctx.saved_tensors
    dq, dk, dv, dbias = _backward_op()(
        grad, q, k, v, mask, attn_bias, ctx.mask_type, ctx.max_seq_len, ctx.max_seq_len, ctx.silu_scale,
        seq_offset, seq_offset, num_context, num_target, ctx.target_group_size, ctx.alpha,
    )  # fmt: skip
    return _fit_grads((dq, dk, dv, None, dbias if attn_bias is not None else None), ctx)


def _jagged_delta_setup_context(ctx, inputs, output=None):
    (q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale, seq_offset, seq_offset_k,
     num_context, num_target, target_group_size, alpha, _det) = _unpack(inputs, _DELTA_DEFAULTS)  # fmt: skip
    _reject_mask_grad(mask, "hstu_jagged.delta")
    ctx.save_for_backward(q, k, v, mask, attn_bias, seq_offset, seq_offset_k, num_context, num_target)
    ctx.mask_type = mask_type
    ctx.max_seq_len = max_seq_len
    ctx.max_seq_len_k = max_seq_len_k
    ctx.silu_scale = silu_scale
    ctx.target_group_size = target_group_size
    ctx.alpha = alpha


def _jagged_delta_backward(ctx, grad):
    q, k, v, mask, attn_bias, seq_offset, seq_offset_k, num_context, num_target = ctx.saved_tensors
    dq, dk, dv, dbias = _backward_op()(
        grad, q, k, v, mask, attn_bias, ctx.mask_type, ctx.max_seq_len, ctx.max_seq_len_k, ctx.silu_scale,
        seq_offset, seq_offset_k, num_context, num_target, ctx.target_group_size, ctx.alpha,
    )  # fmt: skip
    return _fit_grads((dq, dk, dv, None, dbias if attn_bias is not None else None), ctx)


# hstu_dense: (q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale)
# (torch_extension/hstu_v1_autograd.py:90-135 of the reference)
_DENSE_DEFAULTS = (None, None, None, None, None, 0, 0, 0.0)


def _dense_setup_context(ctx, inputs, output=None):
    q, k, v, mask, attn_bias, mask_type, max_seq_len, silu_scale = _unpack(inputs, _DENSE_DEFAULTS)
    _reject_mask_grad(mask, "hstu_dense")
    ctx.save_for_backward(q, k, v, mask, attn_bias)
    ctx.mask_type = mask_type
    ctx.max_seq_len = max_seq_len
    ctx.silu_scale = silu_scale


def _dense_backward(ctx, grad):
    q, k, v, mask, attn_bias = ctx.saved_tensors
    dq, dk, dv, dbias = torch.ops.ops_rec.hstu_dense_backward(
        grad, q, k, v, mask, attn_bias, ctx.mask_type, ctx.max_seq_len, ctx.silu_scale
    )
    # without attn_bias the op returns a 256-aligned placeholder: dropped
    return _fit_grads((dq, dk, dv, None, dbias if attn_bias is not None else None, None, None, None), ctx)


_registered = False
_registration_errors = {}


def _register_one(name, op_overload, backward, setup_context):
    try:
        torch.library.register_autograd(op_overload, backward, setup_context=setup_context)
    except Exception as exc:  # noqa: BLE001 -- API differences across torch versions are recorded, not raised
        _registration_errors[name] = f"{type(exc).__name__}: {exc}"
        logger.warning("ops_rec.autograd.hstu_v1: register '%s' failed: %s: %s", name, type(exc).__name__, exc)
        return False
    logger.info("ops_rec.autograd.hstu_v1: registered autograd for '%s'", name)
    return True


def register_autograd():
    """Entry point called by ``ops_rec.autograd`` at import; safe to call more than once."""
    global _registered
    if _registered:
        return
    _registered = True
    ok = True
    ok &= _register_one("hstu_jagged.equal", torch.ops.ops_rec.hstu_jagged.equal, _jagged_equal_backward,
                        _jagged_equal_setup_context)  # fmt: skip
    ok &= _register_one("hstu_jagged.delta", torch.ops.ops_rec.hstu_jagged.delta, _jagged_delta_backward,
                        _jagged_delta_setup_context)  # fmt: skip
    ok &= _register_one("hstu_dense", torch.ops.ops_rec.hstu_dense.default, _dense_backward, _dense_setup_context)
    if not ok:
        warnings.warn(
            "ops_rec.autograd.hstu_v1: some autograd registrations failed, see "
            f"ops_rec.autograd.hstu_v1_autograd._registration_errors: {_registration_errors}",
            stacklevel=2,
        )
