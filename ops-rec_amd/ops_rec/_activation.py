"""Operators around HSTU attention in an HSTU layer (``ops_rec.ascendc.activation``).

``ln_mul(x, u, gamma, beta)``: ``LayerNorm(x) * u`` over the rows of a 2-D matrix, schema and checks of the
reference's adapter (ascendc/activation/ln_mul/torch_extension/ln_mul_plugin.cpp:30-51, 68-71), epsilon 1e-5 as
fixed by its host tiling (ascendc/activation/ln_mul/op_host/ln_mul.cpp:75).  The reference takes fp32 only; here
x / u may also be bf16 / fp16 (what the attention kernels write) with gamma / beta in fp32 or in that type.  Like
the reference's registration, the operator carries no autograd formula.

``distance_in_linear_silu(x, weight, bias, attr_dict)`` (``in_linear_silu`` in the reference's documentation):
``mixed = x @ weight^T + bias``, ``linear_output = mixed``, ``(user, value, query, key) = split(silu(mixed))``; schema
and checks of ascendc/activation/in_linear_silu/torch_extension/in_linear_silu_plugin.cpp:36-110.  Its backward
operator ``in_linear_silu_backward`` (schema of in_linear_silu_backward_plugin.cpp:155-160) runs its element-wise stage
and the bias gradient as one HIP kernel and the two products as library matrix products; the autograd formula that joins the two is the reference's (torch_extension/_autograd.py:33-86).
"""

from __future__ import annotations

import ctypes
from typing import List, Optional

import torch

from . import _native
from ._ops import _DTYPE_CODE, _check, _lib_cuda, _lib_def, _lib_meta

LN_MUL_EPSILON = 1e-5

_lib_def.define("ln_mul(Tensor x, Tensor u, Tensor gamma, Tensor beta) -> Tensor")


# Validated calls, by everything but the addresses: (shapes, dtypes, devices, contiguity) -> the parameter block with its
# scalar fields filled.  A layer repeats one description per step with new tensors; on a hit the checks and the filling of
# the block are skipped and only the addresses are set (the checks cost more host time than the kernels of a small layer
# take: [20292, 512] bf16 ln_mul 18.7 us per call for a 10.4 us kernel before, in_linear_silu 30 us for small shapes).
_CALL_CACHE: dict = {}
_CALL_CACHE_MAX = 256


def _tensor_key(t: Optional[torch.Tensor]):
    return None if t is None else (tuple(t.shape), t.dtype, t.device, t.is_contiguous())


def _remember(key, params) -> None:
    if len(_CALL_CACHE) >= _CALL_CACHE_MAX:
        _CALL_CACHE.clear()
    _CALL_CACHE[key] = bytes(params)


def _launch(fn, params, device: torch.device, what: str) -> None:
    """``fn(params, stream)`` of the C ABI on the current stream of ``device``."""
    if device.index is None or device.index == torch.cuda.current_device():
        rc = fn(ctypes.byref(params), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    else:
        with torch.cuda.device(device):
            rc = fn(ctypes.byref(params), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        raise RuntimeError(f"{what} failed ({rc}): {_native.last_error()}")


def _non_empty(t: torch.Tensor, name: str) -> None:
    # check_tensor_non_empty (ascendc/common/torch_plugin/common_utils.h:34-39)
    _check(t is not None, f"{name} tensor must be defined")
    _check(t.numel() > 0, f"{name} tensor must be non-empty")
    _check(t.dim() > 0, f"{name} tensor must have non-zero dimensions")


def _ln_mul_shapes(x, u, gamma, beta) -> None:
    _check(x.dim() == 2, "The x should be 2D")
    _check(u.dim() == 2, "The u should be 2D")
    _check(gamma.dim() == 1, "The gamma should be 1D")
    _check(beta.dim() == 1, "The beta should be 1D")
    _check(x.shape == u.shape, "x and u must have identical shape")


def ln_mul(x, u, gamma, beta):
    key = ("ln_mul", _tensor_key(x), _tensor_key(u), _tensor_key(gamma), _tensor_key(beta))
    cached = _CALL_CACHE.get(key)
    if cached is not None and key[1][3] and key[2][3] and key[3][3] and key[4][3]:  # (contiguous tensors: used as they are)
        out = torch.empty_like(x)
        p = _native.LnMulParams.from_buffer_copy(cached)
        p.x, p.u, p.gamma, p.beta, p.out = x.data_ptr(), u.data_ptr(), gamma.data_ptr(), beta.data_ptr(), out.data_ptr()
        _launch(_native.load().ln_mul_fwd, p, x.device, "ln_mul")
        return out
    for t, name in ((x, "x"), (u, "u"), (gamma, "gamma"), (beta, "beta")):
        _non_empty(t, name)
    for t, name in ((x, "x"), (u, "u"), (gamma, "gamma"), (beta, "beta")):
        _check(t.is_cuda and t.device == x.device, f"{name} tensor must be on the GPU of x, but got {t.device}")
    _ln_mul_shapes(x, u, gamma, beta)
    _check(x.dtype in (torch.float32, torch.bfloat16, torch.float16), f"unsupported dtype {x.dtype}")
    _check(u.dtype == x.dtype, "x and u must have the same dtype")
    _check(gamma.dtype == beta.dtype and gamma.dtype in (torch.float32, x.dtype),
           "gamma and beta must both be float32 or both of the dtype of x")  # fmt: skip
    # the kernel indexes gamma / beta by column without a bound of their own
    _check(gamma.numel() == x.size(1) and beta.numel() == x.size(1), "gamma and beta must have x.size(1) elements")
    x_c, u_c, g_c, b_c = x.contiguous(), u.contiguous(), gamma.contiguous(), beta.contiguous()
    out = torch.empty_like(x_c)
    p = _native.new_ln_mul_params()
    p.x, p.u, p.gamma, p.beta, p.out = x_c.data_ptr(), u_c.data_ptr(), g_c.data_ptr(), b_c.data_ptr(), out.data_ptr()
    p.rows, p.cols = x_c.size(0), x_c.size(1)
    p.dtype, p.affine_dtype = _DTYPE_CODE[x_c.dtype], _DTYPE_CODE[g_c.dtype]
    p.epsilon = LN_MUL_EPSILON
    _launch(_native.load().ln_mul_fwd, p, x_c.device, "ln_mul")
    _remember(key, p)  # (the library took the description)
    return out


def ln_mul_meta(x, u, gamma, beta):
    # ascendc/activation/ln_mul/torch_extension/ln_mul_plugin.cpp:81-89
    _check(x.dim() == 2, "x must be 2D")
    _check(u.dim() == 2, "u must be 2D")
    _check(gamma.dim() == 1, "gamma must be 1D")
    _check(beta.dim() == 1, "beta must be 1D")
    _check(x.shape == u.shape, "x and u must share the same shape")
    return torch.empty_like(x)


_lib_cuda.impl("ln_mul", ln_mul)
_lib_meta.impl("ln_mul", ln_mul_meta)


# ---------------------------------------------------------------- in_linear_silu ----

_MIN_DIM, _MAX_DIM = 16, 512 * 16

_lib_def.define("distance_in_linear_silu(Tensor x, Tensor weight, Tensor bias, int[] attr_dict) -> "
                "(Tensor, Tensor, Tensor, Tensor, Tensor)")  # fmt: skip
_lib_def.define("in_linear_silu_backward(Tensor x, Tensor weight, Tensor? bias, Tensor user_grad, Tensor value_grad, "
                "Tensor query_grad, Tensor key_grad, Tensor linear_output, int[] attr_dict) -> "
                "(Tensor, Tensor, Tensor, Tensor)")  # fmt: skip


def _in_linear_silu_shapes(x, weight, bias, split: List[int]) -> None:
    # IsValidShape (in_linear_silu_plugin.cpp:36-66)
    _non_empty(x, "x")
    _non_empty(weight, "weight")
    _check(x.dim() == 2, "x must be 2D")
    _check(weight.dim() == 2, "weight must be 2D")
    _check(len(split) == 4, "splitList must have 4 elements.")
    for s in split:
        _check(_MIN_DIM <= s <= _MAX_DIM and s % _MIN_DIM == 0, "uvqk dim must in range[16, 8192] and multiples of 16.")
    k, n = x.size(1), weight.size(0)
    _check(_MIN_DIM <= k <= _MAX_DIM and k % _MIN_DIM == 0, "x dim[1] must in range[16, 8192] and multiples of 16.")
    _check(4 * _MIN_DIM <= n <= 4 * _MAX_DIM and n % _MIN_DIM == 0,
           "weight dim[0] must in range[64, 32768] and multiples of 16.")  # fmt: skip
    _check(sum(split) == n, "weight_dim[0] must equal to sum(splitList).")
    _check(weight.size(1) == k, "weight dim[1] must equal to x dim[1].")
    _check(n % (4 * k) == 0, "weight dim[0] must be a multiple of 4 x dim[1]")
    if bias is not None:
        _non_empty(bias, "bias")
        _check(bias.dim() == 1, "bias must be 1D")
        _check(bias.size(0) == n, "bias dim[0] must equal to weight dim[0].")


def distance_in_linear_silu(x, weight, bias, attr_dict):
    split = [int(s) for s in attr_dict]
    key = ("in_linear_silu", _tensor_key(x), _tensor_key(weight), _tensor_key(bias), tuple(split))
    cached = _CALL_CACHE.get(key)
    if cached is not None and key[1][3] and key[2][3] and (bias is None or key[3][3]):
        m, n = x.size(0), weight.size(0)
        outs = [torch.empty((m, s_), dtype=x.dtype, device=x.device) for s_ in split]
        linear_output = torch.empty((m, n), dtype=x.dtype, device=x.device)
        p = _native.InLinearSiluParams.from_buffer_copy(cached)
        p.x, p.weight, p.bias = x.data_ptr(), weight.data_ptr(), (bias.data_ptr() if bias is not None else None)
        p.user, p.value, p.query, p.key = (t.data_ptr() for t in outs)
        p.linear_output = linear_output.data_ptr()
        _launch(_native.load().in_linear_silu_fwd, p, x.device, "in_linear_silu")
        return outs[0], outs[1], outs[2], outs[3], linear_output
    _in_linear_silu_shapes(x, weight, bias, split)
    _check(x.dtype in (torch.bfloat16, torch.float16), f"x must be float16 or bfloat16, got {x.dtype}")
    _check(weight.dtype == x.dtype, "weight must have the dtype of x")
    _check(x.is_cuda and weight.device == x.device, "x and weight must be on the same GPU")
    m, k, n = x.size(0), x.size(1), weight.size(0)
    x_c, w_c = x.contiguous(), weight.contiguous()
    b_c = None
    if bias is not None:
        _check(bias.device == x.device, "bias must be on the GPU of x")
        _check(bias.dtype == torch.float32, "bias must be float32")
        b_c = bias.contiguous()
    outs = [torch.empty((m, s), dtype=x.dtype, device=x.device) for s in split]
    linear_output = torch.empty((m, n), dtype=x.dtype, device=x.device)
    p = _native.new_in_linear_silu_params()
    p.x, p.weight, p.bias = x_c.data_ptr(), w_c.data_ptr(), (b_c.data_ptr() if b_c is not None else None)
    p.user, p.value, p.query, p.key = (t.data_ptr() for t in outs)
    p.linear_output = linear_output.data_ptr()
    p.m, p.n, p.k = m, n, k
    for i, s in enumerate(split):
        p.split[i] = s
    p.dtype = _DTYPE_CODE[x.dtype]
    _launch(_native.load().in_linear_silu_fwd, p, x.device, "in_linear_silu")
    _remember(key, p)  # (the library took the description)
    return outs[0], outs[1], outs[2], outs[3], linear_output


def distance_in_linear_silu_meta(x, weight, bias, attr_dict):
    # in_linear_silu_plugin.cpp:90-103
    m, n = x.size(0), weight.size(0)
    outs = [x.new_empty((m, s)) for s in attr_dict]
    return outs[0], outs[1], outs[2], outs[3], x.new_empty((m, n))


def silu_backward_stage(linear_output, grads, split, want_bias_grad=True):
    """``d_mixed`` [m, n] in the type of ``linear_output`` and the fp32 column sums (or None), through
    ``in_linear_silu_bwd_dmixed`` of the C ABI."""
    lin = linear_output.contiguous()
    gs = [g.contiguous() for g in grads]
    m, n = lin.shape
    d_mixed = torch.empty_like(lin)
    sums = torch.empty(n, dtype=torch.float32, device=lin.device) if want_bias_grad else None
    p = _native.new_in_linear_silu_bwd_params()
    p.linear_output = lin.data_ptr()
    p.user_grad, p.value_grad, p.query_grad, p.key_grad = (g.data_ptr() for g in gs)
    p.d_mixed = d_mixed.data_ptr()
    p.bias_grad = sums.data_ptr() if sums is not None else None
    p.m, p.n = m, n
    for i, s_ in enumerate(split):
        p.split[i] = int(s_)
    p.dtype = _DTYPE_CODE[lin.dtype]
    lib = _native.load()
    need = ctypes.c_uint64(0)
    rc = lib.in_linear_silu_bwd_dmixed_workspace_size(ctypes.byref(p), ctypes.byref(need))
    if rc != 0:
        raise RuntimeError(f"in_linear_silu_backward failed ({rc}): {_native.last_error()}")
    ws = torch.empty(need.value, dtype=torch.uint8, device=lin.device) if need.value else None
    with torch.cuda.device(lin.device):
        rc = lib.in_linear_silu_bwd_dmixed(ctypes.byref(p), ctypes.c_void_p(ws.data_ptr() if ws is not None else None),
                                           need.value, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))  # fmt: skip
    if rc != 0:
        raise RuntimeError(f"in_linear_silu_backward failed ({rc}): {_native.last_error()}")
    return d_mixed, sums


def in_linear_silu_backward(x, weight, bias: Optional[torch.Tensor], user_grad, value_grad, query_grad, key_grad,
                            linear_output, attr_dict):  # fmt: skip
    """Gradients of x, weight and bias (in_linear_silu_backward_plugin.cpp:40-153): with z = linear_output,
    d mixed = cat(grads) * sigmoid(z) * (1 + z * (1 - sigmoid(z))); d x = d mixed @ weight; d weight = d mixed^T @ x;
    d bias = column sums of d mixed.  The element-wise stage and the column sums are one HIP kernel
    (``in_linear_silu_bwd_dmixed`` of the C ABI); the two products are library matrix products."""
    split = [int(s) for s in attr_dict]
    _in_linear_silu_shapes(x, weight, bias, split)
    grads = (user_grad, value_grad, query_grad, key_grad)
    for g, name in zip(grads, ("user_grad", "value_grad", "query_grad", "key_grad")):
        _non_empty(g, name)
        _check(g.dim() == 2, f"{name} must be 2D")
    _non_empty(linear_output, "linear_output")
    _check(linear_output.dim() == 2, "linear_output must be 2D")
    _check(all(g.size(1) == s for g, s in zip(grads, split)),
           "user_grad, value_grad, query_grad, key_grad dim[1] must be equal to split_list.")  # fmt: skip
    _check(all(g.size(0) == x.size(0) for g in grads) and linear_output.size(0) == x.size(0),
           "user_grad, value_grad, query_grad, key_grad linear_output dim[0] must equal to x dim[0].")  # fmt: skip
    _check(linear_output.size(1) == weight.size(0), "linear_output dim[1] must equal to weight dim[0].")
    _check(x.dtype in (torch.bfloat16, torch.float16), f"x must be float16 or bfloat16, got {x.dtype}")
    _check(all(t.dtype == x.dtype for t in (weight, linear_output, *grads)),
           "weight, linear_output and the gradients must have the dtype of x")  # fmt: skip
    _check(all(t.is_cuda and t.device == x.device for t in (weight, linear_output, *grads)),
           "all tensors must be on the GPU of x")  # fmt: skip
    d_mixed, bias_sums = silu_backward_stage(linear_output, grads, split, want_bias_grad=bias is not None)
    x_grad = d_mixed @ weight
    weight_grad = d_mixed.t() @ x
    bias_grad = bias_sums.to(bias.dtype) if bias is not None else None
    return x_grad, weight_grad, bias_grad, None


def in_linear_silu_backward_meta(x, weight, bias, user_grad, value_grad, query_grad, key_grad, linear_output, attr_dict):
    return torch.empty_like(x), torch.empty_like(weight), (torch.empty_like(bias) if bias is not None else None), None


_lib_cuda.impl("distance_in_linear_silu", distance_in_linear_silu)
_lib_meta.impl("distance_in_linear_silu", distance_in_linear_silu_meta)
_lib_cuda.impl("in_linear_silu_backward", in_linear_silu_backward)
_lib_meta.impl("in_linear_silu_backward", in_linear_silu_backward_meta)


def _ils_setup_context(ctx, inputs, output):
    # torch_extension/_autograd.py:33-52
    x, weight, bias, attr_dict = inputs
    ctx.has_bias = bias is not None
    if ctx.has_bias:
        ctx.save_for_backward(x, weight, bias, output[-1])
    else:
        ctx.save_for_backward(x, weight, output[-1])
    ctx.attr_dict = list(attr_dict)


def _ils_backward(ctx, user_grad, value_grad, query_grad, key_grad, linear_output_grad):
    # torch_extension/_autograd.py:55-86: the gradient of linear_output is ignored, as there
    if ctx.has_bias:
        x, weight, bias, linear_output = ctx.saved_tensors
    else:
        (x, weight, linear_output), bias = ctx.saved_tensors, None
    x_grad, weight_grad, bias_grad, _ = torch.ops.ops_rec.in_linear_silu_backward(
        x, weight, bias, user_grad, value_grad, query_grad, key_grad, linear_output, ctx.attr_dict)  # fmt: skip
    return x_grad, weight_grad, bias_grad, None


_ils_autograd_registered = False


def register_in_linear_silu_autograd() -> None:
    """Idempotent, like the reference's ``register_autograd`` (torch_extension/_autograd.py:89-101)."""
    global _ils_autograd_registered
    if _ils_autograd_registered:
        return
    torch.library.register_autograd("ops_rec::distance_in_linear_silu", _ils_backward, setup_context=_ils_setup_context)
    _ils_autograd_registered = True


register_in_linear_silu_autograd()
