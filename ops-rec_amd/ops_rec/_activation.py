"""Operators around HSTU attention in an HSTU layer (``ops_rec.ascendc.activation``).

``ln_mul(x, u, gamma, beta)``: ``LayerNorm(x) * u`` over the rows of a 2-D matrix, schema and checks of the
reference's adapter (ascendc/activation/ln_mul/torch_extension/ln_mul_plugin.cpp:30-51, 68-71), epsilon 1e-5 as
fixed by its host tiling (ascendc/activation/ln_mul/op_host/ln_mul.cpp:75).  The reference takes fp32 only; here
x / u may also be bf16 / fp16 (what the attention kernels write) with gamma / beta in fp32 or in that type.  Like
the reference's registration, the operator carries no autograd formula.
"""

from __future__ import annotations

import ctypes

import torch

from . import _native
from ._ops import _DTYPE_CODE, _check, _lib_cuda, _lib_def, _lib_meta

LN_MUL_EPSILON = 1e-5

_lib_def.define("ln_mul(Tensor x, Tensor u, Tensor gamma, Tensor beta) -> Tensor")


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
    lib = _native.load()
    with torch.cuda.device(x_c.device):
        rc = lib.ln_mul_fwd(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        raise RuntimeError(f"ln_mul failed ({rc}): {_native.last_error()}")
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
