"""ctypes binding of the C ABI declared in ``include/hstu_mi355.h``.

The library is loaded from ``ops_rec/_lib``; if it is missing the import fails loudly on
first use -- there is no CPU or eager fallback for the operator.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

from . import _build

HSTU_OK = 0
DT_BF16, DT_FP16, DT_FP32, DT_FP8_E4M3 = 0, 1, 2, 3
IDX_I32, IDX_I64 = 0, 1

EXPORTED_SYMBOLS = (
    "hstu_jagged_fwd_workspace_size",
    "hstu_jagged_fwd",
    "hstu_jagged_fwd_noalloc",
    "hstu_jagged_fwd_noalloc_max_workspace",
    "hstu_last_error",
    "hstu_reload_switches",
    "hstu_version",
    "hstu_jagged_fwd_kernel_name",
    "hstu_jagged_bwd_workspace_size",
    "hstu_jagged_bwd",
    "hstu_paged_fwd_workspace_size",
    "hstu_paged_fwd",
    "ln_mul_fwd",
    "ln_mul_fwd_kernel_name",
    "in_linear_silu_fwd",
    "in_linear_silu_fwd_kernel_name",
    "in_linear_silu_bwd_dmixed_workspace_size",
    "in_linear_silu_bwd_dmixed",
)


class FwdParams(ctypes.Structure):
    """Mirror of ``hstu_jagged_fwd_params``."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32),
        ("index_dtype", ctypes.c_int32),
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("mask", ctypes.c_void_p),
        ("attn_bias", ctypes.c_void_p),
        ("seq_offset_q", ctypes.c_void_p),
        ("seq_offset_k", ctypes.c_void_p),
        ("num_context", ctypes.c_void_p),
        ("num_target", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("total_q", ctypes.c_int64),
        ("total_k", ctypes.c_int64),
        ("num_heads_q", ctypes.c_int64),
        ("num_heads_k", ctypes.c_int64),
        ("head_dim_qk", ctypes.c_int64),
        ("head_dim_v", ctypes.c_int64),
        ("n_offsets", ctypes.c_int64),
        ("mask_type", ctypes.c_int64),
        ("max_seq_len_q", ctypes.c_int64),
        ("max_seq_len_k", ctypes.c_int64),
        ("target_group_size", ctypes.c_int64),
        ("silu_scale", ctypes.c_double),
        ("alpha", ctypes.c_double),
        ("deterministic", ctypes.c_int32),
        ("fp8_scaled_p", ctypes.c_int32),
        ("q_descale", ctypes.c_void_p),
        ("k_descale", ctypes.c_void_p),
        ("v_descale", ctypes.c_void_p),
    ]


class BwdParams(ctypes.Structure):
    """Mirror of ``hstu_jagged_bwd_params``."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("reserved0", ctypes.c_uint32),
        ("fwd", FwdParams),
        ("grad", ctypes.c_void_p),
        ("grad_q", ctypes.c_void_p),
        ("grad_k", ctypes.c_void_p),
        ("grad_v", ctypes.c_void_p),
        ("grad_attn_bias", ctypes.c_void_p),
    ]


class PagedParams(ctypes.Structure):
    """Mirror of ``hstu_paged_fwd_params``."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("reserved0", ctypes.c_uint32),
        ("fwd", FwdParams),
        ("kv_cache", ctypes.c_void_p),
        ("page_offsets", ctypes.c_void_p),
        ("page_ids", ctypes.c_void_p),
        ("last_page_len", ctypes.c_void_p),
        ("seq_offset_t", ctypes.c_void_p),
        ("num_pages", ctypes.c_int64),
        ("page_size", ctypes.c_int64),
        ("n_page_ids", ctypes.c_int64),
    ]


class LnMulParams(ctypes.Structure):
    """Mirror of ``ln_mul_params`` (include/ops_rec_activation_mi355.h)."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("reserved0", ctypes.c_uint32),
        ("x", ctypes.c_void_p),
        ("u", ctypes.c_void_p),
        ("gamma", ctypes.c_void_p),
        ("beta", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("rows", ctypes.c_int64),
        ("cols", ctypes.c_int64),
        ("dtype", ctypes.c_int32),
        ("affine_dtype", ctypes.c_int32),
        ("epsilon", ctypes.c_float),
        ("reserved1", ctypes.c_uint32),
    ]


class InLinearSiluParams(ctypes.Structure):
    """Mirror of ``in_linear_silu_params`` (include/ops_rec_activation_mi355.h)."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("reserved0", ctypes.c_uint32),
        ("x", ctypes.c_void_p),
        ("weight", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("user", ctypes.c_void_p),
        ("value", ctypes.c_void_p),
        ("query", ctypes.c_void_p),
        ("key", ctypes.c_void_p),
        ("linear_output", ctypes.c_void_p),
        ("m", ctypes.c_int64),
        ("n", ctypes.c_int64),
        ("k", ctypes.c_int64),
        ("split", ctypes.c_int64 * 4),
        ("dtype", ctypes.c_int32),
        ("reserved1", ctypes.c_uint32),
    ]


class InLinearSiluBwdParams(ctypes.Structure):
    """Mirror of ``in_linear_silu_bwd_params`` (include/ops_rec_activation_mi355.h)."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("reserved0", ctypes.c_uint32),
        ("linear_output", ctypes.c_void_p),
        ("user_grad", ctypes.c_void_p),
        ("value_grad", ctypes.c_void_p),
        ("query_grad", ctypes.c_void_p),
        ("key_grad", ctypes.c_void_p),
        ("d_mixed", ctypes.c_void_p),
        ("bias_grad", ctypes.c_void_p),
        ("m", ctypes.c_int64),
        ("n", ctypes.c_int64),
        ("split", ctypes.c_int64 * 4),
        ("dtype", ctypes.c_int32),
        ("reserved1", ctypes.c_uint32),
    ]


_lib: Optional[ctypes.CDLL] = None


def library_path() -> str:
    return _build.LIB_PATH


def reload_switches() -> None:
    """Has the library read its ``HSTU_MI355_*`` switches from the environment again (it reads them once per process
    otherwise) and drops the call descriptions the Python side has cached, whose workspace sizes depend on them."""
    load().hstu_reload_switches()
    from . import _ops

    _ops._PLAN_CACHE.clear()


def load() -> ctypes.CDLL:
    """Load the HIP library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"HIP library not found at {path}. Build it first (python -c 'import __graft_entry__ as g; g.build()' "
            "or ops_rec._build.build()); the operator has no fallback path."
        )
    lib = ctypes.CDLL(path)
    lib.hstu_jagged_fwd_workspace_size.restype = ctypes.c_int
    lib.hstu_jagged_fwd_workspace_size.argtypes = [ctypes.POINTER(FwdParams), ctypes.POINTER(ctypes.c_uint64)]
    lib.hstu_jagged_fwd.restype = ctypes.c_int
    lib.hstu_jagged_fwd.argtypes = [ctypes.POINTER(FwdParams), ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
    lib.hstu_jagged_fwd_noalloc.restype = ctypes.c_int
    lib.hstu_jagged_fwd_noalloc.argtypes = [ctypes.POINTER(FwdParams), ctypes.c_void_p]
    lib.hstu_jagged_fwd_noalloc_max_workspace.restype = ctypes.c_uint64
    lib.hstu_jagged_fwd_noalloc_max_workspace.argtypes = []
    lib.hstu_last_error.restype = ctypes.c_char_p
    lib.hstu_last_error.argtypes = []
    lib.hstu_reload_switches.restype = None
    lib.hstu_reload_switches.argtypes = []
    lib.hstu_version.restype = ctypes.c_int
    lib.hstu_version.argtypes = []
    lib.hstu_jagged_fwd_kernel_name.restype = ctypes.c_char_p
    lib.hstu_jagged_fwd_kernel_name.argtypes = [ctypes.POINTER(FwdParams)]
    lib.hstu_jagged_bwd_workspace_size.restype = ctypes.c_int
    lib.hstu_jagged_bwd_workspace_size.argtypes = [ctypes.POINTER(BwdParams), ctypes.POINTER(ctypes.c_uint64)]
    lib.hstu_jagged_bwd.restype = ctypes.c_int
    lib.hstu_jagged_bwd.argtypes = [ctypes.POINTER(BwdParams), ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
    lib.hstu_paged_fwd_workspace_size.restype = ctypes.c_int
    lib.hstu_paged_fwd_workspace_size.argtypes = [ctypes.POINTER(PagedParams), ctypes.POINTER(ctypes.c_uint64)]
    lib.hstu_paged_fwd.restype = ctypes.c_int
    lib.hstu_paged_fwd.argtypes = [ctypes.POINTER(PagedParams), ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
    lib.ln_mul_fwd.restype = ctypes.c_int
    lib.ln_mul_fwd.argtypes = [ctypes.POINTER(LnMulParams), ctypes.c_void_p]
    lib.ln_mul_fwd_kernel_name.restype = ctypes.c_char_p
    lib.ln_mul_fwd_kernel_name.argtypes = [ctypes.POINTER(LnMulParams)]
    lib.in_linear_silu_fwd.restype = ctypes.c_int
    lib.in_linear_silu_fwd.argtypes = [ctypes.POINTER(InLinearSiluParams), ctypes.c_void_p]
    lib.in_linear_silu_fwd_kernel_name.restype = ctypes.c_char_p
    lib.in_linear_silu_fwd_kernel_name.argtypes = [ctypes.POINTER(InLinearSiluParams)]
    lib.in_linear_silu_bwd_dmixed_workspace_size.restype = ctypes.c_int
    lib.in_linear_silu_bwd_dmixed_workspace_size.argtypes = [ctypes.POINTER(InLinearSiluBwdParams),
                                                             ctypes.POINTER(ctypes.c_uint64)]  # fmt: skip
    lib.in_linear_silu_bwd_dmixed.restype = ctypes.c_int
    lib.in_linear_silu_bwd_dmixed.argtypes = [ctypes.POINTER(InLinearSiluBwdParams), ctypes.c_void_p, ctypes.c_uint64,
                                              ctypes.c_void_p]  # fmt: skip
    _lib = lib
    return lib


def last_error() -> str:
    return load().hstu_last_error().decode("utf-8", "replace")


def new_params() -> FwdParams:
    p = FwdParams()
    p.struct_size = ctypes.sizeof(FwdParams)
    return p


def new_in_linear_silu_params() -> InLinearSiluParams:
    p = InLinearSiluParams()
    p.struct_size = ctypes.sizeof(InLinearSiluParams)
    return p


def new_in_linear_silu_bwd_params() -> InLinearSiluBwdParams:
    p = InLinearSiluBwdParams()
    p.struct_size = ctypes.sizeof(InLinearSiluBwdParams)
    return p


def new_ln_mul_params() -> LnMulParams:
    p = LnMulParams()
    p.struct_size = ctypes.sizeof(LnMulParams)
    return p


def new_bwd_params() -> BwdParams:
    p = BwdParams()
    p.struct_size = ctypes.sizeof(BwdParams)
    p.fwd.struct_size = ctypes.sizeof(FwdParams)
    return p
