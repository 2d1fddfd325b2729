"""ctypes loader for the scalar C restatement (``hstu_bruteforce.c``).  Test infrastructure only."""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libhstu_bruteforce.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``hstu_bruteforce.c`` with gcc (via the Makefile beside it)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return _SO


def _load():
    global _lib
    if _lib is None:
        build()
        lib = ctypes.CDLL(_SO)
        lib.hstu_bruteforce_forward.restype = ctypes.c_int
        lib.hstu_bruteforce_forward.argtypes = (
            [ctypes.c_void_p] * 9 + [ctypes.c_int64] * 8 + [ctypes.c_double, ctypes.c_int64, ctypes.c_double, ctypes.c_void_p]
        )
        lib.hstu_bruteforce_mask.restype = None
        lib.hstu_bruteforce_mask.argtypes = [ctypes.c_int64] * 5 + [ctypes.c_void_p]
        _lib = lib
    return _lib


def _f32(t: Optional[torch.Tensor]):
    if t is None:
        return None
    return np.ascontiguousarray(t.detach().to(torch.float32).cpu().numpy())


def _i64(t):
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().tolist()
    return np.ascontiguousarray(np.asarray(list(t), dtype=np.int64))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def forward(
    q,
    k,
    v,
    mask=None,
    attn_bias=None,
    mask_type=0,
    max_seq_len=0,
    max_seq_len_k=None,
    silu_scale=0.0,
    seq_offset=None,
    seq_offset_k=None,
    num_context=None,
    num_target=None,
    target_group_size=0,
    alpha=1.0,
) -> torch.Tensor:
    """Same argument meaning as ``hstu_oracle.hstu_jagged_forward``; returns float32 ``[T_q, N_q, D_v]``."""
    lib = _load()
    if max_seq_len_k is None:
        max_seq_len_k = max_seq_len
    qa, ka, va = _f32(q), _f32(k), _f32(v)
    ma, ba = _f32(mask), _f32(attn_bias)
    oq = _i64(seq_offset)
    ok = _i64(seq_offset_k) if seq_offset_k is not None else oq
    ctx, tgt = _i64(num_context), _i64(num_target)
    out = np.zeros((qa.shape[0], qa.shape[1], va.shape[2]), dtype=np.float32)
    rc = lib.hstu_bruteforce_forward(
        _ptr(qa), _ptr(ka), _ptr(va), _ptr(ma), _ptr(ba), _ptr(oq), _ptr(ok), _ptr(ctx), _ptr(tgt),
        len(oq), qa.shape[1], ka.shape[1], qa.shape[2], va.shape[2], int(max_seq_len), int(max_seq_len_k),
        int(mask_type), float(silu_scale), int(target_group_size or 0), float(1.0 if alpha is None else alpha),
        _ptr(out),
    )  # fmt: skip
    if rc != 0:
        raise ValueError(f"hstu_bruteforce_forward rejected its arguments (code {rc})")
    return torch.from_numpy(out)


def mask(s_q, s_k=None, num_context=0, num_target=0, target_group_size=0) -> np.ndarray:
    lib = _load()
    if s_k is None:
        s_k = s_q
    m = np.zeros((s_q, s_k), dtype=np.float32)
    lib.hstu_bruteforce_mask(s_q, s_k, int(num_context or 0), int(num_target or 0), int(target_group_size or 0), _ptr(m))
    return m
