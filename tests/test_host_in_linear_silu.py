"""in_linear_silu without a GPU: registration and Meta inference, the C ABI's status codes (the adapter's limits,
in_linear_silu_plugin.cpp:36-66) and its choice of kernel variant (validation only: nothing is launched)."""

import ctypes
import re

import pytest
import torch

import ops_rec
from ops_rec import _native


def test_ops_are_registered_and_reachable_as_in_the_reference():
    fwd = torch.ops.ops_rec.distance_in_linear_silu
    assert str(fwd.default._schema) == (
        "ops_rec::distance_in_linear_silu(Tensor x, Tensor weight, Tensor bias, int[] attr_dict) -> "
        "(Tensor, Tensor, Tensor, Tensor, Tensor)"
    )
    bwd = torch.ops.ops_rec.in_linear_silu_backward
    assert "Tensor? bias" in str(bwd.default._schema) and str(bwd.default._schema).endswith(
        "int[] attr_dict) -> (Tensor, Tensor, Tensor, Tensor)"
    )
    act = ops_rec.ascendc.activation
    assert act.distance_in_linear_silu is fwd and act.in_linear_silu is fwd and act.in_linear_silu_backward is bwd
    from ops_rec.ascendc.activation import in_linear_silu  # noqa: F401


def test_meta_inference():
    x = torch.empty(7, 32, device="meta", dtype=torch.float16)
    w = torch.empty(256, 32, device="meta", dtype=torch.float16)
    b = torch.empty(256, device="meta")
    outs = torch.ops.ops_rec.distance_in_linear_silu(x, w, b, [48, 48, 80, 80])
    assert [tuple(t.shape) for t in outs] == [(7, 48), (7, 48), (7, 80), (7, 80), (7, 256)]
    assert all(t.dtype == torch.float16 and t.device.type == "meta" for t in outs)
    grads = [torch.empty(7, s, device="meta", dtype=torch.float16) for s in (48, 48, 80, 80)]
    dx, dw, db, none = torch.ops.ops_rec.in_linear_silu_backward(x, w, b, *grads, outs[4], [48, 48, 80, 80])
    assert dx.shape == x.shape and dw.shape == w.shape and db.shape == b.shape and none is None


def test_autograd_registration_is_idempotent():
    from ops_rec import _activation

    _activation.register_in_linear_silu_autograd()
    _activation.register_in_linear_silu_autograd()


def _valid():
    p = _native.new_in_linear_silu_params()
    p.x, p.weight, p.bias = 0x1000, 0x2000, 0x3000  # never dereferenced
    p.user, p.value, p.query, p.key, p.linear_output = 0x4000, 0x5000, 0x6000, 0x7000, 0x8000
    p.m, p.n, p.k = 100, 256, 64
    for i in range(4):
        p.split[i] = 64
    p.dtype = _native.DT_BF16
    return p


def test_c_abi_validation_codes():
    lib = _native.load()
    assert lib.in_linear_silu_fwd(None, None) == 161001
    p = _valid()
    assert lib.in_linear_silu_fwd_kernel_name(ctypes.byref(p)).decode() == "in_linear_silu_bf16_stages2_tile128"
    p.bias = None  # no bias is allowed
    assert lib.in_linear_silu_fwd_kernel_name(ctypes.byref(p)).decode() == "in_linear_silu_bf16_stages2_tile128"

    def split(*v):
        def apply(p):
            for i, s in enumerate(v):
                p.split[i] = s
        return apply

    def field(name, value):
        return lambda p: setattr(p, name, value)

    for change, code, text in [
        (field("struct_size", 8), 161002, "struct_size"),
        (field("x", None), 161001, "must all be given"),
        (field("key", None), 161001, "must all be given"),
        (field("linear_output", None), 161001, "must all be given"),
        (field("dtype", _native.DT_FP32), 161002, "bf16 or fp16"),
        (field("m", 0), 161002, "non-empty"),
        (split(64, 64, 64, 48), 161002, "sum\\(splitList\\)"),
        (split(64, 72, 56, 64), 161002, "uvqk dim"),
        (split(0, 128, 64, 64), 161002, "uvqk dim"),
        (field("k", 24), 161002, "x dim\\[1\\]"),
        (field("k", 8), 161002, "x dim\\[1\\]"),
        (field("k", 8208), 161002, "x dim\\[1\\]"),
        (field("n", 48), 161002, "weight dim\\[0\\]"),
        (field("k", 128), 161002, "multiple of 4 x dim"),  # n = 256 is not a multiple of 4 * 128
        (field("weight", 0x2008), 161002, "multiple of 16 bytes"),
        (field("bias", 0x3004), 161002, "multiple of 16 bytes"),
    ]:
        p = _valid()
        change(p)
        got = lib.in_linear_silu_fwd(ctypes.byref(p), None)  # refused before any device call
        assert got == code, (text, got, _native.last_error())
        assert re.search(text, _native.last_error()), _native.last_error()
        assert lib.in_linear_silu_fwd_kernel_name(ctypes.byref(p)) is None


def test_kernel_variant_selection():
    lib = _native.load()

    def name(k, n, dtype=_native.DT_BF16):
        p = _valid()
        p.k, p.n, p.dtype = k, n, dtype
        for i in range(4):
            p.split[i] = n // 4
        return lib.in_linear_silu_fwd_kernel_name(ctypes.byref(p)).decode()

    # a ring of two k steps and four workgroups per CU for short k, three stages in the middle, 128 x 256 tiles from k = 1024 on (measured)
    assert name(16, 64) == "in_linear_silu_bf16_stages2_tile128"
    assert name(64, 9216) == "in_linear_silu_bf16_stages2_tile128"
    assert name(128, 1024) == "in_linear_silu_bf16_stages3_tile128"
    assert name(512, 2048) == "in_linear_silu_bf16_stages3_tile128"
    assert name(768, 3072) == "in_linear_silu_bf16_stages2_tile128"
    assert name(1024, 4096) == "in_linear_silu_bf16_stages2_tile256"
    assert name(8192, 32768, _native.DT_FP16) == "in_linear_silu_f16_stages2_tile256"


def test_no_cpu_implementation():
    x = torch.zeros(4, 16, dtype=torch.float16)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.ops_rec.distance_in_linear_silu(x, torch.zeros(64, 16, dtype=torch.float16), torch.zeros(64), [16] * 4)


def test_backward_stage_c_abi_validation_codes():
    lib = _native.load()
    ws = ctypes.c_uint64(99)

    def valid():
        p = _native.new_in_linear_silu_bwd_params()
        p.linear_output, p.user_grad, p.value_grad, p.query_grad, p.key_grad = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000
        p.d_mixed, p.bias_grad = 0x6000, 0x7000
        p.m, p.n = 130, 256
        for i in range(4):
            p.split[i] = 64
        p.dtype = _native.DT_FP16
        return p

    p = valid()
    assert lib.in_linear_silu_bwd_dmixed_workspace_size(ctypes.byref(p), ctypes.byref(ws)) == 0
    assert ws.value == 3 * 256 * 4  # ceil(130 / 64) partial rows of n floats
    p.bias_grad = None
    assert lib.in_linear_silu_bwd_dmixed_workspace_size(ctypes.byref(p), ctypes.byref(ws)) == 0 and ws.value == 0
    assert lib.in_linear_silu_bwd_dmixed_workspace_size(ctypes.byref(p), None) == 161001
    assert lib.in_linear_silu_bwd_dmixed(None, None, 0, None) == 161001
    # a missing or short workspace is refused before any device call
    p = valid()
    assert lib.in_linear_silu_bwd_dmixed(ctypes.byref(p), None, 0, None) == 161004
    assert lib.in_linear_silu_bwd_dmixed(ctypes.byref(p), ctypes.c_void_p(0x9000), 100, None) == 161004
    for name, value, code, text in [
        ("struct_size", 4, 161002, "struct_size"),
        ("linear_output", None, 161001, "must all be given"),
        ("key_grad", None, 161001, "must all be given"),
        ("d_mixed", None, 161001, "must all be given"),
        ("dtype", _native.DT_FP32, 161002, "bf16 or fp16"),
        ("m", 0, 161002, "non-empty"),
        ("n", 272, 161002, "sum\\(split_list\\)"),
        ("n", 48, 161002, "weight dim\\[0\\]"),
        ("user_grad", 0x2004, 161002, "multiple of 16 bytes"),
    ]:
        p = valid()
        setattr(p, name, value)
        got = lib.in_linear_silu_bwd_dmixed_workspace_size(ctypes.byref(p), ctypes.byref(ws))
        assert got == code, (name, got, _native.last_error())
        assert re.search(text, _native.last_error()), _native.last_error()
