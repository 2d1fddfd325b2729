"""ln_mul without a GPU: registration and Meta inference, the adapter's argument checks, the C ABI's status codes
and its choice of kernel variant (validation only: nothing is launched)."""

import ctypes
import re

import pytest
import torch

import ops_rec
from ops_rec import _native


def test_op_is_registered_and_reachable_as_in_the_reference():
    op = torch.ops.ops_rec.ln_mul
    assert str(op.default._schema) == "ops_rec::ln_mul(Tensor x, Tensor u, Tensor gamma, Tensor beta) -> Tensor"
    assert ops_rec.ascendc.activation.ln_mul is op
    from ops_rec.ascendc.activation import ln_mul  # noqa: F401

    with pytest.raises(AttributeError, match="not built for gfx950"):
        ops_rec.ascendc.activation.no_such_op


def test_meta_inference_and_checks():
    x = torch.empty(5, 48, device="meta", dtype=torch.bfloat16)
    g = torch.empty(48, device="meta")
    y = torch.ops.ops_rec.ln_mul(x, x, g, g)
    assert y.shape == (5, 48) and y.dtype == torch.bfloat16 and y.device.type == "meta"
    with pytest.raises(RuntimeError, match="x must be 2D"):
        torch.ops.ops_rec.ln_mul(x[0], x, g, g)
    with pytest.raises(RuntimeError, match="share the same shape"):
        torch.ops.ops_rec.ln_mul(x, x[:3], g, g)
    with pytest.raises(RuntimeError, match="gamma must be 1D"):
        torch.ops.ops_rec.ln_mul(x, x, g[None], g)


def test_no_cpu_implementation():
    x = torch.zeros(2, 4)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.ops_rec.ln_mul(x, x, torch.ones(4), torch.zeros(4))


def _valid():
    p = _native.new_ln_mul_params()
    p.x, p.u, p.gamma, p.beta, p.out = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000  # never dereferenced
    p.rows, p.cols = 100, 512
    p.dtype = p.affine_dtype = _native.DT_FP32
    p.epsilon = 1e-5
    return p


def test_c_abi_validation_codes():
    lib = _native.load()
    assert lib.ln_mul_fwd(None, None) == 161001
    assert lib.ln_mul_fwd_kernel_name(None) is None
    for field, value, code, text in [
        ("struct_size", 8, 161002, "struct_size"),
        ("x", None, 161001, "must all be given"),
        ("out", None, 161001, "must all be given"),
        ("beta", None, 161001, "must all be given"),
        ("rows", 0, 161002, "non-empty"),
        ("cols", 0, 161002, "non-empty"),
        ("rows", 1 << 31, 161002, "rows"),
        ("dtype", _native.DT_FP8_E4M3, 161002, "fp32, bf16, fp16"),
        ("affine_dtype", _native.DT_BF16, 161002, "gamma / beta"),
        ("epsilon", -1.0, 161002, "epsilon"),
        ("epsilon", float("nan"), 161002, "epsilon"),
    ]:
        p = _valid()
        setattr(p, field, value)
        # an invalid description is refused before any device call
        got = lib.ln_mul_fwd(ctypes.byref(p), None)
        assert got == code, (field, value, got, _native.last_error())
        assert re.search(text, _native.last_error()), (field, _native.last_error())
        assert lib.ln_mul_fwd_kernel_name(ctypes.byref(p)) is None


def test_kernel_variant_selection():
    lib = _native.load()

    def name(**kw):
        p = _valid()
        for k, v in kw.items():
            setattr(p, k, v)
        return lib.ln_mul_fwd_kernel_name(ctypes.byref(p)).decode()

    bf16 = dict(dtype=_native.DT_BF16)
    # a row goes to the variant with the smallest capacity (lanes x 16-byte chunks per lane) that holds it
    assert name(cols=4) == "ln_mul_f32_g8_v1"
    assert name(cols=32) == "ln_mul_f32_g8_v1"
    assert name(cols=64) == "ln_mul_f32_g16_v1"
    assert name(cols=96) == "ln_mul_f32_g8_v3"
    assert name(cols=256) == "ln_mul_f32_g16_v4"
    assert name(cols=512) == "ln_mul_f32_g64_v2"
    assert name(cols=768) == "ln_mul_f32_g64_v3"
    assert name(cols=512, **bf16) == "ln_mul_bf16_g16_v4"
    assert name(cols=512, dtype=_native.DT_FP16, affine_dtype=_native.DT_FP16) == "ln_mul_f16_g16_v4"
    assert name(cols=12288) == "ln_mul_f32_g256_v12"
    assert name(cols=2048) == "ln_mul_f32_g64_v8"
    assert name(cols=4096) == "ln_mul_f32_g256_v4"
    assert name(cols=16384) == "ln_mul_f32_g256_v16"
    assert name(cols=32768, **bf16) == "ln_mul_bf16_g256_v16"
    # rows that are not a whole number of aligned 16-byte chunks, or too long for the registers of a workgroup
    assert name(cols=1) == "ln_mul_f32_g64_any"
    assert name(cols=1022) == "ln_mul_f32_g64_any"
    assert name(cols=516, **bf16) == "ln_mul_bf16_g64_any"
    assert name(cols=16388) == "ln_mul_f32_g256_any"
    assert name(cols=512, x=0x1004) == "ln_mul_f32_g64_any"
    assert name(cols=4096, gamma=0x3008) == "ln_mul_f32_g256_any"
