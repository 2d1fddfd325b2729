"""CPU-only checks of the host side: schemas and overload resolution, argument checks, Meta shape
inference, the proxy module, the autograd wrapper's plumbing, and the C ABI (symbols, struct,
status codes) -- no kernel is launched here."""

import ctypes
import os
import re

import pytest
import torch

import ops_rec
from ops_rec import _native, _ops
from ops_rec.autograd import hstu_v1_autograd as ag
import helpers

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _meta_inputs(total=10, heads=4, dim=32, dim_v=None, dtype=torch.bfloat16):
    q = torch.empty(total, heads, dim, device="meta", dtype=dtype)
    v = torch.empty(total, heads, dim_v or dim, device="meta", dtype=dtype)
    offs = torch.empty(3, device="meta", dtype=torch.int32)
    return q, q, v, offs


# ---------------------------------------------------------------- schemas / dispatch ----


def test_ops_are_registered_with_both_overloads():
    pkt = torch.ops.ops_rec.hstu_jagged
    assert set(pkt.overloads()) == {"equal", "delta"}
    assert set(torch.ops.ops_rec.hstu_jagged_backward.overloads()) == {"equal", "delta"}
    eq = pkt.equal._schema
    assert [a.name for a in eq.arguments] == [
        "q", "k", "v", "mask", "attn_bias", "mask_type", "max_seq_len", "silu_scale", "seq_offset", "num_context",
        "num_target", "target_group_size", "alpha", "deterministic",
    ]  # fmt: skip
    de = pkt.delta._schema
    assert [a.name for a in de.arguments][6:11] == ["max_seq_len", "max_seq_len_k", "silu_scale", "seq_offset",
                                                    "seq_offset_k"]  # fmt: skip


def test_packet_resolves_equal_and_delta_by_argument_types():
    q, k, v, offs = _meta_inputs()
    op = ops_rec.ascendc.attention.hstu_jagged
    # 9 positional (equal), keyword form (equal), 11 positional (delta): the reference's examples
    assert op(q, k, v, None, None, 0, 6, 1.0 / 6, offs).shape == (10, 4, 32)
    assert op(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=6, silu_scale=0.0, seq_offset=offs).shape == (10, 4, 32)
    assert op(q, k, v, None, None, 0, 6, 8, 1.0 / 6, offs, offs).shape == (10, 4, 32)
    assert op.equal(q, k, v, None, None, 0, 6, 0, offs).shape == (10, 4, 32)  # int accepted for silu_scale


def test_meta_shape_and_dtype_inference():
    q, k, v, offs = _meta_inputs(dim=64, dim_v=32)
    out = torch.ops.ops_rec.hstu_jagged.equal(q, k, v, None, None, 0, 6, 0.0, offs)
    assert out.shape == (10, 4, 32) and out.dtype == torch.bfloat16 and out.device.type == "meta"
    q8 = torch.empty(10, 4, 64, device="meta", dtype=torch.float8_e4m3fn)
    out8 = torch.ops.ops_rec.hstu_jagged.equal(q8, q8, q8, None, None, 0, 6, 0.0, offs)
    assert out8.dtype == torch.float16  # fp8 inputs produce half outputs, as in the reference adapter
    with pytest.raises(RuntimeError, match="3D"):
        torch.ops.ops_rec.hstu_jagged.equal(q[0], k, v, None, None, 0, 6, 0.0, offs)
    dq, dk, dv, db = torch.ops.ops_rec.hstu_jagged_backward.equal(out, q, k, v, None, None, 0, 6, 0.0, offs)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape and db is None


def test_no_cpu_implementation():
    q = torch.zeros(4, 2, 32, dtype=torch.bfloat16)
    offs = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.ops_rec.hstu_jagged.equal(q, q, q, None, None, 0, 4, 0.0, offs)


def test_proxy_module_surface():
    att = ops_rec.ascendc.attention
    assert att.hstu_jagged is torch.ops.ops_rec.hstu_jagged
    from ops_rec.ascendc.attention import hstu_jagged, hstu_jagged_backward  # noqa: F401

    assert "hstu_jagged" in dir(att)
    with pytest.raises(AttributeError, match="Available ops"):
        att.no_such_operator


# ---------------------------------------------------------------- argument checks ----


def _cpu_args(**over):
    q = torch.zeros(10, 4, 32, dtype=torch.bfloat16)
    offs = torch.tensor([0, 4, 10], dtype=torch.int32)
    a = dict(q=q, k=q, v=q, mask=None, attn_bias=None, mask_type=0, max_seq_len_q=6, max_seq_len_k=6, silu_scale=0.0,
             seq_offset=offs, seq_offset_k=offs, num_context=None, num_target=None, target_group_size=0, alpha=1.0)  # fmt: skip
    a.update(over)
    return a


@pytest.mark.parametrize(
    "over,msg",
    [
        (dict(q=torch.zeros(10, 32, dtype=torch.bfloat16)), "3D in jagged layout"),
        (dict(seq_offset=torch.tensor([0], dtype=torch.int32)), "at least two element"),
        (dict(seq_offset_k=torch.tensor([0], dtype=torch.int32)), "at least two element"),
        (dict(max_seq_len_q=0), r"expect in \[1, 20480\]"),
        (dict(max_seq_len_q=20481), r"expect in \[1, 20480\]"),
        (dict(max_seq_len_k=0), r"expect in \[1, 20480\]"),
        (dict(mask_type=4), r"maskType expect in \[0, 3\]"),
        (dict(mask_type=-1), r"maskType expect in \[0, 3\]"),
        (dict(mask_type=1), "not support triu"),
        (dict(mask_type=3), "must have valide mask tensor"),
        (dict(v=torch.zeros(9, 4, 32, dtype=torch.bfloat16)), "K, V seqLens mismatch"),
        (dict(v=torch.zeros(10, 2, 32, dtype=torch.bfloat16)), "K, V headNum mismatch"),
        (dict(k=torch.zeros(10, 4, 16, dtype=torch.bfloat16)), "headDIM"),
        (dict(num_context=torch.zeros(3, dtype=torch.int32)), "num_context"),
        (dict(num_target=torch.zeros(1, dtype=torch.int32)), "num_target"),
        (dict(attn_bias=torch.zeros(2, 4, 6, 5, dtype=torch.bfloat16)), "attn_bias must have shape"),
        (dict(attn_bias=torch.zeros(2, 4, 6, 6, dtype=torch.float16)), "attn_bias must have the dtype"),
    ],
)
def test_adapter_rejects_bad_arguments(over, msg):
    # same trigger conditions as the reference adapter's TORCH_CHECKs; raised before any device work
    with pytest.raises(RuntimeError, match=msg):
        _ops.prepare_forward(**_cpu_args(**over))


def test_tensors_on_another_device_are_rejected_before_any_pointer_is_taken():
    # a host seq_offset next to device q / k / v is a common slip; its data_ptr() must never reach a kernel
    dev = torch.device("cuda:0")  # (constructing the device object needs no GPU)
    host = torch.tensor([0, 4, 10], dtype=torch.int32)
    with pytest.raises(RuntimeError, match=r"seq_offset must be on the device of q \(cuda:0\), but it is on cpu"):
        _ops._check_devices(dev, (("k", None), ("seq_offset", host)))
    _ops._check_devices(torch.device("cpu"), (("seq_offset", host), ("mask", None)))  # same device: accepted
    # through the adapter: q, k, v on the "meta" device stand in for device tensors, the offsets are host tensors
    qm = torch.zeros(10, 4, 32, dtype=torch.bfloat16, device="meta")
    for name in ("seq_offset", "num_target", "attn_bias"):
        over = dict(q=qm, k=qm, v=qm)
        if name == "num_target":
            over.update(seq_offset=host.to("meta"), seq_offset_k=host.to("meta"), num_target=torch.zeros(2, dtype=torch.int32))
        elif name == "attn_bias":
            over.update(seq_offset=host.to("meta"), seq_offset_k=host.to("meta"), attn_bias=torch.zeros(2, 4, 6, 6, dtype=torch.bfloat16))
        with pytest.raises(RuntimeError, match=f"{name} must be on the device of q"):
            _ops.prepare_forward(**_cpu_args(**over))
    # the backward and the paged adapter refuse host q outright, before they look at anything else
    q = torch.zeros(10, 4, 32, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="q must be a GPU tensor"):
        _ops._backward_hip(q, q, q, q, None, None, 0, 6, 6, 0.0, host, host, None, None, 0, 1.0)
    with pytest.raises(RuntimeError, match="q must be a GPU tensor"):
        _ops.prepare_forward(**_cpu_args()).launch()


def test_paged_adapter_checks_the_row_counts_of_k_and_v():
    # the new key / value rows are addressed by query row index: k and v must have q's row count
    # (checked before anything touches the device; the tensors here are on the "meta" device)
    m = dict(device="meta")
    q = torch.zeros(10, 4, 32, dtype=torch.bfloat16, **m)
    short = torch.zeros(6, 4, 32, dtype=torch.bfloat16, **m)
    offs = torch.zeros(3, dtype=torch.int32, **m)
    cache = torch.zeros(4, 2, 32, 4, 32, dtype=torch.bfloat16, **m)
    ids = torch.zeros(4, dtype=torch.int32, **m)
    kw = dict(kv_cache=cache, max_seq_len=6, max_seq_len_k=70, seq_offset=offs, seq_offset_k=offs, seq_offset_t=offs,
              page_offsets=offs, page_ids=ids, last_page_len=torch.zeros(2, dtype=torch.int32, **m),
              num_target=torch.zeros(2, dtype=torch.int32, **m), target_group_size=1)  # fmt: skip
    with pytest.raises(RuntimeError, match=r"one row per row of q \(10\), but have 6 and 6"):
        _ops.hstu_paged(q, short, short, **kw)
    with pytest.raises(RuntimeError, match="q must be a GPU tensor"):
        _ops.hstu_paged(q, q, q, **kw)


def test_empty_input_returns_empty_output_without_touching_the_library():
    q = torch.zeros(0, 4, 32, dtype=torch.bfloat16)
    p = _ops.prepare_forward(**_cpu_args(q=q, k=q, v=q, seq_offset=torch.tensor([0, 0], dtype=torch.int32),
                                         seq_offset_k=torch.tensor([0, 0], dtype=torch.int32)))  # fmt: skip
    assert p.launch().shape == (0, 4, 32)


# ---------------------------------------------------------------- autograd wrapper ----


def test_autograd_formulas_are_registered_once():
    assert ag._registered and ag._registration_errors == {}
    ag.register_autograd()  # idempotent
    assert "hstu_v1_autograd" in ops_rec.autograd.__all__


def test_unpack_fills_schema_defaults():
    vals = ag._unpack(("q", "k", "v"), ag._EQUAL_DEFAULTS)
    assert len(vals) == 14 and vals[5] == 0 and vals[7] == 0.0 and vals[12] == 1.0 and vals[13] is False
    vals = ag._unpack(tuple(range(16)), ag._DELTA_DEFAULTS)
    assert vals == tuple(range(16))


def test_fit_grads_pads_and_cuts():
    class Ctx:
        needs_input_grad = (True,) * 9

    assert ag._fit_grads((1, 2, 3, None, 5), Ctx) == (1, 2, 3, None, 5, None, None, None, None)
    Ctx.needs_input_grad = (True,) * 3
    assert ag._fit_grads((1, 2, 3, None, 5), Ctx) == (1, 2, 3)


def test_mask_requiring_grad_is_rejected():
    m = torch.zeros(2, 2, requires_grad=True)
    with pytest.raises(NotImplementedError, match="non-differentiable"):
        ag._reject_mask_grad(m, "hstu_jagged.equal")
    ag._reject_mask_grad(None, "x")
    ag._reject_mask_grad(torch.zeros(2), "x")


# ---------------------------------------------------------------- C ABI ----


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(_ROOT, "include", "hstu_mi355.h")).read()
    header += open(os.path.join(_ROOT, "include", "ops_rec_activation_mi355.h")).read()
    declared = set(re.findall(r"HSTU_API\s+[\w\s\*]+?\b((?:hstu|ln_mul|in_linear_silu)_\w+)\s*\(", header))
    assert declared == set(_native.EXPORTED_SYMBOLS)
    lib = _native.load()
    for sym in declared:
        assert getattr(lib, sym) is not None
    assert lib.hstu_version() >= 1


def test_struct_mirror_matches_library():
    # the library checks struct_size itself: a correct mirror gets past that check
    lib = _native.load()
    p = _native.new_params()
    ws = ctypes.c_uint64(123)
    rc = lib.hstu_jagged_fwd_workspace_size(ctypes.byref(p), ctypes.byref(ws))
    assert rc == 161002 and "at least two element" in _native.last_error()
    p.struct_size = 8
    rc = lib.hstu_jagged_fwd_workspace_size(ctypes.byref(p), ctypes.byref(ws))
    assert rc == 161002 and "struct_size" in _native.last_error()


def _valid_params():
    p = _native.new_params()
    p.dtype = p.out_dtype = _native.DT_BF16
    p.index_dtype = _native.IDX_I32
    fake = 0x1000  # never dereferenced: only validation runs
    p.q = p.k = p.v = p.out = p.seq_offset_q = p.seq_offset_k = fake
    p.total_q = p.total_k = 10
    p.num_heads_q = p.num_heads_k = 4
    p.head_dim_qk = p.head_dim_v = 128
    p.n_offsets = 3
    p.max_seq_len_q = p.max_seq_len_k = 6
    p.silu_scale, p.alpha = 0.0, 1.0
    return p


def test_c_abi_validation_codes():
    lib = _native.load()
    ws = ctypes.c_uint64(7)

    def rc(p):
        return lib.hstu_jagged_fwd_workspace_size(ctypes.byref(p), ctypes.byref(ws))

    p = _valid_params()
    assert rc(p) == 0 and ws.value == 0
    assert lib.hstu_jagged_fwd_kernel_name(ctypes.byref(p)).decode().startswith("hstu_fwd_bf16_d128")
    assert lib.hstu_jagged_fwd_workspace_size(None, ctypes.byref(ws)) == 161001
    assert lib.hstu_jagged_fwd_workspace_size(ctypes.byref(p), None) == 161001
    for field, value, code, text in [
        ("q", None, 161001, "must not be NULL"),
        ("seq_offset_q", None, 161001, "must not be NULL"),
        ("mask_type", 1, 161002, "triu"),
        ("mask_type", 3, 161002, "valide mask"),
        ("mask_type", 9, 161002, r"\[0, 3\]"),
        ("max_seq_len_q", 0, 161002, "20480"),
        ("max_seq_len_k", 30000, 161002, "20480"),
        ("n_offsets", 2050, 161002, "batchSize"),
        ("num_heads_q", 17, 161002, "head num"),
        ("num_heads_k", 3, 161002, "divisible"),
        ("head_dim_v", 24, 161002, "step 16"),
        ("head_dim_qk", 513, 161002, "512"),
        ("index_dtype", 5, 161002, "index_dtype"),
        ("dtype", 9, 161002, "unknown dtype"),
    ]:
        p = _valid_params()
        setattr(p, field, value)
        got = rc(p)
        assert got == code, (field, value, got, _native.last_error())
        assert re.search(text, _native.last_error()), (field, _native.last_error())
    # launching with an invalid description is refused before any device call
    p = _valid_params()
    p.mask_type = 1
    assert lib.hstu_jagged_fwd(ctypes.byref(p), None, 0, None) == 161002


def test_kernel_variant_selection():
    lib = _native.load()

    def name(**kw):
        p = _valid_params()
        for k, v in kw.items():
            setattr(p, k, v)
        n = lib.hstu_jagged_fwd_kernel_name(ctypes.byref(p))
        return n.decode() if n else None

    long = dict(max_seq_len_q=100, max_seq_len_k=100)
    assert "_d32_" in name(head_dim_qk=16, head_dim_v=16, **long)
    assert "_d64_" in name(head_dim_qk=64, head_dim_v=48, **long)
    assert "_d128_" in name(head_dim_qk=64, head_dim_v=128, **long)
    assert "_d256_" in name(head_dim_qk=256, head_dim_v=256, **long)
    # sequences of at most 32 / 64 rows and keys: the kernel for tiny sequences, head-dim slots 64, 128, 256
    assert name(head_dim_qk=16, head_dim_v=16) == "hstu_fwd_bf16_d64_tiny32"
    assert name(head_dim_qk=64, head_dim_v=128, max_seq_len_q=33) == "hstu_fwd_bf16_d128_tiny64"
    assert name(head_dim_qk=256, head_dim_v=256, max_seq_len_k=64) == "hstu_fwd_bf16_d256_tiny64"
    assert "_tiny" not in name(max_seq_len_k=65) and "_tiny" not in name(q=0x1008)
    assert "rabtrue" in name(attn_bias=0x2000)
    assert "masktrue" in name(mask=0x2000, mask_type=3)
    assert "f16" in name(dtype=_native.DT_FP16, out_dtype=_native.DT_FP16)
    # what the reference accepts beyond the tuned kernels (head dims up to 512, any q/k head dim) goes to the kernel
    # written for coverage
    assert name(head_dim_qk=12, head_dim_v=16) == "hstu_fwd_generic_bf16"
    assert name(head_dim_qk=1, head_dim_v=512, dtype=_native.DT_FP16, out_dtype=_native.DT_FP16) == "hstu_fwd_generic_f16"
    assert name(head_dim_qk=512, head_dim_v=512, dtype=_native.DT_FP32, out_dtype=_native.DT_FP32) == "hstu_fwd_generic_f32"
    # 16-bit inputs with a head dim above 256 and a q/k head dim that is a multiple of 8: the matrix-pipe kernel for 512
    assert name(head_dim_qk=264, head_dim_v=64, attn_bias=0x2000) == "hstu_fwd_wide_bf16_rab1_mask0"
    assert name(head_dim_qk=64, head_dim_v=512, dtype=_native.DT_FP16, out_dtype=_native.DT_FP16, mask=0x2000,
                mask_type=3) == "hstu_fwd_wide_f16_rab0_mask1"  # fmt: skip
    assert name(head_dim_qk=260, head_dim_v=272) == "hstu_fwd_generic_bf16"


def test_fp8_variant_selection_and_limits():
    lib = _native.load()

    def name(**kw):
        p = _valid_params()
        p.dtype = _native.DT_FP8_E4M3
        p.out_dtype = _native.DT_FP16
        for k, v in kw.items():
            setattr(p, k, v)
        n = lib.hstu_jagged_fwd_kernel_name(ctypes.byref(p))
        return n.decode() if n else None

    assert name() == "hstu_fwd_f8e4m3_f16_d128"
    assert name(out_dtype=_native.DT_BF16) == "hstu_fwd_f8e4m3_bf16_d128"
    assert name(head_dim_qk=32, head_dim_v=48).endswith("_d64")  # fp8 rows are padded to at least 64 bytes
    assert name(head_dim_qk=256, head_dim_v=256).endswith("_d256")
    # attn_bias / custom mask in e4m3, as the reference's OpDef allows (op_host/hstu_jagged_forward.cpp:65-66)
    assert name(attn_bias=0x2000) == "hstu_fwd_f8e4m3_f16_d128_rabtrue_maskfalse"
    assert name(mask=0x2000, mask_type=3, out_dtype=_native.DT_BF16) == "hstu_fwd_f8e4m3_bf16_d128_rabfalse_masktrue"
    # head dims above 256 and q/k head dims that are not multiples of 16: the coverage kernel's e4m3 instantiation
    assert name(head_dim_qk=24, head_dim_v=16) == "hstu_fwd_generic_f8e4m3_f16"
    assert name(head_dim_qk=512, head_dim_v=512, out_dtype=_native.DT_BF16) == "hstu_fwd_generic_f8e4m3_bf16"
    assert name(head_dim_qk=1, head_dim_v=272) == "hstu_fwd_generic_f8e4m3_f16"
    assert name(out_dtype=_native.DT_FP32) is None
    assert re.search("fp16 .* or bf16", _native.last_error()), _native.last_error()


def test_dense_op_is_registered_with_meta_inference():
    op = ops_rec.ascendc.attention.hstu_dense
    q = torch.empty(3, 40, 2, 64, device="meta", dtype=torch.bfloat16)
    v = torch.empty(3, 40, 2, 32, device="meta", dtype=torch.bfloat16)
    out = op(q, q, v, None, None, 0, 40, 0.0)
    assert out.shape == (3, 40, 2, 32) and out.dtype == torch.bfloat16
    with pytest.raises(RuntimeError, match="4D in dense layout"):
        op(q[0], q[0], v[0], None, None, 0, 40, 0.0)


def _copy_fwd(dst, src):
    ctypes.memmove(ctypes.byref(dst), ctypes.byref(src), ctypes.sizeof(_native.FwdParams))


def test_backward_c_abi_validation_codes():
    lib = _native.load()
    ws = ctypes.c_uint64(7)
    fake = 0x1000

    def make(**over):
        b = _native.new_bwd_params()
        f = _valid_params()
        for k, v in over.pop("fwd", {}).items():
            setattr(f, k, v)
        _copy_fwd(b.fwd, f)
        b.grad = b.grad_q = b.grad_k = b.grad_v = fake
        for k, v in over.items():
            setattr(b, k, v)
        return b

    def rc(b):
        return lib.hstu_jagged_bwd_workspace_size(ctypes.byref(b), ctypes.byref(ws))

    assert rc(make()) == 0 and ws.value == 0
    assert lib.hstu_jagged_bwd_workspace_size(None, ctypes.byref(ws)) == 161001
    assert lib.hstu_jagged_bwd_workspace_size(ctypes.byref(make()), None) == 161001
    assert rc(make(fwd=dict(out=None))) == 0  # the forward's output is not an input of the backward
    for over, code, text in [
        (dict(struct_size=8), 161002, "struct_size"),
        (dict(grad=None), 161001, "grad"),
        (dict(grad_k=None), 161001, "grad_k"),
        (dict(grad_attn_bias=fake), 161002, "without attn_bias"),
        (dict(fwd=dict(mask_type=1)), 161002, "triu"),
        (dict(fwd=dict(num_heads_k=3)), 161002, "divisible"),
        (dict(fwd=dict(dtype=_native.DT_FP8_E4M3, out_dtype=_native.DT_FP16)), 161003, "bf16, fp16 and fp32"),
    ]:
        got = rc(make(**over))
        assert got == code, (over, got, _native.last_error())
        assert re.search(text, _native.last_error()), (over, _native.last_error())
    # fp32 inputs and head dims beyond the tuned kernels are taken (by the generic kernels), as in the reference
    for fwd in (dict(dtype=_native.DT_FP32, out_dtype=_native.DT_FP32), dict(head_dim_qk=512, head_dim_v=512),
                dict(head_dim_qk=12, head_dim_v=16)):
        assert rc(make(fwd=fwd)) == 0, (fwd, _native.last_error())
    # launching with an invalid description is refused before any device call
    assert lib.hstu_jagged_bwd(ctypes.byref(make(fwd=dict(mask_type=1))), None, 0, None) == 161002


def test_backward_workspace_follows_the_launch_order(monkeypatch):
    """hstu_jagged_bwd_workspace_size asks for the workspace of the launch order the library will take: a plane of
    [batch, heads, max_q, max_k] elements for dS; for dS and P together one 128-byte line per query row of the batch
    and 32-key block -- all blocks of a row, or, for a causal mask over equal offsets without context rows, those at or
    below the diagonal only, bounded from the row count with 32 rows of slack per sequence; or none (the two-launch
    order; also whenever HSTU_MI355_BWD_HANDOFF=0)."""
    lib = _native.load()
    ws = ctypes.c_uint64(7)
    fake = 0x1000

    def size(grad_attn_bias=None, **fwd):
        b = _native.new_bwd_params()
        f = _valid_params()
        for k, v in fwd.items():
            setattr(f, k, v)
        if grad_attn_bias is not None:
            f.attn_bias = fake
        _copy_fwd(b.fwd, f)
        b.grad = b.grad_q = b.grad_k = b.grad_v = fake
        b.grad_attn_bias = grad_attn_bias
        assert lib.hstu_jagged_bwd_workspace_size(ctypes.byref(b), ctypes.byref(ws)) == 0, _native.last_error()
        return ws.value

    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", None)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_WORKSPACE_MB", None)
    c2 = dict(n_offsets=33, num_heads_q=4, num_heads_k=4, total_q=20292, total_k=20292, max_seq_len_q=1024, max_seq_len_k=1024)
    def pair(rows=20292, batch=32, heads=4, blocks=32):  # causal, equal offsets, no context rows
        return heads * (((rows + 32 * batch) * (blocks + 1) + 1) // 2) * 128

    def pair_all_blocks(rows=20292, heads=4, blocks=32):
        # (an odd number of lines per row: the lines of a block's 32 rows then fall on different memory channels)
        return heads * rows * (blocks | 1) * 128

    one = 32 * 4 * 1024 * 1024 * 2
    full = 32 * 1024
    assert size(**c2) == pair()  # a jagged batch whose planes stay in the memory-side cache: five products
    assert pair() < 185e6 < 0.35 * (32 * 4 * 1024 * 32 * 128)  # a third of one line per (padded row, block)
    assert size(**dict(c2, total_q=full, total_k=full)) == one  # the same without padding: three launches
    assert size(**dict(c2, head_dim_qk=64, head_dim_v=64)) == pair()  # small planes pay at every head dim
    assert size(**dict(c2, head_dim_qk=64, head_dim_v=64, num_heads_q=8, num_heads_k=8, total_q=full, total_k=full)) == 0  # larger ones: two launches
    # rows of [max_q][max_k] tensors that are not multiples of 16 bytes: the pair plane has its own layout and is taken all
    # the same when the call has no such tensor; with an attn_bias and its gradient the call runs in two launches
    assert size(**dict(c2, max_seq_len_q=1020, max_seq_len_k=1020)) == pair()
    assert size(grad_attn_bias=fake, **dict(c2, max_seq_len_q=1020, max_seq_len_k=1020)) == 0
    assert size(**dict(c2, head_dim_qk=256, head_dim_v=256, total_q=full, total_k=full)) == pair(rows=full)
    # long rows at head dim 128: two launches -- but max_seq_len is a bound, and the same 20292 rows under a bound of 4096
    # are priced by their mean length (the planes, sized for the bound: the host does not see the offsets)
    assert size(**dict(c2, max_seq_len_q=4096, max_seq_len_k=4096, total_q=32 * 4096, total_k=32 * 4096)) == 0
    assert size(**dict(c2, max_seq_len_q=4096, max_seq_len_k=4096)) == pair(blocks=128)
    # with an attn_bias gradient dS goes through the gradient itself in the three-launch order: planes or nothing
    assert size(grad_attn_bias=fake, **c2) in (0, pair())
    assert size(grad_attn_bias=fake, **dict(c2, total_q=full, total_k=full, head_dim_qk=64, head_dim_v=64)) == 0
    assert size(grad_attn_bias=fake, **dict(c2, n_offsets=9, total_q=5000, total_k=5000)) == pair(rows=5000, batch=8)  # a small gradient
    assert size(grad_attn_bias=fake, **dict(c2, head_dim_qk=256, head_dim_v=256)) == pair()
    # fp32: the matrix-instruction kernels (head dims up to 128) hand dS and P over in fp32, a plane per sequence; the
    # generic ones do not
    assert size(**dict(c2, dtype=_native.DT_FP32, out_dtype=_native.DT_FP32)) == 32 * 4 * 1024 * 64 * 32 * 4
    assert size(**dict(c2, dtype=_native.DT_FP32, out_dtype=_native.DT_FP32, head_dim_qk=256, head_dim_v=256)) == 0
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "0")
    assert size(**c2) == 0
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "1")
    assert size(**c2) == one and size(**dict(c2, head_dim_qk=64, head_dim_v=64)) == one
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_HANDOFF", "2")
    assert size(**c2) == pair()
    # every block of a row where the host cannot tell that rows see no key past their own: no mask, context rows,
    # key offsets of their own
    assert size(**dict(c2, mask_type=2)) == pair_all_blocks()
    assert size(**dict(c2, num_context=fake)) == pair_all_blocks()
    assert size(**dict(c2, seq_offset_k=fake + 64)) == pair_all_blocks()
    # batches of sequences of at most 32 rows and keys run in one launch that needs no workspace -- without bias or
    # custom mask, head dims up to 256 in multiples of 8, 16-byte aligned tensors; HSTU_MI355_SHORT=0 switches it off
    tiny = dict(c2, total_q=600, total_k=600, max_seq_len_q=32, max_seq_len_k=32)
    tiny_pair = pair(rows=600, blocks=1)
    assert size(**tiny) == 0 and size(**dict(tiny, head_dim_qk=256, head_dim_v=256)) == 0
    assert size(**dict(tiny, max_seq_len_q=40, max_seq_len_k=40)) == 0  # (the kernel for few query rows, below)
    assert size(**dict(tiny, max_seq_len_q=72, max_seq_len_k=72)) == pair(rows=600, blocks=3)
    assert size(**dict(tiny, q=fake + 8)) == tiny_pair
    assert size(grad_attn_bias=fake, **tiny) == tiny_pair
    # ... and so do sequences of at most 64 query rows against keys of any length at head dims up to 128 with as many
    # K/V heads as query heads
    few = dict(c2, total_q=1500, max_seq_len_q=64, head_dim_qk=64, head_dim_v=48, seq_offset_k=fake + 64)
    assert size(**few) == 0 and size(**dict(few, head_dim_qk=128, head_dim_v=96)) == 0
    for other in (dict(max_seq_len_q=72), dict(head_dim_qk=136), dict(num_heads_k=2), dict(k=fake + 8)):
        assert size(**dict(few, **other)) > 0
    assert size(grad_attn_bias=fake, **few) > 0
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", "0")
    assert size(**tiny) == tiny_pair and size(**few) > 0
    helpers.set_switch(monkeypatch, "HSTU_MI355_SHORT", None)
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_WORKSPACE_MB", "300")  # the limit of the workspace
    assert size(**dict(c2, mask_type=2)) == one
    helpers.set_switch(monkeypatch, "HSTU_MI355_BWD_WORKSPACE_MB", "100")
    assert size(**c2) == 0

def test_paged_c_abi_validation_codes():
    lib = _native.load()
    ws = ctypes.c_uint64(7)
    fake = 0x1000

    def make(**over):
        pp = _native.PagedParams()
        pp.struct_size = ctypes.sizeof(_native.PagedParams)
        f = _valid_params()
        for k, v in over.pop("fwd", {}).items():
            setattr(f, k, v)
        _copy_fwd(pp.fwd, f)
        pp.kv_cache = pp.page_offsets = pp.page_ids = fake
        pp.num_pages, pp.page_size, pp.n_page_ids = 4, 64, 4
        for k, v in over.items():
            setattr(pp, k, v)
        return pp

    def rc(pp):
        return lib.hstu_paged_fwd_workspace_size(ctypes.byref(pp), ctypes.byref(ws))

    assert rc(make()) == 0  # (no device here: the optional split workspace is reported as 0)
    # fp32 has no paged kernel: the rows are gathered into the workspace first, K and V of total_k rows each
    assert rc(make(fwd=dict(dtype=_native.DT_FP32, out_dtype=_native.DT_FP32))) == 0
    assert ws.value == 2 * 10 * 4 * 128 * 4
    for over, code, text in [
        (dict(struct_size=8), 161002, "struct_size"),
        (dict(kv_cache=None), 161001, "kv_cache"),
        (dict(page_ids=None), 161001, "page_ids"),
        (dict(page_size=48), 161002, "32, 64, 128 or 256"),
        (dict(num_pages=0), 161002, "must not be empty"),
        (dict(fwd=dict(head_dim_v=64)), 161002, "one head dim"),
        (dict(fwd=dict(dtype=_native.DT_FP8_E4M3, out_dtype=_native.DT_FP16)), 161003, "fp8"),
        (dict(fwd=dict(max_seq_len_q=0)), 161002, "20480"),
    ]:
        got = rc(make(**over))
        assert got == code, (over, got, _native.last_error())
        assert re.search(text, _native.last_error()), (over, _native.last_error())
    assert lib.hstu_paged_fwd(ctypes.byref(make(page_size=48)), None, 0, None) == 161002
    # the gather path refuses to run without its workspace
    pp = make(fwd=dict(dtype=_native.DT_FP32, out_dtype=_native.DT_FP32))
    assert lib.hstu_paged_fwd(ctypes.byref(pp), None, 0, None) == 161004 and "workspace" in _native.last_error()


def test_paged_and_dense_backward_ops_are_registered():
    assert [a.name for a in torch.ops.ops_rec.hstu_paged.default._schema.arguments][:4] == ["q", "k", "v", "kv_cache"]
    assert len(torch.ops.ops_rec.hstu_paged.default._schema.arguments) == 20
    q = torch.empty(10, 4, 32, device="meta", dtype=torch.float16)
    idx = torch.empty(3, device="meta", dtype=torch.int32)
    cache = torch.empty(2, 2, 32, 4, 32, device="meta", dtype=torch.float16)
    out = torch.ops.ops_rec.hstu_paged(q, q, q, cache, None, None, 0, 6, 6, 0.0, idx, idx, idx, idx, idx, idx[:2], idx[:2], 1)
    assert out.shape == q.shape and out.dtype == torch.float16
    g = torch.empty(2, 5, 4, 32, device="meta", dtype=torch.bfloat16)
    dq, dk, dv, db = torch.ops.ops_rec.hstu_dense_backward(g, g, g, g, None, None, 0, 5, 0.0)
    assert dq.shape == g.shape and tuple(db.shape) == (2, 4, 256, 256)


def test_public_headers_are_plain_c(tmp_path):
    # the boundary is a C ABI: both headers must compile as C99 and as C++11 on their own, and the struct sizes the
    # Python mirrors assume must be the ones the C compiler sees
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc on this host")
    src = tmp_path / "abi.c"
    src.write_text(
        '#include "hstu_mi355.h"\n#include "ops_rec_activation_mi355.h"\n#include <stdio.h>\n'
        "int main(void) { printf(\"%zu %zu %zu %zu %zu %zu %zu\\n\", sizeof(hstu_jagged_fwd_params), "
        "sizeof(hstu_jagged_bwd_params), sizeof(hstu_paged_fwd_params), sizeof(ln_mul_params), "
        "sizeof(in_linear_silu_params), sizeof(in_linear_silu_bwd_params), sizeof(void*)); return 0; }\n"
    )
    inc = os.path.join(_ROOT, "include")
    exe = tmp_path / "abi"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, str(src), "-o", str(exe)], check=True)
    sizes = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    mirrors = [_native.FwdParams, _native.BwdParams, _native.PagedParams, _native.LnMulParams, _native.InLinearSiluParams,
               _native.InLinearSiluBwdParams, ctypes.c_void_p]  # fmt: skip
    assert sizes == [ctypes.sizeof(m) for m in mirrors]
    gxx = shutil.which("g++")
    if gxx is not None:
        subprocess.run([gxx, "-std=c++11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc,
                        str(src)], check=True)  # fmt: skip


def test_forward_descriptions_are_cached_by_everything_but_the_addresses():
    """``prepare_forward`` keeps a validated description and patches only addresses on a repeat; a description
    that differs in any shape, type or scalar is validated afresh (the cache must never skip a check that would
    fail), and the cache is emptied with the switches."""
    from ops_rec import _ops

    key = lambda **kw: _ops._plan_key(**{**base, **kw})  # noqa: E731
    t = lambda *shape, dtype=torch.bfloat16: torch.zeros(*shape, dtype=dtype)  # noqa: E731
    offs = torch.tensor([0, 3, 7], dtype=torch.int32)
    base = dict(q=t(7, 2, 64), k=t(7, 2, 64), v=t(7, 2, 64), mask=None, attn_bias=None, mask_type=0, max_seq_len_q=8,
                max_seq_len_k=8, silu_scale=0.0, seq_offset=offs, seq_offset_k=offs, num_context=None, num_target=None,
                target_group_size=0, alpha=1.0, deterministic=False, out_dtype=None, q_descale=None, k_descale=None,
                v_descale=None, fp8_scaled_p=False)  # fmt: skip
    same = key(q=t(7, 2, 64), k=t(7, 2, 64), v=t(7, 2, 64))
    assert same == key() and hash(same) == hash(key())
    for change in (dict(q=t(8, 2, 64)), dict(v=t(7, 2, 32)), dict(k=t(7, 2, 64, dtype=torch.float16)), dict(mask_type=2),
                   dict(max_seq_len_q=16), dict(silu_scale=0.5), dict(alpha=0.25), dict(target_group_size=2),
                   dict(seq_offset_k=offs.clone()), dict(seq_offset=offs.long(), seq_offset_k=offs.long()),
                   dict(attn_bias=t(2, 2, 8, 8)), dict(num_context=offs[:2]), dict(q=t(7, 4, 64)[:, ::2]),
                   dict(deterministic=True)):  # fmt: skip
        assert key(**change) != same, change
    _ops._PLAN_CACHE["x"] = None
    _native.reload_switches()
    assert not _ops._PLAN_CACHE


def test_backward_workspace_that_cannot_be_allocated_is_left_out(monkeypatch):
    """The backward's workspace is optional scratch: when the allocator has no room for it the adapter passes none
    (the library then takes an order that needs none) instead of failing a call the reference's backward would serve."""
    from ops_rec import _ops

    calls = []

    def no_room(*args, **kwargs):
        calls.append(args)
        raise torch.cuda.OutOfMemoryError("HIP out of memory (test)")

    assert _ops._new_workspace(0, torch.device("cpu")) is None  # nothing asked for, nothing allocated
    monkeypatch.setattr(_ops.torch, "empty", no_room)
    assert _ops._new_workspace(1 << 20, torch.device("cpu")) is None and len(calls) == 1
    monkeypatch.undo()
    ws = _ops._new_workspace(4096, torch.device("cpu"))
    assert ws is not None and ws.numel() == 4096 and ws.dtype == torch.uint8
