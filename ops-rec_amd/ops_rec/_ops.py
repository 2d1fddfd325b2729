"""Operator registration for ``torch.ops.ops_rec.hstu_jagged[_backward]``.

Mirrors the reference adapter for this path
(ascendc/attention/hstu_v1/torch_extension/hstu_jagged_plugin.cpp):

* the four schema strings are the reference's (``:188-247``) -- they are the calling contract;
* ``_forward_impl`` does the argument normalisation and checks of
  ``hstu_deltaq_forward_impl_npu`` (``:22-67``) and then calls the C ABI of the HIP library
  where the reference calls ``aclnnHstuJaggedForward`` (``:63-65``);
* device tensors dispatch on the ``CUDA`` key (PyTorch-ROCm's key for HIP tensors), shape
  inference for ``torch.compile`` on ``Meta`` (``:269-351``); autograd is attached from Python
  (``ops_rec/autograd/hstu_v1_autograd.py``), not here (``:258-263``).

There is no CPU implementation: calling the op on CPU tensors raises, as it does in the
reference (which registers only the NPU and Meta keys).
"""

from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _native

_MAX_SEQ_LEN = 20480

_SCHEMAS = (
    "hstu_jagged.equal(Tensor q, Tensor k, Tensor v, Tensor? mask=None, Tensor? attn_bias=None, int mask_type=0, "
    "int max_seq_len=0, float silu_scale=0.0, Tensor seq_offset=None, Tensor? num_context=None, "
    "Tensor? num_target=None, int? target_group_size=0, float? alpha=1.0, bool deterministic=False) -> Tensor",
    "hstu_jagged_backward.equal(Tensor grad, Tensor q, Tensor k, Tensor v, Tensor? mask=None, "
    "Tensor? attn_bias=None, int mask_type=0, int max_seq_len=0, float silu_scale=0.0, Tensor seq_offset=None, "
    "Tensor? num_context=None, Tensor? num_target=None, int? target_group_size=0, float? alpha=1.0) "
    "-> (Tensor, Tensor, Tensor, Tensor)",
    "hstu_jagged.delta(Tensor q, Tensor k, Tensor v, Tensor? mask=None, Tensor? attn_bias=None, int mask_type=0, "
    "int max_seq_len=0, int max_seq_len_k=0, float silu_scale=0.0, Tensor seq_offset=None, "
    "Tensor seq_offset_k=None, Tensor? num_context=None, Tensor? num_target=None, int? target_group_size=0, "
    "float? alpha=1.0, bool deterministic=False) -> Tensor",
    "hstu_jagged_backward.delta(Tensor grad, Tensor q, Tensor k, Tensor v, Tensor? mask=None, "
    "Tensor? attn_bias=None, int mask_type=0, int max_seq_len=0, int max_seq_len_k=0, float silu_scale=0.0, "
    "Tensor seq_offset=None, Tensor seq_offset_k=None, Tensor? num_context=None, Tensor? num_target=None, "
    "int? target_group_size=0, float? alpha=1.0) -> (Tensor, Tensor, Tensor, Tensor)",
    # dense [B, S, N, D] layout (torch_extension/hstu_dense_plugin.cpp:156-172)
    "hstu_dense(Tensor q, Tensor k, Tensor v, Tensor? mask=None, Tensor? attn_bias=None, int mask_type=0, "
    "int max_seq_len=0, float silu_scale=0.0) -> Tensor",
    "hstu_dense_backward(Tensor grad, Tensor q, Tensor k, Tensor v, Tensor? mask, Tensor? attn_bias, int mask_type=0, "
    "int max_seq_len=0, float silu_scale=0.0) -> (Tensor, Tensor, Tensor, Tensor)",
    # paged KV cache (torch_extension/hstu_paged_plugin.cpp:71-92)
    "hstu_paged(Tensor q, Tensor k, Tensor v, Tensor kv_cache=None, Tensor? mask=None, Tensor? attn_bias=None, "
    "int mask_type=0, int max_seq_len=0, int max_seq_len_k=0, float silu_scale=0.0, Tensor seq_offset=None, "
    "Tensor seq_offset_k=None, Tensor seq_offset_t=None, Tensor page_offsets=None, Tensor page_ids=None, "
    "Tensor last_page_len=None, Tensor num_target=None, int target_group_size=0, float? alpha=1.0, "
    "bool deterministic=False) -> Tensor",
)

_lib_def = torch.library.Library("ops_rec", "DEF")
for _s in _SCHEMAS:
    _lib_def.define(_s)
_lib_cuda = torch.library.Library("ops_rec", "IMPL", "CUDA")
_lib_meta = torch.library.Library("ops_rec", "IMPL", "Meta")

_DTYPE_CODE = {
    torch.bfloat16: _native.DT_BF16,
    torch.float16: _native.DT_FP16,
    torch.float32: _native.DT_FP32,
    torch.float8_e4m3fn: _native.DT_FP8_E4M3,
}


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _max_seq_len_check(value: int, what: str) -> None:
    _check(1 <= value <= _MAX_SEQ_LEN, f"{what} check failed: maxSeqLen expect in [1, 20480], but value is {value}")


def _mask_check(mask_type: int, mask_defined: bool) -> None:
    _check(0 <= mask_type <= 3, f"maskType expect in [0, 3], but value is {mask_type}")
    _check(mask_type != 1, "maskType current not support triu now, pls use custome mask")
    _check(not (mask_type == 3 and not mask_defined), "use custome mask must have valide mask tensor")


def _check_devices(device: torch.device, named) -> None:
    """Every tensor argument must live on the GPU the call runs on.  The kernels read the offsets, counts and page
    tables through raw device addresses: a host tensor among them (``seq_offset=torch.tensor([...])`` without
    ``device=``) would hand the kernel a host pointer, which is a GPU memory fault, not a Python error.
    (That q itself is a GPU tensor is checked where a launch is about to happen.)"""
    for name, t in named:
        if t is not None:
            _check(t.device == device, f"{name} must be on the device of q ({device}), but it is on {t.device}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None or t.numel() == 0:
        return None
    return t.data_ptr()


def _out_dtype(q: torch.Tensor) -> torch.dtype:
    return torch.float16 if q.dtype == torch.float8_e4m3fn else q.dtype


class PreparedForward:
    """A validated forward call: the filled C-ABI parameter block, its output tensor and the
    tensors it points into.  ``launch()`` enqueues it on the current stream; it may be launched
    repeatedly (benchmarks, steady-state serving with static shapes)."""

    __slots__ = ("params", "out", "workspace", "workspace_bytes", "device", "_keep")

    def __init__(self, params, out, workspace, workspace_bytes, device, keep):
        self.params = params
        self.out = out
        self.workspace = workspace
        self.workspace_bytes = workspace_bytes
        self.device = device
        self._keep = keep

    def launch(self, stream: Optional[int] = None) -> torch.Tensor:
        if self.out.numel() == 0:
            return self.out
        _check(self.device.type == "cuda", f"q must be a GPU tensor, but it is on {self.device}")
        lib = _native.load()
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        rc = lib.hstu_jagged_fwd(ctypes.byref(self.params), _ptr(self.workspace), self.workspace_bytes,
                                 ctypes.c_void_p(stream))  # fmt: skip
        if rc != _native.HSTU_OK:
            raise RuntimeError(f"hstu_jagged_fwd failed ({rc}): {_native.last_error()}")
        return self.out

    def kernel_name(self) -> str:
        name = _native.load().hstu_jagged_fwd_kernel_name(ctypes.byref(self.params))
        return name.decode() if name else ""


# Validated calls, by everything but the addresses: (shapes, dtypes, devices, scalars) -> (parameter block with the
# scalar fields filled, workspace bytes).  A steady-state caller repeats one description with new tensors; on a hit
# the checks below, the filling of the block and the workspace-size call are skipped and only the addresses are
# patched in.  The library's answer depends on its switches too: ``_native.reload_switches()`` empties the cache.
_PLAN_CACHE: dict = {}
_PLAN_CACHE_MAX = 256


def _meta(t: Optional[torch.Tensor]):
    return None if t is None else (t.shape, t.dtype, t.device, t.is_contiguous())


def _plan_key(q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale, seq_offset, seq_offset_k,
              num_context, num_target, target_group_size, alpha, deterministic, out_dtype, q_descale, k_descale,
              v_descale, fp8_scaled_p):  # fmt: skip
    return (_meta(q), _meta(k), _meta(v), _meta(mask), _meta(attn_bias), mask_type, max_seq_len_q, max_seq_len_k,
            silu_scale, _meta(seq_offset), seq_offset_k is seq_offset or _meta(seq_offset_k), _meta(num_context),
            _meta(num_target), target_group_size, alpha, deterministic, out_dtype, _meta(q_descale), _meta(k_descale),
            _meta(v_descale), fp8_scaled_p)  # fmt: skip


def _prepare_from_plan(plan, q, k, v, mask, attn_bias, seq_offset, seq_offset_k, num_context, num_target, scales):
    """A cached description applied to new tensors (all of them contiguous and of the index type already: a
    description is only cached when nothing had to be copied or converted)."""
    template, ws_bytes, out_shape, out_dtype, use_mask = plan
    p = _native.FwdParams.from_buffer_copy(template)
    out = torch.empty(out_shape, dtype=out_dtype, device=q.device)
    mask_c = mask if use_mask else None
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    p.mask, p.attn_bias = _ptr(mask_c), _ptr(attn_bias)
    p.seq_offset_q, p.seq_offset_k = seq_offset.data_ptr(), seq_offset_k.data_ptr()
    p.num_context, p.num_target = _ptr(num_context), _ptr(num_target)
    p.out = out.data_ptr()
    p.q_descale, p.k_descale, p.v_descale = (_ptr(t) for t in scales)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    keep = (q, k, v, mask_c, attn_bias, seq_offset, seq_offset_k, num_context, num_target, *scales)
    return PreparedForward(p, out, ws, ws_bytes, q.device, keep)


def prepare_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: Optional[torch.Tensor],
    attn_bias: Optional[torch.Tensor],
    mask_type: int,
    max_seq_len_q: int,
    max_seq_len_k: int,
    silu_scale: float,
    seq_offset: torch.Tensor,
    seq_offset_k: torch.Tensor,
    num_context: Optional[torch.Tensor],
    num_target: Optional[torch.Tensor],
    target_group_size: Optional[int],
    alpha: Optional[float],
    deterministic: bool = False,
    *,
    out_dtype: Optional[torch.dtype] = None,
    q_descale: Optional[torch.Tensor] = None,
    k_descale: Optional[torch.Tensor] = None,
    v_descale: Optional[torch.Tensor] = None,
    fp8_scaled_p: bool = False,
) -> PreparedForward:
    """Argument normalisation and checks of the reference adapter
    (torch_extension/hstu_jagged_plugin.cpp:22-67), ending in a filled parameter block.

    The keyword-only arguments belong to the fp8 extension (``hstu_jagged_fp8``): output type
    (fp16 as in the reference, or bf16), per-head fp32 dequantisation scales, and the rounding point of P:
    ``fp8_scaled_p=True`` is the reference's, ``P = e4m3(silu(X) * silu_scale * M)``
    (hstu_forward_v1/test/pytest/test_hstu_jagged.py:183-195), and what a call through the reference's own
    entry point with e4m3 tensors gets; ``False`` quantises ``silu(X) * M`` and applies ``silu_scale`` to the
    fp32 output."""
    key = None
    if isinstance(q, torch.Tensor) and isinstance(seq_offset, torch.Tensor) and isinstance(seq_offset_k, torch.Tensor):
        key = _plan_key(q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale, seq_offset,
                        seq_offset_k, num_context, num_target, target_group_size, alpha, deterministic, out_dtype,
                        q_descale, k_descale, v_descale, fp8_scaled_p)  # fmt: skip
        plan = _PLAN_CACHE.get(key)
        if plan is not None:
            return _prepare_from_plan(plan, q, k, v, mask, attn_bias, seq_offset, seq_offset_k, num_context,
                                      num_target, (q_descale, k_descale, v_descale))  # fmt: skip
    _check(q.dim() == 3, "The q should be 3D in jagged layout")
    _check(seq_offset is not None and seq_offset_k is not None, "seq_offset is required")
    _check(seq_offset.dim() == 1 and seq_offset.size(0) >= 2,
           "acSeqOffset params error should have at least two element.")  # fmt: skip
    _check(seq_offset_k.dim() == 1 and seq_offset_k.size(0) >= 2,
           "acSeqOffsetK params error should have at least two element.")  # fmt: skip
    _check(seq_offset.dtype in (torch.int32, torch.int64), "seq_offset must be int32 or int64")
    _check(k.dim() == 3 and v.dim() == 3, "The k and v should be 3D in jagged layout")
    _check(q.dtype == k.dtype == v.dtype, "q, k, v must share one dtype")
    _check(q.dtype in _DTYPE_CODE, f"unsupported dtype {q.dtype}")
    _check_devices(q.device, (("k", k), ("v", v), ("mask", mask), ("attn_bias", attn_bias), ("seq_offset", seq_offset),
                              ("seq_offset_k", seq_offset_k), ("num_context", num_context), ("num_target", num_target),
                              ("q_descale", q_descale), ("k_descale", k_descale), ("v_descale", v_descale)))  # fmt: skip

    idx_dtype = seq_offset.dtype
    offs_q = seq_offset.contiguous()
    offs_k = offs_q if seq_offset_k is seq_offset else seq_offset_k.to(idx_dtype).contiguous()
    q_c, k_c, v_c = q.contiguous(), k.contiguous(), v.contiguous()
    batch = offs_q.size(0) - 1
    ctx = num_context.to(idx_dtype).contiguous() if num_context is not None else None
    tgt = num_target.to(idx_dtype).contiguous() if num_target is not None else None
    group = 0 if target_group_size is None else int(target_group_size)
    real_alpha = 1.0 if alpha is None else float(alpha)

    _max_seq_len_check(int(max_seq_len_q), "maxSeqLen")
    _max_seq_len_check(int(max_seq_len_k), "maxSeqLenK")
    _mask_check(int(mask_type), mask is not None)
    _check(offs_k.size(0) == offs_q.size(0), "seq_offset and seq_offset_k must have the same length")
    _check(k_c.size(0) == v_c.size(0), "K, V seqLens mismatch")
    _check(k_c.size(1) == v_c.size(1), "K, V headNum mismatch")
    _check(q_c.size(2) == k_c.size(2), "Q, K, V headDIM Shape Check failed")
    if ctx is not None:
        _check(ctx.dim() == 1 and ctx.size(0) == batch, f"The length of num_context expect {batch}")
    if tgt is not None:
        _check(tgt.dim() == 1 and tgt.size(0) == batch, f"The length of num_target expect {batch}")
    bias_shape = (batch, q_c.size(1), int(max_seq_len_q), int(max_seq_len_k))
    bias = None
    if attn_bias is not None:
        _check(attn_bias.dtype == q.dtype, "attn_bias must have the dtype of q")
        _check(tuple(attn_bias.shape) == bias_shape, f"attn_bias must have shape {bias_shape}")
        bias = attn_bias.contiguous()
    mask_c = None
    if mask is not None and int(mask_type) == 3:
        _check(mask.dtype == q.dtype, "mask must have the dtype of q")
        _check(tuple(mask.shape) == bias_shape, f"mask must have shape {bias_shape}")
        mask_c = mask.contiguous()

    is_fp8 = q_c.dtype == torch.float8_e4m3fn
    _check(is_fp8 or (out_dtype is None and q_descale is None and k_descale is None and v_descale is None
                      and not fp8_scaled_p),
           "out_dtype, descales and fp8_scaled_p are only taken with fp8 inputs")  # fmt: skip
    if out_dtype is None:
        out_dtype = _out_dtype(q_c)
    _check(not is_fp8 or out_dtype in (torch.float16, torch.bfloat16), "fp8 inputs produce fp16 or bf16 output")
    scales = []
    for name, t, heads in (("q_descale", q_descale, q_c.size(1)), ("k_descale", k_descale, k_c.size(1)),
                           ("v_descale", v_descale, k_c.size(1))):  # fmt: skip
        if t is not None:
            _check(t.dtype == torch.float32 and t.dim() == 1 and t.size(0) == heads and t.device == q_c.device,
                   f"{name} must be a float32 tensor of {heads} per-head scales on the device of q")  # fmt: skip
            t = t.contiguous()
        scales.append(t)
    # Every row of a well-formed call is written by the kernel (rows past the last offset are zero-filled there), so
    # the zero-fill of the reference adapter (:56-59) is not repeated here.  Well-formed: the first offset is 0 and no
    # sequence is longer than max_seq_len; rows before a non-zero first offset and rows of a sequence past
    # max_seq_len belong to no work item and keep what the allocator handed out, where the reference returns zeros
    # (tests/test_gpu_output_rows.py pins which rows those are).
    out = torch.empty((q_c.size(0), q_c.size(1), v_c.size(2)), dtype=out_dtype, device=q_c.device)
    keep = (q_c, k_c, v_c, mask_c, bias, offs_q, offs_k, ctx, tgt, *scales)
    p = _native.new_params()
    if out.numel() == 0:
        return PreparedForward(p, out, None, 0, q_c.device, keep)

    real_scale = (1.0 / float(max_seq_len_q)) if float(silu_scale) == 0.0 else float(silu_scale)

    lib = _native.load()
    p.dtype = _DTYPE_CODE[q_c.dtype]
    p.out_dtype = _DTYPE_CODE[out_dtype]
    p.index_dtype = _native.IDX_I64 if idx_dtype == torch.int64 else _native.IDX_I32
    p.q, p.k, p.v = _ptr(q_c), _ptr(k_c), _ptr(v_c)
    p.mask, p.attn_bias = _ptr(mask_c), _ptr(bias)
    p.seq_offset_q, p.seq_offset_k = _ptr(offs_q), _ptr(offs_k)
    p.num_context, p.num_target = _ptr(ctx), _ptr(tgt)
    p.out = _ptr(out)
    p.total_q, p.total_k = q_c.size(0), k_c.size(0)
    p.num_heads_q, p.num_heads_k = q_c.size(1), k_c.size(1)
    p.head_dim_qk, p.head_dim_v = q_c.size(2), v_c.size(2)
    p.n_offsets = offs_q.size(0)
    p.mask_type = int(mask_type)
    p.max_seq_len_q, p.max_seq_len_k = int(max_seq_len_q), int(max_seq_len_k)
    p.target_group_size = group
    p.silu_scale = real_scale
    p.alpha = real_alpha
    p.deterministic = 1 if deterministic else 0
    p.fp8_scaled_p = 1 if (is_fp8 and fp8_scaled_p) else 0
    p.q_descale, p.k_descale, p.v_descale = (_ptr(t) for t in scales)

    ws_bytes = ctypes.c_uint64(0)
    rc = lib.hstu_jagged_fwd_workspace_size(ctypes.byref(p), ctypes.byref(ws_bytes))
    if rc != _native.HSTU_OK:
        raise RuntimeError(f"hstu_jagged_fwd_workspace_size failed ({rc}): {_native.last_error()}")
    ws = None
    if ws_bytes.value:
        ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=q_c.device)
    # remember the description when the tensors went in as they came (nothing copied, nothing converted): the same
    # description with other tensors then needs only their addresses
    as_given = (q_c is q and k_c is k and v_c is v and offs_q is seq_offset and offs_k is seq_offset_k and ctx is num_context
                and tgt is num_target and bias is attn_bias and (mask_c is None or mask_c is mask)
                and all(t is g for t, g in zip(scales, (q_descale, k_descale, v_descale))))  # fmt: skip
    if key is not None and as_given:
        if len(_PLAN_CACHE) >= _PLAN_CACHE_MAX:
            _PLAN_CACHE.clear()
        _PLAN_CACHE[key] = (bytes(p), ws_bytes.value, tuple(out.shape), out_dtype, mask_c is not None)
    return PreparedForward(p, out, ws, ws_bytes.value, q_c.device, keep)


def _forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale, seq_offset,
                  seq_offset_k, num_context, num_target, target_group_size, alpha, deterministic=False):  # fmt: skip
    # (e4m3 tensors through the reference's entry point: the reference's rounding point of P)
    prepared = prepare_forward(q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale,
                               seq_offset, seq_offset_k, num_context, num_target, target_group_size, alpha,
                               deterministic, fp8_scaled_p=q.dtype == torch.float8_e4m3fn)  # fmt: skip
    with torch.cuda.device(prepared.device):
        return prepared.launch()


def hstu_jagged_fp8(q, k, v, q_descale=None, k_descale=None, v_descale=None, *, mask=None, attn_bias=None, mask_type=0,
                    max_seq_len=0, max_seq_len_k=None, silu_scale=0.0, seq_offset=None, seq_offset_k=None,
                    num_context=None, num_target=None, target_group_size=0, alpha=1.0, out_dtype=torch.bfloat16):  # fmt: skip
    """Forward on fp8-e4m3 (``torch.float8_e4m3fn``) Q / K / V with per-head fp32 dequantisation scales.

    An extension: the reference's fp8 path (``hstu_jagged`` called with e4m3 tensors, which this package serves
    too, rounding point and all) has no scales and a half output.  Here ``x = x8 * descale[head]`` for each of
    q, k, v (``None`` = 1), P is re-quantised to e4m3 BEFORE ``silu_scale`` is applied (the reference's order puts
    ``silu(X) / max_seq_len`` below e4m3's range), and the output is ``out_dtype`` (bf16 or fp16).  ``attn_bias``
    and a custom ``mask`` are e4m3 tensors like q."""
    _check(q.dtype == torch.float8_e4m3fn, "hstu_jagged_fp8 takes float8_e4m3fn tensors")
    offs_k = seq_offset if seq_offset_k is None else seq_offset_k
    max_k = max_seq_len if max_seq_len_k is None else max_seq_len_k
    prepared = prepare_forward(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_k, silu_scale, seq_offset, offs_k,
                               num_context, num_target, target_group_size, alpha, False, out_dtype=out_dtype,
                               q_descale=q_descale, k_descale=k_descale, v_descale=v_descale)  # fmt: skip
    with torch.cuda.device(prepared.device):
        return prepared.launch()


# Python kernels receive only the arguments the caller passed, so the schema defaults are
# repeated in the signatures below.


def hstu_jagged_equal(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, silu_scale=0.0,
                      seq_offset=None, num_context=None, num_target=None, target_group_size=0, alpha=1.0,
                      deterministic=False):  # fmt: skip
    return _forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len, silu_scale, seq_offset,
                         seq_offset, num_context, num_target, target_group_size, alpha, deterministic)  # fmt: skip


def hstu_jagged_delta(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, max_seq_len_k=0,
                      silu_scale=0.0, seq_offset=None, seq_offset_k=None, num_context=None, num_target=None,
                      target_group_size=0, alpha=1.0, deterministic=False):  # fmt: skip
    return _forward_impl(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale, seq_offset,
                         seq_offset_k, num_context, num_target, target_group_size, alpha, deterministic)  # fmt: skip


def _forward_meta(q, v):
    _check(q.dim() == 3, "The q should be 3D in jagged layout")
    return q.new_empty((q.shape[0], q.shape[1], v.shape[2]), dtype=_out_dtype(q))


def hstu_jagged_equal_meta(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, silu_scale=0.0,
                           seq_offset=None, num_context=None, num_target=None, target_group_size=0, alpha=1.0,
                           deterministic=False):  # fmt: skip
    return _forward_meta(q, v)


def hstu_jagged_delta_meta(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, max_seq_len_k=0,
                           silu_scale=0.0, seq_offset=None, seq_offset_k=None, num_context=None, num_target=None,
                           target_group_size=0, alpha=1.0, deterministic=False):  # fmt: skip
    return _forward_meta(q, v)


# ----------------------------------------------------------------------------------------------
# backward op: HIP kernels through the C ABI (_backward_hip) -- the tuned MFMA kernels for bf16 / fp16 with head
# dims up to 256, the library's generic fp32-arithmetic kernels for the rest (fp32 inputs, larger or odd head dims),
# which HSTU_MI355_GENERIC_BACKWARD=1 in the environment also selects for comparisons.
#   X = alpha (S + rab),  sig = sigmoid(X),  P = X sig scale M
#   dV = P^T dO,  dX = (dO V^T) scale M sig (1 + X (1 - sig)),  dS = dRab = alpha dX,  dQ = dS K,  dK = dS^T Q
# (ascendc/attention/hstu_v1/hstu_backward_v1/op_kernel/vector_score.h:159-205)
# ----------------------------------------------------------------------------------------------


def _new_grad(like: torch.Tensor) -> torch.Tensor:
    """Storage for one of dq / dk / dv / the bias gradient."""
    return torch.empty_like(like)


def _new_workspace(n_bytes: int, device) -> Optional[torch.Tensor]:
    """The workspace ``hstu_jagged_bwd`` asked for, or None when the device has no room for it: the library then
    runs the launch order that needs none (everything recomputed where it is used), so a backward never fails for
    want of scratch memory the reference's backward would not have needed."""
    if n_bytes == 0:
        return None
    try:
        return torch.empty(n_bytes, dtype=torch.uint8, device=device)
    except torch.cuda.OutOfMemoryError:
        return None


def _launch_backward(p, ws_bytes: int, device) -> None:
    ws = _new_workspace(ws_bytes, device)
    stream = torch.cuda.current_stream(device).cuda_stream
    rc = _native.load().hstu_jagged_bwd(ctypes.byref(p), _ptr(ws), ws.numel() if ws is not None else 0, ctypes.c_void_p(stream))
    if rc != _native.HSTU_OK:
        raise RuntimeError(f"hstu_jagged_bwd failed ({rc}): {_native.last_error()}")


def _backward_from_plan(plan, grad, q, k, v, mask, attn_bias, seq_offset, seq_offset_k, num_context, num_target):
    """A cached backward description applied to new tensors (all contiguous and of the index type already: a description
    is only cached when nothing had to be copied or converted)."""
    template, ws_bytes, use_mask = plan
    p = _native.BwdParams.from_buffer_copy(template)
    dq, dk, dv = _new_grad(q), _new_grad(k), _new_grad(v)
    dbias = _new_grad(attn_bias) if attn_bias is not None else None
    f = p.fwd
    f.q, f.k, f.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    f.mask, f.attn_bias = _ptr(mask if use_mask else None), _ptr(attn_bias)
    f.seq_offset_q, f.seq_offset_k = seq_offset.data_ptr(), seq_offset_k.data_ptr()
    f.num_context, f.num_target = _ptr(num_context), _ptr(num_target)
    p.grad, p.grad_q, p.grad_k, p.grad_v, p.grad_attn_bias = grad.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), _ptr(dbias)
    _launch_backward(p, ws_bytes, q.device)
    return dq, dk, dv, dbias


def _backward_hip(grad, q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale, seq_offset,
                  seq_offset_k, num_context, num_target, group, alpha):  # fmt: skip
    """The backward through the C ABI (``hstu_jagged_bwd``): one to four kernels on the current stream, with the
    workspace the library asks for (dS, or dS and P, handed from the query-tile kernel to the key-tile workgroups).
    Validated calls are cached like the forward's, by everything but the addresses."""
    key = ("bwd", _meta(grad), _meta(q), _meta(k), _meta(v), _meta(mask), _meta(attn_bias), mask_type, max_seq_len_q,
           max_seq_len_k, silu_scale, _meta(seq_offset), seq_offset_k is seq_offset or _meta(seq_offset_k),
           _meta(num_context), _meta(num_target), group, alpha)  # fmt: skip
    plan = _PLAN_CACHE.get(key)
    if plan is not None:
        return _backward_from_plan(plan, grad, q, k, v, mask, attn_bias, seq_offset, seq_offset_k, num_context, num_target)
    _check(q.device.type == "cuda", f"q must be a GPU tensor, but it is on {q.device}")
    _check_devices(q.device, (("grad", grad), ("k", k), ("v", v), ("mask", mask), ("attn_bias", attn_bias),
                              ("seq_offset", seq_offset), ("seq_offset_k", seq_offset_k), ("num_context", num_context),
                              ("num_target", num_target)))  # fmt: skip
    idx_dtype = seq_offset.dtype
    offs_q = seq_offset.contiguous()
    offs_k = offs_q if seq_offset_k is seq_offset else seq_offset_k.to(idx_dtype).contiguous()
    q_c, k_c, v_c, g_c = q.contiguous(), k.contiguous(), v.contiguous(), grad.contiguous()
    batch = offs_q.size(0) - 1
    ctx = num_context.to(idx_dtype).contiguous() if num_context is not None else None
    tgt = num_target.to(idx_dtype).contiguous() if num_target is not None else None
    _check(g_c.dtype == q_c.dtype == k_c.dtype == v_c.dtype, "grad, q, k, v must share one dtype")
    _check(tuple(g_c.shape) == (q_c.size(0), q_c.size(1), v_c.size(2)), "grad must have the shape of the forward output")
    bias_shape = (batch, q_c.size(1), int(max_seq_len_q), int(max_seq_len_k))
    bias = mask_c = None
    if attn_bias is not None:
        _check(attn_bias.dtype == q.dtype and tuple(attn_bias.shape) == bias_shape, f"attn_bias must be {bias_shape} of q's dtype")
        bias = attn_bias.contiguous()
    if int(mask_type) == 3:
        _check(mask is not None and mask.dtype == q.dtype and tuple(mask.shape) == bias_shape,
               f"mask must be {bias_shape} of q's dtype")  # fmt: skip
        mask_c = mask.contiguous()
    # every row of dq / dk / dv and every element of the bias gradient is written by the call (rows past the last
    # offset and the bias gradient outside what the query tiles sweep are zero-filled there)
    dq, dk, dv = _new_grad(q_c), _new_grad(k_c), _new_grad(v_c)
    if q_c.numel() == 0 and k_c.numel() == 0:
        return dq, dk, dv, (torch.zeros_like(bias) if bias is not None else None)
    dbias = _new_grad(bias) if bias is not None else None
    p = _native.new_bwd_params()
    f = p.fwd
    f.dtype = f.out_dtype = _DTYPE_CODE[q_c.dtype]
    f.index_dtype = _native.IDX_I64 if idx_dtype == torch.int64 else _native.IDX_I32
    f.q, f.k, f.v = _ptr(q_c), _ptr(k_c), _ptr(v_c)
    f.mask, f.attn_bias = _ptr(mask_c), _ptr(bias)
    f.seq_offset_q, f.seq_offset_k = _ptr(offs_q), _ptr(offs_k)
    f.num_context, f.num_target = _ptr(ctx), _ptr(tgt)
    f.total_q, f.total_k = q_c.size(0), k_c.size(0)
    f.num_heads_q, f.num_heads_k = q_c.size(1), k_c.size(1)
    f.head_dim_qk, f.head_dim_v = q_c.size(2), v_c.size(2)
    f.n_offsets = offs_q.size(0)
    f.mask_type = int(mask_type)
    f.max_seq_len_q, f.max_seq_len_k = int(max_seq_len_q), int(max_seq_len_k)
    f.target_group_size = group
    f.silu_scale = (1.0 / float(max_seq_len_q)) if float(silu_scale) == 0.0 else float(silu_scale)
    f.alpha = alpha
    p.grad, p.grad_q, p.grad_k, p.grad_v, p.grad_attn_bias = _ptr(g_c), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(dbias)
    lib = _native.load()
    ws_bytes = ctypes.c_uint64(0)
    rc = lib.hstu_jagged_bwd_workspace_size(ctypes.byref(p), ctypes.byref(ws_bytes))
    if rc != _native.HSTU_OK:
        raise RuntimeError(f"hstu_jagged_bwd_workspace_size failed ({rc}): {_native.last_error()}")
    _launch_backward(p, ws_bytes.value, q_c.device)
    # (cached when every tensor was taken as it came: the next call with this description only patches addresses in)
    same = (q_c is q and k_c is k and v_c is v and g_c is grad and offs_q is seq_offset and
            (offs_k is seq_offset_k or seq_offset_k is seq_offset) and ctx is num_context and tgt is num_target and
            bias is attn_bias and (mask_c is None or mask_c is mask))  # fmt: skip
    if same:
        if len(_PLAN_CACHE) >= _PLAN_CACHE_MAX:
            _PLAN_CACHE.clear()
        _PLAN_CACHE[key] = (bytes(p), ws_bytes.value, mask_c is not None)
    return dq, dk, dv, dbias


def _backward_impl(grad, q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale, seq_offset,
                   seq_offset_k, num_context, num_target, target_group_size, alpha):  # fmt: skip
    _check(seq_offset.size(0) >= 2, "seqOffsetQ params error should have at least two element.")
    _check(seq_offset_k.size(0) >= 2, "seqOffsetK params error should have at least two element.")
    _max_seq_len_check(int(max_seq_len_q), "maxSeqLenQ")
    _max_seq_len_check(int(max_seq_len_k), "maxSeqLenK")
    if num_context is not None or num_target is not None:
        _check(num_context is not None, "numContext is required when numTarget or targetGroupSize is not None")
        _check(num_target is not None, "numTarget is required when numContext or targetGroupSize is not None")
    group = 0 if target_group_size is None else int(target_group_size)
    a = 1.0 if alpha is None else float(alpha)
    _check(q.dtype in (torch.bfloat16, torch.float16, torch.float32), f"q must be bfloat16, float16 or float32, got {q.dtype}")
    _mask_check(int(mask_type), mask is not None)
    return _backward_hip(grad, q, k, v, mask, attn_bias, mask_type, max_seq_len_q, max_seq_len_k, silu_scale,
                         seq_offset, seq_offset_k, num_context, num_target, group, a)  # fmt: skip


def hstu_jagged_backward_equal(grad, q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, silu_scale=0.0,
                               seq_offset=None, num_context=None, num_target=None, target_group_size=0,
                               alpha=1.0):  # fmt: skip
    return _backward_impl(grad, q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len, silu_scale,
                          seq_offset, seq_offset, num_context, num_target, target_group_size, alpha)  # fmt: skip


def hstu_jagged_backward_delta(grad, q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0,
                               max_seq_len_k=0, silu_scale=0.0, seq_offset=None, seq_offset_k=None,
                               num_context=None, num_target=None, target_group_size=0, alpha=1.0):  # fmt: skip
    return _backward_impl(grad, q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale,
                          seq_offset, seq_offset_k, num_context, num_target, target_group_size, alpha)  # fmt: skip


def _backward_meta(grad, q, k, v, attn_bias) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    _check(grad.dim() == 3, "The grad should be 3D in jagged layout")
    dbias = torch.empty_like(attn_bias) if attn_bias is not None else None
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), dbias


def hstu_jagged_backward_equal_meta(grad, q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0,
                                    silu_scale=0.0, seq_offset=None, num_context=None, num_target=None,
                                    target_group_size=0, alpha=1.0):  # fmt: skip
    return _backward_meta(grad, q, k, v, attn_bias)


def hstu_jagged_backward_delta_meta(grad, q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0,
                                    max_seq_len_k=0, silu_scale=0.0, seq_offset=None, seq_offset_k=None,
                                    num_context=None, num_target=None, target_group_size=0, alpha=1.0):  # fmt: skip
    return _backward_meta(grad, q, k, v, attn_bias)


_DENSE_OFFSETS: dict = {}


def _dense_offsets(batch: int, s_len: int, dev) -> torch.Tensor:
    """``0, S, 2S, ..`` (batch + 1 values, int32) on ``dev``: the offsets of a dense batch, built once per shape (a
    layer calls with one shape step after step; the tensor is only ever read)."""
    key = (batch, s_len, dev)
    offs = _DENSE_OFFSETS.get(key)
    if offs is None:
        if len(_DENSE_OFFSETS) >= 64:
            _DENSE_OFFSETS.clear()
        offs = torch.arange(0, (batch + 1) * max(s_len, 1), max(s_len, 1), dtype=torch.int32, device=dev)[: batch + 1]
        _DENSE_OFFSETS[key] = offs
    return offs


def hstu_dense(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, silu_scale=0.0):
    """Dense ``[B, S, N, D]`` forward (torch_extension/hstu_dense_plugin.cpp:19-40): every sequence has the full
    length S, no alpha (1.0), no context / target arguments.  Served by the jagged kernel on a view
    ``[B * S, N, D]`` with offsets ``0, S, 2S, ...``; output ``empty_like(q)`` as in the reference."""
    _check(q.dim() == 4, "The q should be 4D in dense layout")
    _check(k.dim() == 4 and v.dim() == 4, "The k and v should be 4D in dense layout")
    _max_seq_len_check(int(max_seq_len), "maxSeqLen")
    _mask_check(int(mask_type), mask is not None)
    batch, s_q, s_k = q.size(0), q.size(1), k.size(1)
    _check(k.size(0) == batch and v.size(0) == batch and v.size(1) == s_k, "Q, K, V batch / sequence shapes mismatch")
    real_scale = (1.0 / float(max_seq_len)) if float(silu_scale) == 0.0 else float(silu_scale)
    qc, kc, vc = q.contiguous(), k.contiguous(), v.contiguous()
    dev = qc.device
    offs_q = _dense_offsets(batch, s_q, dev)
    offs_k = offs_q if s_k == s_q else _dense_offsets(batch, s_k, dev)
    if batch == 0 or s_q == 0:
        return torch.empty((batch, s_q, q.size(2), v.size(3)), dtype=_out_dtype(qc), device=dev)
    out = _forward_impl(qc.view(batch * s_q, q.size(2), q.size(3)), kc.view(batch * s_k, k.size(2), k.size(3)),
                        vc.view(batch * s_k, v.size(2), v.size(3)), mask, attn_bias, mask_type, max(s_q, 1), max(s_k, 1),
                        real_scale, offs_q, offs_k, None, None, 0, 1.0)  # fmt: skip
    return out.view(batch, s_q, q.size(2), v.size(3))


def hstu_dense_meta(q, k, v, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, silu_scale=0.0):
    _check(q.dim() == 4, "The q should be 4D in dense layout")
    return torch.empty((q.size(0), q.size(1), q.size(2), v.size(3)), dtype=_out_dtype(q), device=q.device)


def hstu_paged(q, k, v, kv_cache=None, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, max_seq_len_k=0,
               silu_scale=0.0, seq_offset=None, seq_offset_k=None, seq_offset_t=None, page_offsets=None, page_ids=None,
               last_page_len=None, num_target=None, target_group_size=0, alpha=1.0, deterministic=False):  # fmt: skip
    """Forward with a paged KV cache (torch_extension/hstu_paged_plugin.cpp:21-69): the keys / values of a sequence
    are its cached rows (pages of ``kv_cache`` [num_pages, 2, page_size, N_k, D]) followed by the rows of its
    ``num_target`` new tokens, taken from the end of its segment of ``k`` / ``v``.  ``seq_offset_k`` describes the
    resulting key ranges.  Same checks and argument normalisation as the reference adapter; output like ``q``."""
    for name, t in (("kv_cache", kv_cache), ("page_ids", page_ids), ("last_page_len", last_page_len)):
        _check(t is not None and t.numel() > 0, f"{name} must be a non-empty tensor")
    _check(seq_offset is not None and seq_offset_k is not None and seq_offset_t is not None and page_offsets is not None,
           "seq_offset, seq_offset_k, seq_offset_t and page_offsets are required")  # fmt: skip
    _check(q.dim() == 3, "The q should be 3D in jagged layout")
    for name, t in (("acSeqOffsetq", seq_offset), ("acSeqOffsetK", seq_offset_k), ("acSeqOffsetT", seq_offset_t)):
        _check(t.dim() == 1 and t.size(0) >= 2, f"{name} params error should have at least two element.")
    _check(num_target is None or int(target_group_size) > 0,
           "targetGroupSize must be greater than 0 when numTarget is defined")  # fmt: skip
    _check(k.dim() == 3 and v.dim() == 3, "The k and v should be 3D in jagged layout")
    # the new key / value rows of a sequence are read at the row indices of its query segment
    _check(k.size(0) == q.size(0) and v.size(0) == q.size(0),
           f"k and v must hold one row per row of q ({q.size(0)}), but have {k.size(0)} and {v.size(0)}")  # fmt: skip
    _check(q.device.type == "cuda", f"q must be a GPU tensor, but it is on {q.device}")
    _check_devices(q.device, (("kv_cache", kv_cache), ("seq_offset_t", seq_offset_t), ("page_offsets", page_offsets),
                              ("page_ids", page_ids), ("last_page_len", last_page_len)))  # fmt: skip
    _check(kv_cache.dim() == 5 and kv_cache.size(1) == 2, "kv_cache must be [num_pages, 2, page_size, heads, dim]")
    _check(kv_cache.dtype == q.dtype, "kv_cache must have the dtype of q")
    _check(kv_cache.size(3) == k.size(1) and kv_cache.size(4) == k.size(2) and v.size(2) == k.size(2),
           "kv_cache rows must have the heads and head dim of k and v")  # fmt: skip
    idx_dtype = seq_offset.dtype
    cache = kv_cache.contiguous()
    p_offs = page_offsets.to(idx_dtype).contiguous()
    p_ids = page_ids.to(idx_dtype).contiguous()
    last_len = last_page_len.to(idx_dtype).contiguous()
    offs_t = seq_offset_t.to(idx_dtype).contiguous()
    _check(p_offs.dim() == 1 and p_offs.size(0) == seq_offset.size(0), "page_offsets must have the length of seq_offset")
    prepared = prepare_forward(q, k, v, mask, attn_bias, mask_type, max_seq_len, max_seq_len_k, silu_scale, seq_offset,
                               seq_offset_k, None, num_target, target_group_size, alpha, deterministic)  # fmt: skip
    if prepared.out.numel() == 0:
        return prepared.out
    pp = _native.PagedParams()
    pp.struct_size = ctypes.sizeof(_native.PagedParams)
    pp.fwd = prepared.params
    # an upper bound on the end of the key ranges that needs no device read: every page full plus every input row
    pp.fwd.total_k = p_ids.numel() * cache.size(2) + q.size(0)
    pp.kv_cache, pp.page_offsets, pp.page_ids = _ptr(cache), _ptr(p_offs), _ptr(p_ids)
    pp.last_page_len, pp.seq_offset_t = _ptr(last_len), _ptr(offs_t)
    pp.num_pages, pp.page_size, pp.n_page_ids = cache.size(0), cache.size(2), p_ids.numel()
    lib = _native.load()
    ws_bytes = ctypes.c_uint64(0)
    rc = lib.hstu_paged_fwd_workspace_size(ctypes.byref(pp), ctypes.byref(ws_bytes))
    if rc != _native.HSTU_OK:
        raise RuntimeError(f"hstu_paged_fwd_workspace_size failed ({rc}): {_native.last_error()}")
    ws = torch.empty(max(ws_bytes.value, 1), dtype=torch.uint8, device=q.device)
    stream = torch.cuda.current_stream(q.device).cuda_stream
    rc = lib.hstu_paged_fwd(ctypes.byref(pp), _ptr(ws), ws_bytes.value, ctypes.c_void_p(stream))
    if rc != _native.HSTU_OK:
        raise RuntimeError(f"hstu_paged_fwd failed ({rc}): {_native.last_error()}")
    return prepared.out


def hstu_paged_meta(q, k, v, kv_cache=None, mask=None, attn_bias=None, mask_type=0, max_seq_len=0, max_seq_len_k=0,
                    silu_scale=0.0, seq_offset=None, seq_offset_k=None, seq_offset_t=None, page_offsets=None,
                    page_ids=None, last_page_len=None, num_target=None, target_group_size=0, alpha=1.0,
                    deterministic=False):  # fmt: skip
    _check(q.dim() == 3, "The q should be 3D in jagged layout")
    return torch.empty_like(q)


def hstu_dense_backward(grad, q, k, v, mask, attn_bias, mask_type=0, max_seq_len=0, silu_scale=0.0):
    """Gradients of ``hstu_dense`` (torch_extension/hstu_dense_plugin.cpp:41-151): equal shapes for grad, q, k, v
    ([B, S, N, D], seqLen == maxSeqLen), alpha 1, served by the jagged backward on the [B * S, N, D] views.  When
    there is no attn_bias the reference returns a zero placeholder with the sequence length rounded up to 256;
    so does this."""
    _check(grad.dim() == 4, "The grad should be 4D in normal layout")
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check(t.dim() == 4, f"The {name} should be 4D in normal layout")
        _check(t.shape == grad.shape, f"Q and {name.upper() if name != 'q' else 'grad'} batch size check failed")
        _check(t.dtype == grad.dtype, f"grad dtype should be the same as {name} dtype, but got grad: {grad.dtype} and {name}: {t.dtype}")
    _check(grad.dtype in (torch.float16, torch.float32, torch.bfloat16),
           f"float16, float32 or bfloat16 tensor expected but got a tensor with dtype: {grad.dtype}")  # fmt: skip
    batch, s_len, heads, dim = grad.shape
    _check(1 <= batch <= 2048, f"batchSize expect in [1, 2048], but value is {batch}")
    _check(1 <= s_len <= _MAX_SEQ_LEN, f"seqLen expect in [1, 20480], but value is {s_len}")
    _check(1 <= heads <= 16, f"headNum expect in [1, 16], but value is {heads}")
    _check(16 <= dim <= 512, f"headDim expect in [16, 512], but value is {dim}")
    _max_seq_len_check(int(max_seq_len), "maxSeqLen")
    _mask_check(int(mask_type), mask is not None)
    plane = (batch, heads, s_len, s_len)
    for name, t in (("mask", mask if int(mask_type) == 3 else None), ("attnBias", attn_bias)):
        if t is not None:
            _check(t.dim() == 4 and tuple(t.shape) == plane, f"The {name} should be {plane}")
            _check(t.dtype == grad.dtype, f"{name} dtype should be the same as grad dtype, but got {name}: {t.dtype} and grad: {grad.dtype}")
    _check(s_len == int(max_seq_len), "seqLen must be equal to maxSeqLen")
    dev = grad.device
    offs = _dense_offsets(batch, s_len, dev)
    flat = lambda t: t.contiguous().view(batch * s_len, heads, dim)  # noqa: E731
    dq, dk, dv, dbias = _backward_impl(flat(grad), flat(q), flat(k), flat(v), mask, attn_bias, mask_type, s_len, s_len,
                                       silu_scale, offs, offs, None, None, 0, 1.0)  # fmt: skip
    if dbias is None:
        padded = (s_len + 255) // 256 * 256
        dbias = torch.zeros((batch, heads, padded, padded), dtype=grad.dtype, device=dev)
    return dq.view(grad.shape), dk.view(grad.shape), dv.view(grad.shape), dbias


def hstu_dense_backward_meta(grad, q, k, v, mask, attn_bias, mask_type=0, max_seq_len=0, silu_scale=0.0):
    _check(grad.dim() == 4, "The grad should be 4D in normal layout")
    if attn_bias is not None:
        dbias = torch.empty_like(attn_bias)
    else:
        padded = (grad.size(1) + 255) // 256 * 256
        dbias = grad.new_empty((grad.size(0), grad.size(2), padded, padded))
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), dbias


_lib_cuda.impl("hstu_dense_backward", hstu_dense_backward)
_lib_meta.impl("hstu_dense_backward", hstu_dense_backward_meta)
_lib_cuda.impl("hstu_paged", hstu_paged)
_lib_meta.impl("hstu_paged", hstu_paged_meta)
_lib_cuda.impl("hstu_dense", hstu_dense)
_lib_meta.impl("hstu_dense", hstu_dense_meta)
_lib_cuda.impl("hstu_jagged.equal", hstu_jagged_equal)
_lib_cuda.impl("hstu_jagged.delta", hstu_jagged_delta)
_lib_cuda.impl("hstu_jagged_backward.equal", hstu_jagged_backward_equal)
_lib_cuda.impl("hstu_jagged_backward.delta", hstu_jagged_backward_delta)
_lib_meta.impl("hstu_jagged.equal", hstu_jagged_equal_meta)
_lib_meta.impl("hstu_jagged.delta", hstu_jagged_delta_meta)
_lib_meta.impl("hstu_jagged_backward.equal", hstu_jagged_backward_equal_meta)
_lib_meta.impl("hstu_jagged_backward.delta", hstu_jagged_backward_delta_meta)
