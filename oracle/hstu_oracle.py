"""CPU oracle for HSTU jagged attention forward.  TEST INFRASTRUCTURE ONLY.

Nothing under ``oracle/`` is part of the shipped operator: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The product path (``ops_rec`` + the HIP
library) never routes through this file.

What it restates (reference files are cited per function; nothing is imported
from the reference and no reference source text is reproduced):

* per sequence ``b`` and head ``h``::

      S = Q_b,h @ K_b,g(h)^T                      g(h) = h // (N_q // N_k)
      X = alpha * (S + attn_bias[b, h, :S_q, :S_k])
      P = silu(X) * silu_scale * M_b              silu_scale == 0 -> 1 / max_seq_len
      O_b,h = P @ V_b,g(h)

* the built-in mask ``M_b`` of ``mask_type == 0`` (lower triangle aligned to the
  bottom-right corner, optional context rows, optional grouped target block),
  ``mask_type == 2`` (no mask) and ``mask_type == 3`` (dense custom mask
  multiplied in).

How each function is pinned (none of them by retyping its own formula):

* ``builtin_mask``          -- against ``builtin_mask_pointwise`` (an independent
  per-point statement that follows the device-side description of the mask) and
  against special cases that reduce to ``tril`` / block-diagonal ``tril``.
* ``hstu_jagged_forward``   -- against the scalar C restatement
  (``hstu_bruteforce.c``: triple loop, double accumulation, ``exp`` from libm),
  against ``torch.nn.functional.silu`` + ``torch.einsum`` on the dense-padded
  path (``hstu_jagged_forward_dense``), and against invariants (linearity in V,
  permutation of sequences, GQA == explicit repeat, delta with S_k == S_q ==
  equal, a repeated trailing offset changes nothing, rab == 0 == no rab).
* ``hstu_jagged_forward_dense`` -- against ``hstu_jagged_forward``.
* ``emulate_lowp`` mode      -- rounding points are read from the reference test
  (see the function); it is only used to apply the reference's own
  "double benchmark" acceptance rule, never as the primary check.

* ``paged_keys_values`` / ``hstu_paged_forward`` -- against a scalar restatement of the
  paged golden's own mask sentence (history columns: lower triangle; target columns:
  identity) written with explicit loops over pages and rows, and against invariance
  under a renumbering of the physical pages (``tests/test_oracle_paged.py``).

The reference holds no stored golden vectors for this path (its tests compare an
NPU run with a golden computed on the fly), so there is nothing to load.
"""

from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch
import torch.nn.functional as F

MASK_TRIL = 0
MASK_TRIU = 1
MASK_NONE = 2
MASK_CUSTOM = 3


# --------------------------------------------------------------------------- #
# masks
# --------------------------------------------------------------------------- #


def builtin_mask(
    s_q: int,
    s_k: Optional[int] = None,
    num_context: int = 0,
    num_target: int = 0,
    target_group_size: int = 0,
) -> np.ndarray:
    """Closed-form mask of ``mask_type == 0`` as a ``[s_q, s_k]`` float32 0/1 array.

    Follows ascendc/attention/hstu_v1/hstu_forward_v1/test/pytest/common.py:118-137:
    lower triangle with diagonal offset ``s_k - s_q``; if ``num_context > 0`` the
    first ``num_context`` rows see every key before the target block; if
    ``num_target > 0`` and ``target_group_size > 0`` the bottom-right
    ``num_target x num_target`` block is replaced by "causal AND same group".
    """
    if s_k is None:
        s_k = s_q
    num_context = int(num_context or 0)
    num_target = int(num_target or 0)
    target_group_size = int(target_group_size or 0)
    rows = np.arange(s_q)[:, None]
    cols = np.arange(s_k)[None, :]
    m = (cols <= rows + (s_k - s_q)).astype(np.float32)
    if num_context > 0:
        m[:num_context, : max(s_k - num_target, 0)] = 1.0
    if target_group_size > 0 and num_target > 0:
        t = num_target
        ti = np.arange(t)[:, None]
        tj = np.arange(t)[None, :]
        blk = ((tj <= ti) & (ti // target_group_size == tj // target_group_size)).astype(np.float32)
        # python slicing semantics of m[-t:, -t:] when t exceeds a dimension: clipped window
        rq = min(t, s_q)
        rk = min(t, s_k)
        m[s_q - rq :, s_k - rk :] = blk[t - rq :, t - rk :]
    return m


def builtin_mask_pointwise(
    s_q: int,
    s_k: Optional[int] = None,
    num_context: int = 0,
    num_target: int = 0,
    target_group_size: int = 0,
) -> np.ndarray:
    """Per-point statement of the same mask, written from the device-side rules.

    Follows ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/
    hstu_dense_causal_mask.h:186-260 (context rows fill ``[0, s_k - num_target)``,
    causal rows fill ``[0, i + s_k - s_q]``, a target row ``i`` with
    ``n = (i - (s_q - num_target)) // g`` full groups above it loses the columns
    ``[s_k - num_target, s_k - num_target + n * g)``).  Deliberately a slow
    double loop with no shared code with ``builtin_mask``.
    """
    if s_k is None:
        s_k = s_q
    c = int(num_context or 0)
    t = int(num_target or 0)
    g = int(target_group_size or 0)
    out = np.zeros((s_q, s_k), dtype=np.float32)
    delta = s_k - s_q
    tbase_q = s_q - t
    tbase_k = s_k - t
    for i in range(s_q):
        for j in range(s_k):
            vis = j <= i + delta
            if c > 0 and i < c and j < tbase_k:
                vis = True
            if t > 0 and g > 0 and i >= tbase_q and i >= 0:
                groups_above = (i - tbase_q) // g
                if groups_above >= 1 and tbase_k <= j < tbase_k + groups_above * g:
                    vis = False
            out[i, j] = 1.0 if vis else 0.0
    return out


def mask_nnz(s_q: int, s_k: int, num_context: int = 0, num_target: int = 0, target_group_size: int = 0) -> int:
    """Number of visible (i, j) pairs of the built-in mask (the FLOP model's nnz)."""
    return int(builtin_mask(s_q, s_k, num_context, num_target, target_group_size).sum())


# --------------------------------------------------------------------------- #
# helpers
# --------------------------------------------------------------------------- #


def effective_batch(seq_offset: Sequence[int]) -> int:
    """Index of the first offset equal to the last one (trailing repeats are dropped sequences).

    Follows .../op_kernel/atlas950/hstu_common_const.h:124-147.
    """
    offs = [int(x) for x in seq_offset]
    last = offs[-1]
    for i, o in enumerate(offs):
        if o == last:
            return i
    return len(offs) - 1


def resolve_silu_scale(silu_scale: float, max_seq_len: int) -> float:
    """``0.0`` means ``1 / max_seq_len`` (torch_extension/hstu_jagged_plugin.cpp:61)."""
    return (1.0 / float(max_seq_len)) if float(silu_scale) == 0.0 else float(silu_scale)


def _round_to(x: torch.Tensor, dtype: Optional[torch.dtype]) -> torch.Tensor:
    if dtype is None or dtype == torch.float32 or dtype == torch.float64:
        return x
    return x.to(dtype).to(x.dtype)


def _as_list(x) -> list:
    if x is None:
        return None
    if isinstance(x, torch.Tensor):
        return [int(v) for v in x.detach().cpu().tolist()]
    return [int(v) for v in x]


# --------------------------------------------------------------------------- #
# forward, per-sequence form
# --------------------------------------------------------------------------- #


def hstu_jagged_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: Optional[torch.Tensor] = None,
    attn_bias: Optional[torch.Tensor] = None,
    mask_type: int = 0,
    max_seq_len: int = 0,
    max_seq_len_k: Optional[int] = None,
    silu_scale: float = 0.0,
    seq_offset=None,
    seq_offset_k=None,
    num_context=None,
    num_target=None,
    target_group_size: int = 0,
    alpha: float = 1.0,
    *,
    compute_dtype: torch.dtype = torch.float32,
    emulate_lowp: Optional[torch.dtype] = None,
    out_dtype: Optional[torch.dtype] = None,
    _p_hook=None,
) -> torch.Tensor:
    """Per-sequence restatement of the jagged forward (CPU).

    Loop structure, bias slicing ``attn_bias[b, :, :S_q, :S_k]`` and the delta
    diagonal follow .../hstu_forward_v1/test/pytest/common.py:189-252; the
    position of ``alpha`` (after the bias add, before SiLU) and the GQA
    ``repeat_interleave`` follow .../hstu_v2/test/pytest/backend/
    pytorch_native_backend.py:48-86.

    ``emulate_lowp=torch.bfloat16`` (or float16) additionally rounds S and P to
    that type, the rounding points of the reference's low-precision golden
    (.../test_hstu_jagged.py:168-198); accumulation stays in ``compute_dtype``.
    Rows of sequences dropped by a repeated trailing offset stay zero
    (torch_extension/hstu_jagged_plugin.cpp:56-59).
    """
    if seq_offset is None:
        raise ValueError("seq_offset is required")
    offs_q = _as_list(seq_offset)
    offs_k = _as_list(seq_offset_k) if seq_offset_k is not None else offs_q
    ctx = _as_list(num_context)
    tgt = _as_list(num_target)
    if max_seq_len_k is None:
        max_seq_len_k = max_seq_len
    scale = resolve_silu_scale(silu_scale, max_seq_len)
    alpha = 1.0 if alpha is None else float(alpha)
    g = int(target_group_size or 0)

    n_q, n_k = q.shape[1], k.shape[1]
    if n_q % n_k != 0:
        raise ValueError("num heads of q must be a multiple of num heads of k")
    ratio = n_q // n_k
    d_v = v.shape[2]
    if out_dtype is None:
        out_dtype = torch.float16 if q.dtype == torch.float8_e4m3fn else q.dtype

    cd = compute_dtype
    qf, kf, vf = q.to(cd), k.to(cd), v.to(cd)
    out = torch.zeros(q.shape[0], n_q, d_v, dtype=cd)
    batch = effective_batch(offs_q)
    for b in range(batch):
        q0, q1 = offs_q[b], offs_q[b + 1]
        k0, k1 = offs_k[b], offs_k[b + 1]
        s_q, s_k = q1 - q0, k1 - k0
        if s_q <= 0:
            continue
        qb = qf[q0:q1]  # [s_q, n_q, d]
        kb = kf[k0:k1].repeat_interleave(ratio, dim=1)  # [s_k, n_q, d]
        vb = vf[k0:k1].repeat_interleave(ratio, dim=1)
        s = torch.einsum("nhd,mhd->hnm", qb, kb)  # [n_q, s_q, s_k]
        s = _round_to(s, emulate_lowp)
        if attn_bias is not None:
            s = s + attn_bias[b, :, :s_q, :s_k].to(cd)
        x = s * alpha
        p = x * torch.sigmoid(x) * scale
        if mask_type == MASK_CUSTOM:
            if mask is None:
                raise ValueError("mask_type 3 needs a mask tensor")
            p = p * mask[b, :, :s_q, :s_k].to(cd)
        elif mask_type == MASK_TRIL:
            m = builtin_mask(s_q, s_k, ctx[b] if ctx else 0, tgt[b] if tgt else 0, g)
            p = p * torch.from_numpy(m).to(cd)[None]
        elif mask_type != MASK_NONE:
            raise ValueError(f"unsupported mask_type {mask_type}")
        p = _round_to(p, emulate_lowp)
        if _p_hook is not None:  # the fp8 definition re-quantises P here
            p = _p_hook(p).to(cd)
        out[q0:q1] = torch.einsum("hnm,mhd->nhd", p, vb)
    return out.to(out_dtype)


# --------------------------------------------------------------------------- #
# forward with fp8-e4m3 inputs and per-head scales
# --------------------------------------------------------------------------- #

E4M3_MAX = 448.0


def quantize_e4m3(x: torch.Tensor) -> torch.Tensor:
    """Round to nearest even onto OCP e4m3fn after clamping to +-448 (the format has no infinity)."""
    return x.clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)


def quantize_per_head(x: torch.Tensor):
    """``x[T, H, d]`` -> (e4m3 tensor, ``descale[H]``) with ``descale = absmax / 448`` per head, the
    quantisation the fp8 workload is defined with."""
    absmax = x.abs().amax(dim=(0, 2)).clamp_min(1e-12).float()
    descale = absmax / E4M3_MAX
    return quantize_e4m3(x.float() / descale[None, :, None]), descale


def hstu_jagged_forward_fp8(
    q8: torch.Tensor,
    k8: torch.Tensor,
    v8: torch.Tensor,
    q_descale: Optional[torch.Tensor],
    k_descale: Optional[torch.Tensor],
    v_descale: Optional[torch.Tensor],
    *,
    quantize_p: bool = True,
    scaled_p: bool = False,
    out_dtype: torch.dtype = torch.float16,
    **kwargs,
) -> torch.Tensor:
    """fp8 forward, on CPU in fp32.  ``scaled_p=True`` is the reference's definition,
    ``P = e4m3(silu(X) * silu_scale * M)`` (hstu_forward_v1/test/pytest/test_hstu_jagged.py:183-195: the golden
    multiplies by silu_scale and the mask, then casts to float8_e4m3fn and back); ``scaled_p=False`` is this
    build's own variant described below.  attn_bias and a custom mask, when given, are e4m3 tensors used as fp32
    values (they follow q's type in the reference, op_host/hstu_jagged_forward.cpp:65-66).

    The reference's fp8 path takes raw e4m3 Q / K / V, keeps S in fp32, re-quantises P to e4m3
    (round to nearest) and accumulates P.V in fp32 into a half output
    (.../hstu_dense_forward_kernel_patten_bsnd.h:76, 279, 453-459, 643-646;
    torch_extension/hstu_jagged_plugin.cpp:53-54).  Two things are added here: per-head
    dequantisation scales (``x = x8 * descale[head]``; ``None`` = 1) and the place of the
    re-quantisation, which is BEFORE ``silu_scale`` is applied: the reference quantises
    ``silu(X) * silu_scale``, which with the default ``silu_scale = 1 / max_seq_len`` lies below
    e4m3's smallest normal number.  With ``silu_scale = 1`` and no scales the two definitions
    coincide.  ``quantize_p=False`` gives the unrounded result on the de-quantised inputs.

    Not pinned by any reference artefact (the reference's fp8 tests are disabled,
    .../test_hstu_jagged.py:687-689): parity unpinned beyond the fp32 formula it shares with
    ``hstu_jagged_forward``, which the checks of that function cover.
    """
    n_q, n_k = q8.shape[1], k8.shape[1]
    one_q, one_k = torch.ones(n_q), torch.ones(n_k)
    qs = one_q if q_descale is None else q_descale.float().cpu()
    ks = one_k if k_descale is None else k_descale.float().cpu()
    vs = one_k if v_descale is None else v_descale.float().cpu()
    qf = q8.float() * qs[None, :, None]
    kf = k8.float() * ks[None, :, None]
    scale = resolve_silu_scale(kwargs.get("silu_scale", 0.0), kwargs["max_seq_len"])
    kw = dict(kwargs)
    kw["silu_scale"] = scale if scaled_p else 1.0  # own variant: P is formed (and rounded) unscaled
    for name in ("attn_bias", "mask"):
        if kw.get(name) is not None:
            kw[name] = kw[name].float()
    # V enters unscaled so that P (e4m3) x V (e4m3) is what is accumulated; its scale goes on the output
    out = hstu_jagged_forward(
        qf, kf, v8.float(), compute_dtype=torch.float32,
        emulate_lowp=None, out_dtype=torch.float32, _p_hook=(quantize_e4m3 if quantize_p else None), **kw,
    )  # fmt: skip
    ratio = n_q // n_k
    out = out * ((1.0 if scaled_p else scale) * vs.repeat_interleave(ratio))[None, :, None]
    return out.to(out_dtype)


# --------------------------------------------------------------------------- #
# forward, dense-padded form (the reference's "PyTorch CPU golden path")
# --------------------------------------------------------------------------- #


def hstu_jagged_forward_dense(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: Optional[torch.Tensor] = None,
    attn_bias: Optional[torch.Tensor] = None,
    mask_type: int = 0,
    max_seq_len: int = 0,
    max_seq_len_k: Optional[int] = None,
    silu_scale: float = 0.0,
    seq_offset=None,
    seq_offset_k=None,
    num_context=None,
    num_target=None,
    target_group_size: int = 0,
    alpha: float = 1.0,
    *,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """Dense-padded restatement: pad to ``[B, H, S, d]``, two einsums, un-pad.

    This is the shape of computation of .../hstu_v2/test/pytest/backend/
    pytorch_native_backend.py:48-86 with the pad / un-pad of
    .../backend/common.py:20-41.  The reference golden receives the mask as a
    dense tensor; here it is built from the same closed form for ``mask_type 0``.
    Timed by ``bench.py`` as the CPU baseline.
    """
    offs_q = _as_list(seq_offset)
    offs_k = _as_list(seq_offset_k) if seq_offset_k is not None else offs_q
    ctx = _as_list(num_context)
    tgt = _as_list(num_target)
    if max_seq_len_k is None:
        max_seq_len_k = max_seq_len
    scale = resolve_silu_scale(silu_scale, max_seq_len)
    alpha = 1.0 if alpha is None else float(alpha)
    g = int(target_group_size or 0)
    batch = effective_batch(offs_q)
    n_q, n_k = q.shape[1], k.shape[1]
    ratio = n_q // n_k
    d_qk, d_v = q.shape[2], v.shape[2]
    cd = compute_dtype

    qd = torch.zeros(batch, max_seq_len, n_q, d_qk, dtype=cd)
    kd = torch.zeros(batch, max_seq_len_k, n_k, d_qk, dtype=cd)
    vd = torch.zeros(batch, max_seq_len_k, n_k, d_v, dtype=cd)
    md = None
    if mask_type == MASK_TRIL:
        md = torch.zeros(batch, 1, max_seq_len, max_seq_len_k, dtype=cd)
    for b in range(batch):
        s_q, s_k = offs_q[b + 1] - offs_q[b], offs_k[b + 1] - offs_k[b]
        qd[b, :s_q] = q[offs_q[b] : offs_q[b + 1]].to(cd)
        kd[b, :s_k] = k[offs_k[b] : offs_k[b + 1]].to(cd)
        vd[b, :s_k] = v[offs_k[b] : offs_k[b + 1]].to(cd)
        if md is not None and s_q > 0:
            m = builtin_mask(s_q, s_k, ctx[b] if ctx else 0, tgt[b] if tgt else 0, g)
            md[b, 0, :s_q, :s_k] = torch.from_numpy(m).to(cd)
    qd = qd.transpose(1, 2)
    kd = kd.transpose(1, 2).repeat_interleave(ratio, dim=1)
    vd = vd.transpose(1, 2).repeat_interleave(ratio, dim=1)
    s = torch.einsum("bhxa,bhya->bhxy", qd, kd)
    if attn_bias is not None:
        s = s + attn_bias[:batch, :, :max_seq_len, :max_seq_len_k].to(cd)
    s = s * alpha
    p = F.silu(s) * scale
    if mask_type == MASK_CUSTOM:
        p = p * mask[:batch, :, :max_seq_len, :max_seq_len_k].to(cd)
    elif md is not None:
        p = p * md
    od = torch.einsum("bhxy,bhyv->bhxv", p, vd).transpose(1, 2)  # [B, S, H, d_v]
    out = torch.zeros(q.shape[0], n_q, d_v, dtype=cd)
    for b in range(batch):
        s_q = offs_q[b + 1] - offs_q[b]
        out[offs_q[b] : offs_q[b + 1]] = od[b, :s_q]
    return out


# --------------------------------------------------------------------------- #
# acceptance rules
# --------------------------------------------------------------------------- #


# --------------------------------------------------------------------------- #
# paged KV cache
# --------------------------------------------------------------------------- #


def paged_keys_values(k, v, kv_cache, seq_offset, seq_offset_k, page_offsets, page_ids, last_page_len, num_target):
    """The key / value rows the paged operator attends to, laid out by ``seq_offset_k``.

    Per sequence: its pages ``page_ids[page_offsets[b] : page_offsets[b + 1]]`` of ``kv_cache``
    [num_pages, 2, page_size, N_k, D] in order, the last one cut at ``last_page_len[b]``, followed by the last
    ``num_target[b]`` rows of its segment of ``k`` / ``v``
    (hstu_forward_v1/test/pytest/test_hstu_paged.py:234-262; common.py:270-285)."""
    offs_q, offs_k = _as_list(seq_offset), _as_list(seq_offset_k)
    p_offs, p_ids, last = _as_list(page_offsets), _as_list(page_ids), _as_list(last_page_len)
    tgt = _as_list(num_target)
    ks, vs = [], []
    for b in range(len(offs_q) - 1):
        q1 = offs_q[b + 1]
        n_pages = p_offs[b + 1] - p_offs[b]
        for j in range(n_pages):
            pid = p_ids[p_offs[b] + j]
            n = last[b] if j == n_pages - 1 else kv_cache.shape[2]
            ks.append(kv_cache[pid, 0, :n])
            vs.append(kv_cache[pid, 1, :n])
        ks.append(k[q1 - tgt[b] : q1])
        vs.append(v[q1 - tgt[b] : q1])
        got = sum(t.shape[0] for t in ks)
        assert got == offs_k[b + 1], f"sequence {b}: {got} key rows, seq_offset_k says {offs_k[b + 1]}"
    return torch.cat(ks, dim=0), torch.cat(vs, dim=0)


def hstu_paged_forward(q, k, v, kv_cache, *, seq_offset, seq_offset_k, page_offsets, page_ids, last_page_len,
                       num_target, target_group_size=1, max_seq_len, max_seq_len_k=None, silu_scale=0.0, alpha=1.0,
                       mask=None, attn_bias=None, mask_type=0, out_dtype=None, emulate_lowp=None):  # fmt: skip
    """Paged forward = the jagged forward on the gathered keys / values, no context rows, grouped targets
    (torch_extension/hstu_paged_plugin.cpp:62-69 passes zeros for num_context; golden common.py:255-300)."""
    k_all, v_all = paged_keys_values(k, v, kv_cache, seq_offset, seq_offset_k, page_offsets, page_ids, last_page_len,
                                     num_target)  # fmt: skip
    return hstu_jagged_forward(q, k_all, v_all, mask=mask, attn_bias=attn_bias, mask_type=mask_type,
                               max_seq_len=max_seq_len, max_seq_len_k=max_seq_len_k, silu_scale=silu_scale,
                               seq_offset=seq_offset, seq_offset_k=seq_offset_k, num_context=None,
                               num_target=num_target, target_group_size=target_group_size, alpha=alpha,
                               out_dtype=out_dtype, emulate_lowp=emulate_lowp)  # fmt: skip


def mismatch_fraction(actual: torch.Tensor, golden: torch.Tensor, atol: float) -> float:
    """Fraction of elements with ``|diff| > atol``.

    The reference's own acceptance rule is ``mismatch_fraction(out, golden, atol) < ratio``
    with (atol, ratio) = bf16 (5e-3, 5e-3), fp16 / fp8 (1e-3, 1e-3), fp32 (1e-4, 1e-4):
    .../hstu_forward_v1/test/pytest/common.py:82-86, test_hstu_jagged.py:216-224.
    """
    a = actual.detach().double().cpu()
    g = golden.detach().double().cpu()
    return float(((a - g).abs() > atol).double().mean()) if a.numel() else 0.0


def double_benchmark_ok(actual: torch.Tensor, lowp_ref: torch.Tensor, fp32_ref: torch.Tensor, multiplier: float = 5.0):
    """``max|actual - fp32_ref| <= multiplier * max|lowp_ref - fp32_ref|`` or ``allclose(actual, lowp_ref)``.

    The second acceptance rule of the reference
    (.../hstu_v2/test/pytest/backend/pytorch_native_backend.py:198-229).
    Returns ``(passed, err_actual, err_lowp)``.
    """
    a = actual.detach().float().cpu().reshape(-1)
    lo = lowp_ref.detach().float().cpu().reshape(-1)
    hi = fp32_ref.detach().float().cpu().reshape(-1)
    if a.numel() == 0:
        return True, 0.0, 0.0
    err_a = float((a - hi).abs().max())
    err_lo = float((lo - hi).abs().max())
    ok = err_a <= multiplier * err_lo or bool(torch.allclose(a, lo))
    return ok, err_a, err_lo


# --------------------------------------------------------------------------- #
# FLOP / byte model (shared by tests and bench so both count the same thing)
# --------------------------------------------------------------------------- #


def causal_effective_flops(
    offs_q, offs_k, n_q: int, d_qk: int, d_v: int, mask_type=0, num_context=None, num_target=None, target_group_size=0
) -> int:
    """``2 * (d_qk + d_v) * n_q * sum_b nnz(M_b)``; SiLU, bias and mask work is not counted."""
    offs_q = _as_list(offs_q)
    offs_k = _as_list(offs_k) if offs_k is not None else offs_q
    ctx = _as_list(num_context)
    tgt = _as_list(num_target)
    total = 0
    for b in range(effective_batch(offs_q)):
        s_q, s_k = offs_q[b + 1] - offs_q[b], offs_k[b + 1] - offs_k[b]
        if mask_type == MASK_TRIL:
            c = ctx[b] if ctx else 0
            t = tgt[b] if tgt else 0
            if c == 0 and (t == 0 or not target_group_size):
                # closed form of the plain lower triangle with diagonal offset s_k - s_q
                d = s_k - s_q
                nnz = sum(min(max(i + d + 1, 0), s_k) for i in range(s_q))
            else:
                nnz = mask_nnz(s_q, s_k, c, t, target_group_size)
        else:
            nnz = s_q * s_k
        total += nnz
    return 2 * (d_qk + d_v) * n_q * total
