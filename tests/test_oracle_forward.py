"""Pins the oracle's forward (``hstu_oracle.hstu_jagged_forward``).

None of these checks retypes the oracle's formula: it is compared with the scalar C restatement
(triple loop, double accumulation, its own mask predicate), with the dense-padded
``F.silu`` + ``einsum`` path, with a torch-library composition on a single sequence, and with
invariants the mathematics fixes.  The reference holds no stored vectors for this path; the
closed-form inputs of its C example are used as a known-input case whose expected output is kept
as a committed fixture produced by the C restatement.
"""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import small_case
from oracle import bruteforce, hstu_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")

VARIANTS = [
    dict(),
    dict(rab=True),
    dict(rab=True, alpha=0.5),
    dict(ctx=3, max_target=6, group=2),
    dict(ctx=3, max_target=6, group=1, rab=True, alpha=0.25),
    dict(max_target=10, group=3),
    dict(ctx=50),
    dict(custom_mask=True),
    dict(custom_mask=True, rab=True),
    dict(heads=4, heads_k=2),
    dict(heads=8, heads_k=1, rab=True),
    dict(dim=16, dim_v=48),
    dict(delta=True),
    dict(delta=True, rab=True, ctx=2, max_target=4, group=2),
    dict(index_dtype=torch.int64),
]


def _oracle(w, **kw):
    return O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs(), **kw)


@pytest.mark.parametrize("variant", VARIANTS, ids=lambda v: ",".join(f"{k}={v[k]}" for k in v) or "plain")
def test_matches_scalar_c_restatement(variant):
    w = small_case(seed=3, **variant)
    got = _oracle(w)
    ref = bruteforce.forward(w.q, w.k, w.v, **w.oracle_kwargs())
    torch.testing.assert_close(got, ref, atol=2e-5, rtol=1e-4)


def test_mask_type_none_matches_c():
    w = small_case(seed=5, rab=True)
    w.mask_type = 2
    torch.testing.assert_close(_oracle(w), bruteforce.forward(w.q, w.k, w.v, **w.oracle_kwargs()), atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("variant", VARIANTS[:10], ids=lambda v: ",".join(f"{k}={v[k]}" for k in v) or "plain")
def test_dense_padded_path_agrees(variant):
    w = small_case(seed=11, **variant)
    a = _oracle(w)
    b = O.hstu_jagged_forward_dense(w.q, w.k, w.v, **w.oracle_kwargs())
    torch.testing.assert_close(a, b, atol=2e-5, rtol=1e-4)


def test_single_sequence_is_textbook_composition():
    # one sequence, one head, no bias: O = (silu(alpha Q K^T) * scale * tril) V with library routines
    torch.manual_seed(0)
    n, d = 23, 16
    q, k, v = torch.randn(n, 1, d), torch.randn(n, 1, d), torch.randn(n, 1, d)
    offs = torch.tensor([0, n], dtype=torch.int32)
    alpha, scale = 0.3, 1.0 / 64
    got = O.hstu_jagged_forward(q, k, v, max_seq_len=64, silu_scale=scale, seq_offset=offs, alpha=alpha)
    s = alpha * (q[:, 0] @ k[:, 0].T)
    ref = (F.silu(s) * scale * torch.tril(torch.ones(n, n))) @ v[:, 0]
    torch.testing.assert_close(got[:, 0], ref, atol=1e-6, rtol=1e-5)


def test_alpha_is_applied_after_the_bias_add():
    # silu(alpha * (s + b)) and silu(alpha * s + b) differ; the oracle must be the former
    w = small_case(seed=2, rab=True, alpha=0.5)
    got = _oracle(w)
    w2 = small_case(seed=2, rab=True, alpha=0.5)
    w2.attn_bias = w2.attn_bias * 2.0  # alpha * (s + b) == alpha * s + b' with b' = alpha * b, so b = 2 b' here
    w2.alpha = 1.0
    w2.q = w2.q * 0.5
    torch.testing.assert_close(got, O.hstu_jagged_forward(w2.q, w2.k, w2.v, out_dtype=torch.float32, **{**w2.oracle_kwargs(), "attn_bias": w.attn_bias * 0.5}), atol=1e-6, rtol=1e-5)


def test_silu_scale_zero_means_one_over_max_seq_len():
    w = small_case(seed=4)
    a = _oracle(w)
    w.silu_scale = 1.0 / w.max_seq_len
    torch.testing.assert_close(a, _oracle(w), atol=0, rtol=0)


def test_zero_bias_equals_no_bias():
    w = small_case(seed=6, rab=True)
    w.attn_bias = torch.zeros_like(w.attn_bias)
    a = _oracle(w)
    w.attn_bias = None
    torch.testing.assert_close(a, _oracle(w), atol=0, rtol=0)


def test_linear_in_v():
    w = small_case(seed=7, rab=True, ctx=2, max_target=5, group=2)
    a = _oracle(w)
    w.v = w.v * 3.0
    torch.testing.assert_close(_oracle(w), a * 3.0, atol=1e-6, rtol=1e-5)


def test_gqa_equals_explicit_repeat():
    w = small_case(seed=8, heads=6, heads_k=2, rab=True)
    a = _oracle(w)
    w.k = w.k.repeat_interleave(3, dim=1)
    w.v = w.v.repeat_interleave(3, dim=1)
    torch.testing.assert_close(a, _oracle(w), atol=0, rtol=0)


def test_delta_with_equal_lengths_equals_equal():
    w = small_case(seed=9, rab=True, ctx=2, max_target=3, group=1)
    a = _oracle(w)
    w.seq_offset_k = w.seq_offset.clone()
    w.max_seq_len_k = w.max_seq_len
    torch.testing.assert_close(a, _oracle(w), atol=0, rtol=0)


def test_repeated_trailing_offset_changes_nothing():
    w = small_case(seed=10, ctx=2, max_target=3, group=1)
    a = _oracle(w)
    w.seq_offset = torch.cat([w.seq_offset, w.seq_offset[-1:]])
    w.num_context = torch.cat([w.num_context, w.num_context[-1:]])
    w.num_target = torch.cat([w.num_target, w.num_target[-1:]])
    torch.testing.assert_close(a, _oracle(w), atol=0, rtol=0)


def test_sequences_are_independent():
    # reversing the order of the sequences permutes the output blocks and nothing else
    w = small_case(seed=12, batch=4)
    a = _oracle(w)
    lens = w.lengths
    offs = w.seq_offset.tolist()
    order = list(reversed(range(len(lens))))
    pieces = lambda t: [t[offs[b] : offs[b + 1]] for b in order]  # noqa: E731
    w2 = small_case(seed=12, batch=4)
    w2.q, w2.k, w2.v = (torch.cat(pieces(t)) for t in (w.q, w.k, w.v))
    w2.seq_offset = torch.tensor([0] + list(np.cumsum([lens[b] for b in order])), dtype=torch.int32)
    b2 = _oracle(w2)
    torch.testing.assert_close(torch.cat(pieces(a)), b2, atol=0, rtol=0)


def test_more_queries_than_keys_leaves_leading_rows_zero():
    torch.manual_seed(1)
    q = torch.randn(6, 1, 8)
    k, v = torch.randn(2, 1, 8), torch.randn(2, 1, 8)
    out = O.hstu_jagged_forward(q, k, v, max_seq_len=6, max_seq_len_k=2, seq_offset=torch.tensor([0, 6]),
                                seq_offset_k=torch.tensor([0, 2]))  # fmt: skip
    assert torch.count_nonzero(out[:4]) == 0 and torch.count_nonzero(out[4:]) > 0


def test_lowp_emulation_is_close_to_fp32():
    w = small_case(seed=13, dtype=torch.bfloat16, std=0.5)
    hi = _oracle(w)
    lo = _oracle(w, emulate_lowp=torch.bfloat16)
    assert (hi - lo).abs().max() < 2e-2
    ok, err_a, err_lo = O.double_benchmark_ok(lo, lo, hi)
    assert ok and err_a == err_lo


def test_known_input_example_matches_fixture():
    # inputs of the reference's C example: q[i] = (i % 3) / 3, k[i] = (i % 5) / 5, v[i] = (i % 7) / 7,
    # q offsets {0, 4, 10}, k offsets {0, 6, 14}, 4 heads, dim 32, mask_type 0, scale 1 / 6
    # (hstu_forward_v1/examples/aclnn/test_aclnn_hstu_forward_jagged.cpp:52-63, 97-100)
    n, d = 4, 32
    q = (torch.arange(10 * n * d) % 3).float().div(3.0).view(10, n, d)
    k = (torch.arange(14 * n * d) % 5).float().div(5.0).view(14, n, d)
    v = (torch.arange(14 * n * d) % 7).float().div(7.0).view(14, n, d)
    oq, ok = torch.tensor([0, 4, 10], dtype=torch.int32), torch.tensor([0, 6, 14], dtype=torch.int32)
    got = O.hstu_jagged_forward(q, k, v, None, None, 0, 6, 8, 1.0 / 6, oq, ok, alpha=1.0)
    fixture = np.load(os.path.join(GOLDEN, "aclnn_example_forward.npz"))
    np.testing.assert_allclose(got.numpy(), fixture["out"], atol=1e-5, rtol=1e-5)
    # the closed-form inputs make row 0 of sequence 0 see keys 0..2 (delta = 2): check one element by hand
    s = [(q[0, 0] * k[j, 0]).sum().item() for j in range(3)]
    p = [x / (1.0 + np.exp(-x)) / 6.0 for x in s]
    expect = sum(p[j] * v[j, 0, 5].item() for j in range(3))
    assert abs(got[0, 0, 5].item() - expect) < 1e-5


@pytest.mark.parametrize("name", ["c1_fp32", "small_ctx_tgt_rab_bf16", "small_delta_gqa_f16"])
def test_golden_fixtures_reproduce(name):
    from golden import make_golden

    w = make_golden.CASES[name]()
    fixture = np.load(os.path.join(GOLDEN, f"{name}.npz"))
    got = O.hstu_jagged_forward(w.q, w.k, w.v, out_dtype=torch.float32, **w.oracle_kwargs())
    np.testing.assert_allclose(got.numpy(), fixture["out"], atol=2e-5, rtol=1e-4)


def test_flop_model():
    offs = [0, 10, 10, 35]
    assert O.causal_effective_flops(offs, None, 4, 128, 128) == 2 * 256 * 4 * (55 + 325)
    assert O.causal_effective_flops(offs, None, 2, 64, 32, mask_type=2) == 2 * 96 * 2 * (100 + 625)


# --------------------------------------------------------------------------- #
# fp8 definition (inputs e4m3 with per-head scales, P re-quantised before silu_scale)
# --------------------------------------------------------------------------- #


def test_e4m3_quantiser_known_values():
    x = torch.tensor([0.0, 1.0, -1.0, 0.3, 17.0, 18.0, 19.0, 447.0, 449.0, 1000.0, -1000.0, 0.0625, 0.001])
    got = O.quantize_e4m3(x).float()
    # 3 mantissa bits: spacing 2 between 16 and 32 (ties to even), 0.03125 between 0.25 and 0.5; no infinity: clamp to 448
    want = torch.tensor([0.0, 1.0, -1.0, 0.3125, 16.0, 18.0, 20.0, 448.0, 448.0, 448.0, -448.0, 0.0625, 0.001953125])
    assert torch.equal(got, want)


def _fp8_case(seed=0, heads=4, heads_k=2, d=32, dv=16):
    g = torch.Generator().manual_seed(seed)
    lengths = [7, 33, 1, 20]
    total = sum(lengths)
    offs = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    q8, qs = O.quantize_per_head(torch.randn(total, heads, d, generator=g))
    k8, ks = O.quantize_per_head(torch.randn(total, heads_k, d, generator=g))
    v8, vs = O.quantize_per_head(torch.randn(total, heads_k, dv, generator=g))
    kw = dict(mask_type=0, max_seq_len=40, silu_scale=0.0, seq_offset=offs, alpha=d**-0.5)
    return (q8, k8, v8), (qs, ks, vs), kw


def test_fp8_unrounded_equals_generic_forward_on_dequantised_inputs():
    (q8, k8, v8), (qs, ks, vs), kw = _fp8_case()
    got = O.hstu_jagged_forward_fp8(q8, k8, v8, qs, ks, vs, quantize_p=False, out_dtype=torch.float32, **kw)
    deq = lambda x8, s: x8.float() * s[None, :, None]  # noqa: E731
    want = O.hstu_jagged_forward(deq(q8, qs), deq(k8, ks), deq(v8, vs), out_dtype=torch.float32, **kw)
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-5)


def test_fp8_scale_algebra():
    (q8, k8, v8), (qs, ks, vs), kw = _fp8_case(seed=3)
    base = O.hstu_jagged_forward_fp8(q8, k8, v8, qs, ks, vs, out_dtype=torch.float32, **kw)
    # the V scale is applied to the fp32 output: a power of two passes through exactly
    twice = O.hstu_jagged_forward_fp8(q8, k8, v8, qs, ks, vs * 2, out_dtype=torch.float32, **kw)
    assert torch.equal(twice, base * 2)
    # a uniform q scale is the same as a factor on alpha (powers of two: exact)
    kw2 = dict(kw, alpha=kw["alpha"] * 4.0)
    moved = O.hstu_jagged_forward_fp8(q8, k8, v8, qs / 4, ks, vs, out_dtype=torch.float32, **kw2)
    assert torch.equal(moved, base)
    # P is rounded before silu_scale: changing silu_scale by a power of two only scales the result
    kw3 = dict(kw, silu_scale=1.0 / 8)
    kw4 = dict(kw, silu_scale=1.0 / 64)
    a = O.hstu_jagged_forward_fp8(q8, k8, v8, qs, ks, vs, out_dtype=torch.float32, **kw3)
    b = O.hstu_jagged_forward_fp8(q8, k8, v8, qs, ks, vs, out_dtype=torch.float32, **kw4)
    assert torch.equal(a, b * 8)


def test_fp8_reduces_to_the_reference_definition_without_scales_and_silu_scale_one():
    # reference: P = rint_e4m3(silu(X) * silu_scale * M), S and the accumulation in fp32, half output
    (q8, k8, v8), _, kw = _fp8_case(seed=5)
    kw = dict(kw, silu_scale=1.0)
    got = O.hstu_jagged_forward_fp8(q8, k8, v8, None, None, None, out_dtype=torch.float16, **kw)
    want = O.hstu_jagged_forward(q8.float(), k8.float(), v8.float(), out_dtype=torch.float16,
                                 _p_hook=O.quantize_e4m3, **kw)  # fmt: skip
    assert torch.equal(got, want)


def test_fp8_reference_rounding_point_is_the_reference_golden_on_one_sequence():
    # scaled_p=True against the lines of the reference's own fp8 golden, written out with library calls for one
    # sequence (hstu_forward_v1/test/pytest/test_hstu_jagged.py:160-198): qk + bias, * alpha, silu, * silu_scale,
    # * mask, cast to float8_e4m3fn and back, matmul with V; GQA by repeating the K/V heads
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(9)
    s_len, heads, heads_k, d = 37, 4, 2, 32
    q8, k8, v8 = (torch.randn(s_len, n, d, generator=g).to(torch.float8_e4m3fn) for n in (heads, heads_k, heads_k))
    bias = (torch.randn(1, heads, s_len, s_len, generator=g) * 0.5).to(torch.float8_e4m3fn)
    mask = (torch.rand(1, heads, s_len, s_len, generator=g) < 0.6).float().to(torch.float8_e4m3fn)
    offs = torch.tensor([0, s_len], dtype=torch.int32)
    for silu_scale in (1.0, 0.25, 1.0 / s_len):
        qk = torch.einsum("nhd,mhd->hnm", q8.float(), k8.float().repeat_interleave(heads // heads_k, dim=1))
        p = F.silu((qk + bias[0].float()) * 0.3) * silu_scale * mask[0].float()
        p = p.to(torch.float8_e4m3fn).float()
        want = torch.einsum("hnm,mhd->nhd", p, v8.float().repeat_interleave(heads // heads_k, dim=1))
        got = O.hstu_jagged_forward_fp8(q8, k8, v8, None, None, None, scaled_p=True, out_dtype=torch.float32, mask=mask,
                                        attn_bias=bias, mask_type=3, max_seq_len=s_len, silu_scale=silu_scale,
                                        seq_offset=offs, alpha=0.3)  # fmt: skip
        torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
        own = O.hstu_jagged_forward_fp8(q8, k8, v8, None, None, None, scaled_p=False, out_dtype=torch.float32, mask=mask,
                                        attn_bias=bias, mask_type=3, max_seq_len=s_len, silu_scale=silu_scale,
                                        seq_offset=offs, alpha=0.3)  # fmt: skip
        if silu_scale == 1.0:
            torch.testing.assert_close(own, want, atol=1e-5, rtol=1e-5)  # the two rounding points coincide
        else:
            assert not torch.allclose(own, want, atol=1e-4, rtol=1e-3)
