"""GPU parity of the fp8-e4m3 forward (configuration C5's arithmetic) against the CPU oracle.

The reference's own fp8 tests are disabled (.../hstu_forward_v1/test/pytest/test_hstu_jagged.py:687-689)
and hold no vectors, so the checks are against this build's oracle:
  * with P re-quantised to e4m3 as the kernel does: atol 1e-3, rtol 1e-2 (what is left is the order of the
    fp32 accumulation and the rounding of the 16-bit output);
  * against the unrounded fp32 result on the de-quantised inputs, the stated tolerance of the fp8 path:
    max |error| <= 4 % of max |reference| + 1e-4 (e4m3 keeps 3 mantissa bits of P).
"""

import pytest
import torch

import ops_rec
from ops_rec import workloads
from oracle import hstu_oracle as O
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(t):
    return None if t is None else t.to(DEV)


def make_case(batch, heads, heads_k, d, dv, lo, hi, seed, scales=True, std=0.5, extra_len=0):
    # as in the reference's tests, context and target tokens come on top of the drawn history length
    lengths = (torch.randint(lo, hi + 1, (batch,), generator=torch.Generator().manual_seed(seed)) + extra_len).tolist()
    w = workloads.make("t", dtype=torch.float32, batch=batch, heads=heads, heads_k=heads_k, dim=d, dim_v=dv, lo=lo,
                       hi=hi, std=std, seed=seed, lengths=lengths)  # fmt: skip
    if scales:
        (q8, qs), (k8, ks), (v8, vs) = (O.quantize_per_head(t) for t in (w.q, w.k, w.v))
    else:
        q8, k8, v8 = (O.quantize_e4m3(t) for t in (w.q, w.k, w.v))
        qs = ks = vs = None
    return w, (q8, k8, v8), (qs, ks, vs)


def check(out, x8, sc, kw):
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    ref_q = O.hstu_jagged_forward_fp8(*x8, *sc, quantize_p=True, out_dtype=torch.float32, **kw)
    ref_u = O.hstu_jagged_forward_fp8(*x8, *sc, quantize_p=False, out_dtype=torch.float32, **kw)
    torch.testing.assert_close(got, ref_q, atol=1e-3, rtol=1e-2)
    assert (got - ref_u).abs().max() <= 0.04 * ref_u.abs().max() + 1e-4


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("ctx,tgt,group,mask_type", [(0, 0, 0, 0), (6, 30, 3, 0), (0, 30, 1, 0), (0, 0, 0, 2)])
@pytest.mark.parametrize("batch,heads,heads_k,d,dv,lo,hi", [
    (2, 2, 2, 128, 128, 5, 40), (3, 4, 4, 128, 128, 100, 300), (3, 4, 2, 128, 64, 100, 300),
    (3, 2, 2, 64, 64, 100, 300), (2, 2, 1, 256, 256, 100, 300), (4, 2, 2, 32, 48, 1, 130), (16, 4, 4, 128, 128, 1, 1024),
])  # fmt: skip
def test_fp8_forward_matrix(batch, heads, heads_k, d, dv, lo, hi, ctx, tgt, group, mask_type, out_dtype):
    w, x8, sc = make_case(batch, heads, heads_k, d, dv, lo, hi, seed=batch * 17 + d, extra_len=ctx + tgt)
    nctx = torch.full((batch,), ctx, dtype=torch.int32) if ctx else None
    ntgt = torch.full((batch,), tgt, dtype=torch.int32) if tgt else None
    kw = dict(mask_type=mask_type, max_seq_len=w.max_seq_len, silu_scale=0.0, seq_offset=w.seq_offset,
              num_context=nctx, num_target=ntgt, target_group_size=group, alpha=d**-0.5)  # fmt: skip
    kwd = dict(kw, seq_offset=dev(w.seq_offset), num_context=dev(nctx), num_target=dev(ntgt))
    out = ops_rec.hstu_jagged_fp8(*(dev(t) for t in x8), *(dev(t) for t in sc), out_dtype=out_dtype, **kwd)
    assert out.dtype == out_dtype
    check(out, x8, sc, kw)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("ctx,tgt,group,mask_type", [(0, 0, 0, 0), (6, 30, 3, 0), (0, 0, 0, 2)])
@pytest.mark.parametrize("batch,heads,heads_k,d,dv,lo,hi", [
    (2, 2, 2, 512, 512, 60, 200), (2, 4, 2, 320, 272, 60, 200), (3, 2, 2, 24, 16, 1, 130), (2, 2, 1, 72, 80, 40, 200),
    (2, 2, 2, 1, 16, 5, 40), (2, 2, 2, 264, 64, 100, 140),
])  # fmt: skip
def test_fp8_head_dims_beyond_the_tuned_kernels(batch, heads, heads_k, d, dv, lo, hi, ctx, tgt, group, mask_type, out_dtype):
    """Everything the reference's tiling admits for its fp8 target -- any q/k head dim in [1, 512], v head dims up
    to 512 in steps of 16 (op_host/tiling_policy.cpp:68-93, dtype list op_host/atlas950/op_def_arch.h:23-24) -- runs:
    head dims above 256 and q/k head dims that are not multiples of 16 on the coverage kernel's e4m3 instantiation."""
    w, x8, sc = make_case(batch, heads, heads_k, d, dv, lo, hi, seed=batch * 13 + d, extra_len=ctx + tgt)
    nctx = torch.full((batch,), ctx, dtype=torch.int32) if ctx else None
    ntgt = torch.full((batch,), tgt, dtype=torch.int32) if tgt else None
    kw = dict(mask_type=mask_type, max_seq_len=w.max_seq_len, silu_scale=0.0, seq_offset=w.seq_offset,
              num_context=nctx, num_target=ntgt, target_group_size=group, alpha=d**-0.5)  # fmt: skip
    kwd = dict(kw, seq_offset=dev(w.seq_offset), num_context=dev(nctx), num_target=dev(ntgt))
    out = ops_rec.hstu_jagged_fp8(*(dev(t) for t in x8), *(dev(t) for t in sc), out_dtype=out_dtype, **kwd)
    assert out.dtype == out_dtype
    check(out, x8, sc, kw)


@pytest.mark.parametrize("d,dv", [(512, 512), (40, 48)])
def test_fp8_beyond_the_tuned_kernels_reference_rounding_point_bias_and_mask(d, dv):
    """The reference's entry point with e4m3 tensors (no scales, fp16 output, P rounded after silu_scale and the
    mask) with an e4m3 attn_bias and custom mask, at head dims the coverage kernel takes."""
    w, x8, _ = make_case(2, 2, 2, d, dv, 20, 90, seed=d, scales=False, std=1.0)
    g = torch.Generator().manual_seed(d + 1)
    shape = (2, 2, w.max_seq_len, w.max_seq_len)
    bias = O.quantize_e4m3(torch.randn(shape, generator=g) * 0.5)
    mask = O.quantize_e4m3(torch.randint(0, 2, shape, generator=g).float())
    for mask_type, m in ((0, None), (3, mask)):
        kw = dict(mask_type=mask_type, max_seq_len=w.max_seq_len, silu_scale=0.25, seq_offset=w.seq_offset, alpha=d**-0.5,
                  attn_bias=bias, mask=m)  # fmt: skip
        out = ops_rec.ascendc.attention.hstu_jagged(dev(x8[0]), dev(x8[1]), dev(x8[2]), dev(m), dev(bias), mask_type,
                                                   w.max_seq_len, 0.25, dev(w.seq_offset), None, None, 0, d**-0.5)  # fmt: skip
        assert out.dtype == torch.float16
        want = O.hstu_jagged_forward_fp8(*x8, None, None, None, scaled_p=True, out_dtype=torch.float32, **kw)
        torch.testing.assert_close(out.float().cpu(), want, atol=2e-3, rtol=1e-2)


def test_reference_entry_point_with_e4m3_tensors_gives_half_output():
    # the reference's fp8 call: raw e4m3 tensors through hstu_jagged, no scales, fp16 out
    # (torch_extension/hstu_jagged_plugin.cpp:53-54); with silu_scale 1 the rounding point makes no difference
    w, x8, _ = make_case(3, 2, 2, 128, 128, 10, 200, seed=11, scales=False, std=1.0)
    out = ops_rec.ascendc.attention.hstu_jagged(*(dev(t) for t in x8), None, None, 0, w.max_seq_len, 1.0,
                                                dev(w.seq_offset), None, None, 0, 128**-0.5)  # fmt: skip
    assert out.dtype == torch.float16
    kw = dict(mask_type=0, max_seq_len=w.max_seq_len, silu_scale=1.0, seq_offset=w.seq_offset, alpha=128**-0.5)
    want = O.hstu_jagged_forward(x8[0].float(), x8[1].float(), x8[2].float(), out_dtype=torch.float32,
                                 _p_hook=O.quantize_e4m3, **kw)  # fmt: skip
    # unscaled inputs make P large, where one e4m3 step is up to 6 % of a term: an element of P that sits on a
    # rounding boundary may fall the other way in the kernel (hardware exp2 / rcp) than in the oracle, so the
    # comparison is by fraction of outliers plus a bound on the largest one
    got = out.float().cpu()
    peak = want.abs().max().item()
    assert O.mismatch_fraction(got, want, 2e-3 * peak) < 5e-3, (peak, (got - want).abs().max().item())
    assert (got - want).abs().max() <= 0.05 * peak


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("d", [64, 128])
def test_p_beyond_the_e4m3_range_saturates(d, out_dtype):
    # scores in the thousands: silu(x) ~ x lies far beyond +-448, the largest e4m3 value; the rounded P must be
    # +-448 there (as the oracle's quantiser clamps), never NaN.  Half of the keys give large negative scores (P ~ 0).
    g = torch.Generator().manual_seed(d)
    lengths = [70, 33]
    total = sum(lengths)
    sign = torch.where(torch.arange(total) % 2 == 0, 1.0, -1.0).view(total, 1, 1)
    q8 = O.quantize_e4m3(torch.full((total, 2, d), 16.0))
    k8 = O.quantize_e4m3(torch.full((total, 2, d), 16.0) * sign)
    v8 = O.quantize_e4m3(torch.randn(total, 2, d, generator=g) * 0.25)
    offs = torch.tensor([0, 70, 103], dtype=torch.int32)
    kw = dict(mask_type=0, max_seq_len=70, silu_scale=1.0, seq_offset=offs, alpha=1.0)
    out = ops_rec.hstu_jagged_fp8(dev(q8), dev(k8), dev(v8), None, None, None, out_dtype=out_dtype,
                                  **dict(kw, seq_offset=dev(offs)))  # fmt: skip
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    want = O.hstu_jagged_forward_fp8(q8, k8, v8, None, None, None, quantize_p=True, out_dtype=torch.float32, **kw)
    assert want.abs().max() > 448  # sums of saturated terms
    torch.testing.assert_close(got, want, atol=1e-2 * want.abs().max().item(), rtol=1e-2)


def test_fp8_int64_offsets_and_delta_lengths():
    # K / V longer than Q (delta form through seq_offset_k), int64 offsets
    g = torch.Generator().manual_seed(4)
    lq, lk = [5, 40, 17], [9, 64, 17]
    oq = torch.tensor([0, 5, 45, 62], dtype=torch.int64)
    ok = torch.tensor([0, 9, 73, 90], dtype=torch.int64)
    q8, qs = O.quantize_per_head(torch.randn(sum(lq), 2, 128, generator=g))
    k8, ks = O.quantize_per_head(torch.randn(sum(lk), 2, 128, generator=g))
    v8, vs = O.quantize_per_head(torch.randn(sum(lk), 2, 128, generator=g))
    kw = dict(mask_type=0, max_seq_len=64, max_seq_len_k=64, silu_scale=0.0, seq_offset=oq, seq_offset_k=ok,
              alpha=0.1)  # fmt: skip
    out = ops_rec.hstu_jagged_fp8(dev(q8), dev(k8), dev(v8), dev(qs), dev(ks), dev(vs),
                                  **dict(kw, seq_offset=dev(oq), seq_offset_k=dev(ok)))  # fmt: skip
    check(out, (q8, k8, v8), (qs, ks, vs), kw)


def test_fp8_rejections():
    w, x8, sc = make_case(2, 2, 2, 128, 128, 5, 40, seed=1)
    a = [dev(t) for t in x8]
    with pytest.raises(RuntimeError, match="float32 tensor of 2 per-head scales"):
        ops_rec.hstu_jagged_fp8(*a, dev(sc[0])[:1], None, None, max_seq_len=w.max_seq_len, seq_offset=dev(w.seq_offset))
    with pytest.raises(RuntimeError, match="fp16 or bf16"):
        ops_rec.hstu_jagged_fp8(*a, max_seq_len=w.max_seq_len, seq_offset=dev(w.seq_offset), out_dtype=torch.float32)
    bias = torch.zeros(2, 2, w.max_seq_len, w.max_seq_len, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="attn_bias must have the dtype of q"):
        ops_rec.ascendc.attention.hstu_jagged(*a, None, bias, 0, w.max_seq_len, 1.0, dev(w.seq_offset))


def e4m3(t):
    return t.to(torch.float8_e4m3fn)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("enable_bias,mask_type", [(True, 0), (True, 2), (False, 3), (True, 3)])
@pytest.mark.parametrize("batch,heads,heads_k,d,dv,max_len", [
    (3, 4, 4, 128, 128, 300), (3, 4, 2, 64, 64, 257), (2, 2, 1, 256, 256, 200), (4, 2, 2, 128, 64, 131),
])  # fmt: skip
def test_fp8_with_attn_bias_and_custom_mask(batch, heads, heads_k, d, dv, max_len, enable_bias, mask_type, out_dtype):
    # attn_bias and the custom mask follow q's type in the reference (e4m3 on its fp8 target,
    # op_host/hstu_jagged_forward.cpp:65-66; bias and MaskType.CUSTOM are part of its fp8 test matrix, disabled there);
    # max_len 257 and 131 give rows that are not 4-byte aligned (the byte-load path)
    w, x8, sc = make_case(batch, heads, heads_k, d, dv, max_len // 3, max_len, seed=batch * 31 + max_len)
    g = torch.Generator().manual_seed(max_len)
    shape = (batch, heads, w.max_seq_len, w.max_seq_len)
    bias = e4m3(torch.randn(shape, generator=g) * 0.5) if enable_bias else None
    mask = e4m3((torch.rand(shape, generator=g) < 0.7).float()) if mask_type == 3 else None
    kw = dict(mask=mask, attn_bias=bias, mask_type=mask_type, max_seq_len=w.max_seq_len, silu_scale=0.0,
              seq_offset=w.seq_offset, alpha=d**-0.5)  # fmt: skip
    kwd = dict(kw, mask=dev(mask), attn_bias=dev(bias), seq_offset=dev(w.seq_offset))
    out = ops_rec.hstu_jagged_fp8(*(dev(t) for t in x8), *(dev(t) for t in sc), out_dtype=out_dtype, **kwd)
    assert out.dtype == out_dtype
    check(out, x8, sc, kw)


@pytest.mark.parametrize("d,enable_bias,mask_type", [(128, True, 0), (64, True, 3), (128, False, 3)])
def test_fp8_long_list_with_attn_bias_takes_the_queues(d, enable_bias, mask_type):
    """A list of several items per resident workgroup with an e4m3 attn_bias and / or custom mask runs on the variant with
    per-XCD queues, like one without them.  Sequences are independent: a few of them cut out and run alone (a short
    list: the plain variant) give the same bits, and those rows are compared with the oracle."""
    from ops_rec import _ops

    batch, heads, max_len = 48, 8, 1024
    g = torch.Generator(device=DEV).manual_seed(d + mask_type)
    lengths = torch.randint(300, max_len + 1, (batch,), generator=torch.Generator().manual_seed(d)).tolist()
    offs = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    total = int(offs[-1])
    x = [torch.randn(total, heads, d, generator=g, device=DEV) * 0.5 for _ in range(3)]
    x8, sc = zip(*(workloads.quantize_fp8(t) for t in x))
    shape = (batch, heads, max_len, max_len)
    bias = (torch.randn(shape, generator=g, device=DEV) * 0.5).to(torch.float8_e4m3fn) if enable_bias else None
    mask = (torch.rand(shape, generator=g, device=DEV) < 0.7).float().to(torch.float8_e4m3fn) if mask_type == 3 else None
    kw = dict(mask=mask, attn_bias=bias, mask_type=mask_type, max_seq_len=max_len, silu_scale=0.0, seq_offset=offs.to(DEV),
              alpha=d**-0.5)  # fmt: skip
    prepared = _ops.prepare_forward(*x8, mask, bias, mask_type, max_len, max_len, 0.0, kw["seq_offset"], kw["seq_offset"], None,
                                    None, 0, kw["alpha"], out_dtype=torch.bfloat16, q_descale=sc[0], k_descale=sc[1],
                                    v_descale=sc[2])  # fmt: skip
    assert prepared.kernel_name().endswith("_queues"), prepared.kernel_name()
    out = ops_rec.hstu_jagged_fp8(*x8, *sc, **kw)
    assert torch.equal(out, ops_rec.hstu_jagged_fp8(*x8, *sc, **kw))  # reproducible
    seqs = [0, 17, 40]
    o = offs.tolist()
    rows = torch.cat([torch.arange(o[b], o[b + 1]) for b in seqs]).to(DEV)
    sub_offs = torch.tensor([0] + list(torch.tensor([lengths[b] for b in seqs]).cumsum(0)), dtype=torch.int32)
    pick = lambda t: None if t is None else t[torch.tensor(seqs, device=DEV)]  # noqa: E731
    sub8 = tuple(t[rows] for t in x8)
    subkw = dict(kw, mask=pick(mask), attn_bias=pick(bias), seq_offset=sub_offs.to(DEV))
    alone = ops_rec.hstu_jagged_fp8(*sub8, *sc, **subkw)
    assert torch.equal(alone, out[rows])
    cpu = lambda t: None if t is None else t.cpu()  # noqa: E731
    check(alone, tuple(t.cpu() for t in sub8), tuple(t.cpu() for t in sc),
          dict(subkw, mask=cpu(subkw["mask"]), attn_bias=cpu(subkw["attn_bias"]), seq_offset=sub_offs))


@pytest.mark.parametrize("silu_scale", [0.0, 0.25])
def test_reference_entry_point_keeps_the_reference_rounding_point(silu_scale):
    # through hstu_jagged with raw e4m3 tensors P is quantised AFTER silu_scale and the mask, as the reference's golden
    # does (test_hstu_jagged.py:183-195); with the default silu_scale = 1 / max_seq_len most of P falls below e4m3's
    # smallest subnormal and rounds to zero there as well
    w, x8, _ = make_case(3, 2, 2, 128, 128, 40, 200, seed=23, scales=False, std=1.0)
    bias = e4m3(torch.randn(3, 2, w.max_seq_len, w.max_seq_len, generator=torch.Generator().manual_seed(2)) * 0.5)
    out = ops_rec.ascendc.attention.hstu_jagged(*(dev(t) for t in x8), None, dev(bias), 0, w.max_seq_len, silu_scale,
                                                dev(w.seq_offset), None, None, 0, 128**-0.5)  # fmt: skip
    assert out.dtype == torch.float16
    kw = dict(attn_bias=bias, mask_type=0, max_seq_len=w.max_seq_len, silu_scale=silu_scale, seq_offset=w.seq_offset,
              alpha=128**-0.5)  # fmt: skip
    want = O.hstu_jagged_forward_fp8(*x8, None, None, None, scaled_p=True, out_dtype=torch.float32, **kw)
    other = O.hstu_jagged_forward_fp8(*x8, None, None, None, scaled_p=False, out_dtype=torch.float32, **kw)
    got = out.float().cpu()
    peak = want.abs().max().item()
    assert peak > 0
    # elements of P on a rounding boundary may fall the other way in the kernel (hardware exp2 / rcp): by fraction of
    # outliers plus a bound on the largest, as in the test above
    assert O.mismatch_fraction(got, want, 2e-3 * peak + 1e-3) < 5e-3, (peak, (got - want).abs().max().item())
    assert (got - want).abs().max() <= 0.06 * peak + 1e-3
    if silu_scale == 0.0:
        # ... and it is not this build's own variant, which keeps the information the reference's order rounds away
        assert (other - want).abs().max() > 10 * (got - want).abs().max()


@pytest.fixture(scope="module")
def c5():
    w = workloads.config("C5", device=DEV)
    (q8, qs), (k8, ks), (v8, vs) = (workloads.quantize_fp8(t) for t in (w.q, w.k, w.v))
    kw = dict(mask_type=0, max_seq_len=w.max_seq_len, silu_scale=w.silu_scale, seq_offset=w.seq_offset, alpha=w.alpha)
    out = ops_rec.hstu_jagged_fp8(q8, k8, v8, qs, ks, vs, **kw)
    torch.cuda.synchronize()
    yield w, (q8, k8, v8), (qs, ks, vs), kw, out
    torch.cuda.empty_cache()


def test_c5_full_size_properties(c5):
    w, x8, sc, kw, out = c5
    assert out.dtype == torch.bfloat16 and torch.isfinite(out.float()).all()
    again = ops_rec.hstu_jagged_fp8(*x8, *sc, **kw)
    assert torch.equal(out, again)  # bitwise reproducible
    doubled = ops_rec.hstu_jagged_fp8(*x8, sc[0], sc[1], sc[2] * 2, **kw)
    assert torch.equal(doubled.float(), out.float() * 2)  # the V scale acts on the fp32 output
    assert (out.float().abs().amax(dim=(1, 2)) > 0).all()  # every row of every sequence was written


def test_c5_sub_batch_matches_oracle(c5, monkeypatch):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")  # (bit-identity with the full batch needs the same order of fp32 sums)
    w, x8, sc, kw, out = c5
    order = sorted(range(len(w.lengths)), key=lambda b: w.lengths[b])
    seqs = sorted(order[:3] + [order[len(order) * 3 // 4]])  # three shortest and one of a few hundred rows
    offs = w.seq_offset.cpu().tolist()
    rows = torch.cat([torch.arange(offs[b], offs[b + 1]) for b in seqs])
    lens = [offs[b + 1] - offs[b] for b in seqs]
    sub_offs = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=w.seq_offset.dtype)
    sub8 = tuple(t[rows.to(DEV)].cpu() for t in x8)
    subkw = dict(kw, seq_offset=sub_offs)
    alone = ops_rec.hstu_jagged_fp8(*(dev(t) for t in sub8), *sc, **dict(subkw, seq_offset=dev(sub_offs)))
    assert torch.equal(alone, out[rows.to(DEV)])  # sequences are independent
    check(alone, sub8, tuple(s.cpu() for s in sc), subkw)
