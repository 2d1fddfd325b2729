"""``ops_rec.ascendc.attention.hstu_paged`` on the GPU (page gather kernel + jagged forward through the C ABI) against
the CPU oracle on the same seeded inputs; cases follow the reference's paged tests
(hstu_forward_v1/test/pytest/test_hstu_paged.py:333-420: page sizes 32..256, full and partial last pages, rows cached
before the request, grouped heads) and its example (examples/torch/test_torch_hstu_forward_paged.py:34-100).
Tolerance: the forward's (atol = rtol = 1e-2 for bf16 / fp16, 1e-4 for fp32)."""

import pytest
import torch

import ops_rec
from helpers import paged_case
from oracle import hstu_oracle as O
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NAMES = ("seq_offset", "seq_offset_k", "page_offsets", "page_ids", "last_page_len", "num_target")


def run_op(c, group=1, alpha=1.0, silu_scale=0.0, **kw):
    d = {n: (t.to(DEV) if torch.is_tensor(t) else t) for n, t in c.items()}
    out = ops_rec.ascendc.attention.hstu_paged(
        d["q"], d["k"], d["v"], d["kv_cache"], mask=kw.get("mask"), attn_bias=kw.get("attn_bias"),
        mask_type=kw.get("mask_type", 0), max_seq_len=c["max_seq_len"], max_seq_len_k=c["max_seq_len_k"],
        silu_scale=silu_scale, seq_offset=d["seq_offset"], seq_offset_k=d["seq_offset_k"], seq_offset_t=d["seq_offset_t"],
        page_offsets=d["page_offsets"], page_ids=d["page_ids"], last_page_len=d["last_page_len"],
        num_target=d["num_target"], target_group_size=group, alpha=alpha)  # fmt: skip
    torch.cuda.synchronize()
    return out


def check(c, group=1, alpha=1.0, silu_scale=0.0, **kw):
    out = run_op(c, group, alpha, silu_scale, **kw)
    assert out.shape == c["q"].shape and out.dtype == c["q"].dtype
    cpu_kw = {n: (t.cpu() if torch.is_tensor(t) else t) for n, t in kw.items()}
    ref = O.hstu_paged_forward(c["q"], c["k"], c["v"], c["kv_cache"], out_dtype=torch.float32, target_group_size=group,
                               alpha=alpha, silu_scale=silu_scale, max_seq_len=c["max_seq_len"],
                               max_seq_len_k=c["max_seq_len_k"], **{n: c[n] for n in NAMES}, **cpu_kw)  # fmt: skip
    tol = 1e-4 if c["q"].dtype == torch.float32 else 1e-2
    torch.testing.assert_close(out.float().cpu(), ref, atol=tol, rtol=tol)
    return out


def test_reference_example_shape():
    # N 4, D 32, page 32, histories 32 (exactly one page) and 48 (last page half full), 4 and 6 targets
    c = paged_case(hist=[32, 48], prev=[0, 0], targets=[4, 6], page_size=32, heads=4, dim=32, dtype=torch.float16, seed=1)
    check(c, silu_scale=1.0 / 54)


@pytest.mark.parametrize("page_size", [32, 64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
def test_page_sizes_and_dtypes(page_size, dtype):
    c = paged_case(hist=[300, 1, 256, 77], prev=[0, 0, 0, 0], targets=[10, 3, 1, 40], page_size=page_size, heads=2,
                   dim=64, dtype=dtype, std=0.5, seed=page_size)  # fmt: skip
    check(c, alpha=0.125)


@pytest.mark.parametrize("group", [1, 3, 64])
def test_rows_cached_before_the_request_and_target_groups(group):
    c = paged_case(hist=[120, 64, 200], prev=[500, 64, 1], targets=[30, 7, 12], page_size=64, heads=4, heads_k=2, dim=128,
                   dtype=torch.bfloat16, std=0.3, seed=group, index_dtype=torch.int64)  # fmt: skip
    check(c, group=group, alpha=128**-0.5)


@pytest.mark.parametrize("dim,page_size", [(256, 128), (192, 32), (256, 256), (160, 64)])
@pytest.mark.parametrize("with_bias", [False, True], ids=["plain", "bias"])
def test_head_dims_of_the_slot_256_read_the_pages_themselves(dim, page_size, with_bias):
    """Head dims above 128 have a paged kernel variant as well (they were gathered into contiguous rows first): rows cached
    before the request, partial last pages, grouped heads, with and without attn_bias on the paged keys."""
    c = paged_case(hist=[140, 64, 33], prev=[700, 0, 130], targets=[12, 7, 40], page_size=page_size, heads=4, heads_k=2,
                   dim=dim, dtype=torch.bfloat16, std=0.3, seed=dim + page_size)  # fmt: skip
    if with_bias:
        g = torch.Generator().manual_seed(3)
        bias = (torch.randn(3, 4, c["max_seq_len"], c["max_seq_len_k"], generator=g) * 0.3).to(torch.bfloat16)
        check(c, attn_bias=bias.to(DEV), alpha=dim**-0.5)
    else:
        check(c, alpha=dim**-0.5)


def test_attn_bias_and_custom_mask_on_paged_keys():
    c = paged_case(hist=[90, 150], prev=[40, 0], targets=[5, 9], page_size=32, heads=2, dim=64, dtype=torch.float16,
                   std=0.5, seed=9)  # fmt: skip
    g = torch.Generator().manual_seed(2)
    shape = (2, 2, c["max_seq_len"], c["max_seq_len_k"])
    bias = (torch.randn(shape, generator=g) * 0.3).to(torch.float16)
    check(c, attn_bias=bias.to(DEV))
    mask = (torch.rand(shape, generator=g) < 0.5).to(torch.float16)
    check(c, mask=mask.to(DEV), mask_type=3)


def test_physical_page_order_does_not_matter():
    a = paged_case(hist=[400, 130], prev=[0, 260], targets=[8, 2], page_size=128, dim=64, dtype=torch.bfloat16, std=0.5,
                   seed=5, shuffle_pages=False)  # fmt: skip
    perm = torch.randperm(a["kv_cache"].shape[0], generator=torch.Generator().manual_seed(6))
    b = dict(a)
    b["kv_cache"] = torch.empty_like(a["kv_cache"])
    b["kv_cache"][perm] = a["kv_cache"]
    b["page_ids"] = perm[a["page_ids"].long()].to(a["page_ids"].dtype)
    assert torch.equal(check(a), check(b))


def test_argument_checks():
    c = paged_case(hist=[40], prev=[0], targets=[2], page_size=32, dim=32, dtype=torch.float16)
    d = {n: (t.to(DEV) if torch.is_tensor(t) else t) for n, t in c.items()}
    args = dict(mask=None, attn_bias=None, mask_type=0, max_seq_len=42, max_seq_len_k=42, silu_scale=0.0,
                seq_offset=d["seq_offset"], seq_offset_k=d["seq_offset_k"], seq_offset_t=d["seq_offset_t"],
                page_offsets=d["page_offsets"], page_ids=d["page_ids"], last_page_len=d["last_page_len"],
                num_target=d["num_target"], target_group_size=1)  # fmt: skip
    with pytest.raises(RuntimeError, match="targetGroupSize must be greater than 0"):
        ops_rec.ascendc.attention.hstu_paged(d["q"], d["k"], d["v"], d["kv_cache"], **dict(args, target_group_size=0))
    with pytest.raises(RuntimeError, match="page_ids must be a non-empty tensor"):
        ops_rec.ascendc.attention.hstu_paged(d["q"], d["k"], d["v"], d["kv_cache"], **dict(args, page_ids=d["page_ids"][:0]))
    odd = d["kv_cache"][:, :, :31].contiguous()  # page size 31
    with pytest.raises(RuntimeError, match="page_size must be 32, 64, 128 or 256"):
        ops_rec.ascendc.attention.hstu_paged(d["q"], d["k"], d["v"], odd, **args)
    with pytest.raises(RuntimeError, match="maxSeqLen"):
        ops_rec.ascendc.attention.hstu_paged(d["q"], d["k"], d["v"], d["kv_cache"], **dict(args, max_seq_len=0))


def test_long_cache_few_query_rows(monkeypatch):
    # the serving shape: a handful of new rows per sequence against thousands of cached ones.  Few items, long
    # sweeps: the key ranges are split over workgroups; without splitting the result is the same to the last rounding
    c = paged_case(hist=[40, 3], prev=[6000, 2500], targets=[16, 50], page_size=256, heads=4, heads_k=2, dim=128,
                   dtype=torch.bfloat16, std=0.3, seed=21)  # fmt: skip
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "1")
    split = check(c, alpha=128**-0.5)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")
    whole = check(c, alpha=128**-0.5)
    torch.testing.assert_close(split.float(), whole.float(), atol=2e-7, rtol=2.0**-7)
