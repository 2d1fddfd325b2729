"""Short work lists (fewer items than resident workgroups): the kernel variant that cuts the key range of long
items into parts, each part swept by another workgroup, the fp32 partial outputs added up in part order by the
workgroup that completes the item.

Checked for every case: the launch reports the split variant and asks for a workspace; the result meets the parity
bar against the CPU oracle; it agrees with the same launch run without splitting (HSTU_MI355_SPLIT=0) to within the
rounding of one output element (a split changes the order of the fp32 sums, nothing else); two more launches give
the same bits again (the partial sums are added in part order whoever arrives last, and the arrival counters are
back at zero after a launch).
"""

import dataclasses

import pytest
import torch

import ops_rec
from ops_rec import _ops, workloads
from oracle import hstu_oracle as O
import helpers

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def prepare(w):
    k_offs = w.seq_offset if w.seq_offset_k is None else w.seq_offset_k
    max_k = w.max_seq_len if w.max_seq_len_k is None else w.max_seq_len_k
    return _ops.prepare_forward(w.q, w.k, w.v, w.mask, w.attn_bias, w.mask_type, w.max_seq_len, max_k, w.silu_scale,
                                w.seq_offset, k_offs, w.num_context, w.num_target, w.target_group_size, w.alpha)  # fmt: skip


def launch(p):
    out = p.launch().clone()
    torch.cuda.synchronize()
    return out


def check_split(w, monkeypatch, atol=1e-2, rtol=1e-2):
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")
    plain = prepare(w)
    assert plain.workspace_bytes == 0 and not plain.kernel_name().endswith("_split")
    want = launch(plain)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "1")
    split = prepare(w)
    assert split.workspace_bytes > 0 and split.kernel_name().endswith("_split"), split.kernel_name()
    got = launch(split)
    assert torch.isfinite(got.float()).all()
    # same numbers up to the order of the fp32 sums: at most one rounding step of the 16-bit output apart
    torch.testing.assert_close(got.float(), want.float(), atol=2e-7, rtol=2.0**-7)
    assert torch.equal(launch(split), got)
    assert torch.equal(launch(split), got)
    c = w.to("cpu")
    ref = O.hstu_jagged_forward(c.q, c.k, c.v, out_dtype=torch.float32, **c.oracle_kwargs())
    torch.testing.assert_close(got.float().cpu(), ref, atol=atol, rtol=rtol)
    return got


def test_one_long_sequence(monkeypatch):
    # 47 query tiles, up to 188 sub-tiles per item: every level above the target length is split, up to 8 parts
    w = workloads.make("long", dtype=torch.bfloat16, device=DEV, seed=3, batch=1, heads=2, dim=128, lo=6000, hi=6000)
    check_split(w, monkeypatch)


def test_few_sequences_rab_context_targets(monkeypatch):
    # rab requests and the hole of grouped targets start in the middle of the key range for parts after the first
    w = workloads.make("rab", dtype=torch.bfloat16, device=DEV, seed=4, batch=3, heads=2, dim=128, lo=300, hi=2500,
                       max_seq_len=2500, rab_std=0.5, num_context=5, max_target=50, target_group_size=3)  # fmt: skip
    check_split(w, monkeypatch)


@pytest.mark.parametrize("n_ctx,max_target,group,dim", [(40, 0, 0, 128), (8, 30, 2, 128), (33, 70, 1, 64)])
def test_context_rows_first_tile_sweeps_all_history(n_ctx, max_target, group, dim, monkeypatch):
    # with context rows the first query tile of a sequence is its longest item: it stands first in the list (and is
    # split like the top tile), and nearly all of its steps see a sub-tile whole from the context rows and not at
    # all from the others (the contexts end in the first or the second wavefront of the tile)
    w = workloads.make("ctx", dtype=torch.bfloat16, device=DEV, seed=12, batch=3, heads=2, dim=dim, lo=900, hi=2600,
                       max_seq_len=2600, num_context=n_ctx, max_target=max_target, target_group_size=group)  # fmt: skip
    check_split(w, monkeypatch)


def test_custom_mask_f16_grouped_heads(monkeypatch):
    w = workloads.make("mask", dtype=torch.float16, device=DEV, seed=5, batch=2, heads=4, heads_k=2, dim=64, lo=700,
                       hi=1800, max_seq_len=1800)  # fmt: skip
    g = torch.Generator(device=DEV).manual_seed(11)
    mask = (torch.rand(2, 4, 1800, 1800, generator=g, device=DEV) < 0.6).to(torch.float16)
    w = dataclasses.replace(w, mask=mask, mask_type=3)
    check_split(w, monkeypatch)


def test_no_mask_all_keys(monkeypatch):
    # mask_type 2: every query tile sweeps all keys, so every level is split alike
    w = workloads.make("full", dtype=torch.bfloat16, device=DEV, seed=6, batch=2, heads=2, dim=128, lo=900, hi=1500,
                       max_seq_len=1500)  # fmt: skip
    w = dataclasses.replace(w, mask_type=2)
    check_split(w, monkeypatch)


def test_more_keys_than_queries(monkeypatch):
    # delta form: 3000 cached keys + the new ones per sequence; causal diagonal shifted by S_k - S_q
    lq, lk = [700, 1200], [3700, 4200]
    g = torch.Generator(device=DEV).manual_seed(8)
    q = (torch.randn(sum(lq), 2, 128, generator=g, device=DEV) * 0.1).to(torch.bfloat16)
    k = (torch.randn(sum(lk), 2, 128, generator=g, device=DEV) * 0.1).to(torch.bfloat16)
    v = (torch.randn(sum(lk), 2, 128, generator=g, device=DEV) * 0.1).to(torch.bfloat16)
    w = workloads.Workload(
        name="delta", q=q, k=k, v=v, seq_offset=torch.tensor([0, 700, 1900], dtype=torch.int32, device=DEV),
        max_seq_len=1200, silu_scale=0.0, alpha=128**-0.5,
        seq_offset_k=torch.tensor([0, 3700, 7900], dtype=torch.int32, device=DEV), max_seq_len_k=4200, lengths=lq,
    )  # fmt: skip
    check_split(w, monkeypatch)


def test_items_much_shorter_than_nominal(monkeypatch):
    # max_seq_len far above the real lengths and no causal bound: the nominal length that decides the number of
    # parts (all of max_seq_len_k) is many times the real one, so most parts of an item are empty
    w = workloads.make("short", dtype=torch.bfloat16, device=DEV, seed=9, batch=3, heads=2, dim=128, lo=40, hi=300,
                       max_seq_len=8192)  # fmt: skip
    w = dataclasses.replace(w, mask_type=2)
    check_split(w, monkeypatch)


def test_fp8_long_sequences(monkeypatch):
    w = workloads.make("f8", dtype=torch.bfloat16, device=DEV, seed=10, batch=2, heads=2, dim=128, lo=2000, hi=5000)
    (q8, qs), (k8, ks), (v8, vs) = (workloads.quantize_fp8(t) for t in (w.q, w.k, w.v))
    kw = dict(mask_type=0, max_seq_len=w.max_seq_len, silu_scale=w.silu_scale, alpha=w.alpha, seq_offset=w.seq_offset)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "0")
    want = ops_rec.hstu_jagged_fp8(q8, k8, v8, qs, ks, vs, **kw)
    helpers.set_switch(monkeypatch, "HSTU_MI355_SPLIT", "1")
    got = ops_rec.hstu_jagged_fp8(q8, k8, v8, qs, ks, vs, **kw)
    torch.testing.assert_close(got.float(), want.float(), atol=2e-7, rtol=2.0**-7)
    assert torch.equal(ops_rec.hstu_jagged_fp8(q8, k8, v8, qs, ks, vs, **kw), got)
    ref = O.hstu_jagged_forward_fp8(q8.cpu(), k8.cpu(), v8.cpu(), qs.cpu(), ks.cpu(), vs.cpu(), out_dtype=torch.float32,
                                    mask_type=0, max_seq_len=w.max_seq_len, silu_scale=w.silu_scale, alpha=w.alpha,
                                    seq_offset=w.seq_offset.cpu())  # fmt: skip
    torch.testing.assert_close(got.float().cpu(), ref, atol=1e-2, rtol=1e-2)


def test_without_workspace_nothing_is_split():
    # a caller that ignores the workspace request is served by the plain variant: same bits as with splitting off
    w = workloads.make("nows", dtype=torch.bfloat16, device=DEV, seed=12, batch=1, heads=1, dim=128, lo=3000, hi=3000)
    p = prepare(w)
    assert p.workspace_bytes > 0
    with_ws = launch(p)
    p.workspace, p.workspace_bytes = None, 0
    without = launch(p)
    torch.testing.assert_close(with_ws.float(), without.float(), atol=2e-7, rtol=2.0**-7)
    c = w.to("cpu")
    ref = O.hstu_jagged_forward(c.q, c.k, c.v, out_dtype=torch.float32, **c.oracle_kwargs())
    torch.testing.assert_close(without.float().cpu(), ref, atol=1e-2, rtol=1e-2)
