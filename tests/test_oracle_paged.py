"""Pins the paged oracle (``oracle.hstu_oracle.hstu_paged_forward``) without the GPU.

The reference's paged golden states the mask in one sentence (hstu_forward_v1/test/pytest/common.py:262-267): a
history row i sees the history columns [0, i]; target row H + j sees all history columns and its own column H + j.
``brute`` below is that sentence with explicit loops over pages, rows and columns and Python floats -- it shares no
code with the oracle (no builtin_mask, no torch matmul) -- for the case the golden covers (no earlier cache, group 1);
the general case (rows cached before this request, larger groups) is pinned through the jagged oracle it reduces to.
"""

import math

import torch

from helpers import paged_case
from oracle import hstu_oracle as O


def brute(c, silu_scale, alpha):
    q, k, v, cache = c["q"].double(), c["k"].double(), c["v"].double(), c["kv_cache"].double()
    offs = c["seq_offset"].tolist()
    p_offs, p_ids, last = c["page_offsets"].tolist(), c["page_ids"].tolist(), c["last_page_len"].tolist()
    tgt = c["num_target"].tolist()
    heads, heads_k, dim = q.shape[1], k.shape[1], q.shape[2]
    page_size = cache.shape[2]
    out = torch.zeros(q.shape, dtype=torch.float64)
    for b in range(len(offs) - 1):
        q0, q1 = offs[b], offs[b + 1]
        s, t = q1 - q0, tgt[b]
        h_len = s - t
        keys, vals = [], []
        for j in range(p_offs[b], p_offs[b + 1]):
            n = last[b] if j == p_offs[b + 1] - 1 else page_size
            for r in range(n):
                keys.append(cache[p_ids[j], 0, r])
                vals.append(cache[p_ids[j], 1, r])
        assert len(keys) == h_len
        for r in range(q0 + h_len, q1):
            keys.append(k[r])
            vals.append(v[r])
        for i in range(s):
            for col in range(s):
                if i < h_len:
                    visible = col <= i
                else:
                    visible = col < h_len or col == i
                if not visible:
                    continue
                for hd in range(heads):
                    g = hd // (heads // heads_k)
                    x = alpha * sum(float(q[q0 + i, hd, d]) * float(keys[col][g, d]) for d in range(dim))
                    p = x / (1.0 + math.exp(-x)) * silu_scale
                    out[q0 + i, hd] += p * vals[col][g]
    return out


def run_oracle(c, **kw):
    names = ("seq_offset", "seq_offset_k", "page_offsets", "page_ids", "last_page_len", "num_target", "max_seq_len",
             "max_seq_len_k")  # fmt: skip
    return O.hstu_paged_forward(c["q"], c["k"], c["v"], c["kv_cache"], out_dtype=torch.float32,
                                **{n: c[n] for n in names}, **kw)  # fmt: skip


def test_paged_oracle_matches_the_goldens_sentence():
    # full last page, partial last page, a sequence of targets only after one cached row
    c = paged_case(hist=[32, 11, 1], prev=[0, 0, 0], targets=[3, 5, 2], page_size=32, heads=2, heads_k=1, dim=8, seed=1)
    got = run_oracle(c, silu_scale=0.25, alpha=0.5, target_group_size=1)
    torch.testing.assert_close(got.double(), brute(c, 0.25, 0.5), atol=1e-5, rtol=1e-5)


def test_renumbering_physical_pages_changes_nothing():
    a = paged_case(hist=[40, 70], prev=[30, 0], targets=[4, 1], page_size=32, dim=16, seed=2, shuffle_pages=False)
    perm = torch.randperm(a["kv_cache"].shape[0], generator=torch.Generator().manual_seed(3))
    b = dict(a)
    b["kv_cache"] = torch.empty_like(a["kv_cache"])
    b["kv_cache"][perm] = a["kv_cache"]  # page p of a is page perm[p] of b
    b["page_ids"] = perm[a["page_ids"].long()].to(a["page_ids"].dtype)
    torch.testing.assert_close(run_oracle(a, target_group_size=1), run_oracle(b, target_group_size=1), atol=0, rtol=0)


def test_rows_cached_earlier_shift_the_diagonal():
    # with rows cached before this request the operator is the "delta" form of the jagged one on the gathered rows:
    # gather by hand with plain indexing and compare
    c = paged_case(hist=[20, 33], prev=[45, 64], targets=[6, 2], page_size=64, dim=16, seed=4)
    k_all, v_all = O.paged_keys_values(c["k"], c["v"], c["kv_cache"], c["seq_offset"], c["seq_offset_k"],
                                       c["page_offsets"], c["page_ids"], c["last_page_len"], c["num_target"])  # fmt: skip
    offs_k = c["seq_offset_k"].tolist()
    assert k_all.shape[0] == offs_k[-1]
    # first sequence: 65 cached rows = one full page + 1 row of the next page, then its 6 target rows of k
    first = c["page_ids"][0].item()
    second = c["page_ids"][1].item()
    assert torch.equal(k_all[:64], c["kv_cache"][first, 0]) and torch.equal(k_all[64], c["kv_cache"][second, 0, 0])
    assert torch.equal(v_all[65:71], c["v"][20:26])
    want = O.hstu_jagged_forward(c["q"], k_all, v_all, mask_type=0, max_seq_len=c["max_seq_len"],
                                 max_seq_len_k=c["max_seq_len_k"], seq_offset=c["seq_offset"],
                                 seq_offset_k=c["seq_offset_k"], num_target=c["num_target"], target_group_size=2,
                                 out_dtype=torch.float32)  # fmt: skip
    torch.testing.assert_close(run_oracle(c, target_group_size=2), want, atol=0, rtol=0)
