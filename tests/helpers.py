"""Shared input builders for the tests (seeded, CPU)."""

from __future__ import annotations

import numpy as np
import torch

from ops_rec import workloads


def set_switch(monkeypatch, name, value):
    """Sets (``value`` a string) or unsets (None) one of the library's ``HSTU_MI355_*`` switches for the rest of the
    test: the library reads its switches from the environment once per process, so it is told to read them again.
    (``tests/conftest.py`` has it read them once more when the test's environment has been put back.)"""
    from ops_rec import _native

    if value is None:
        monkeypatch.delenv(name, raising=False)
    else:
        monkeypatch.setenv(name, value)
    _native.reload_switches()


def poison_workspace(monkeypatch):
    """The backward's workspace is handed out holding NaN in every element, so that a read of something never
    written shows in the gradients.  Returns the list to which the sizes asked for are appended."""
    from ops_rec import _ops

    plain = _ops._new_workspace
    asked = []

    def poisoned(n_bytes, device):
        asked.append(n_bytes)
        ws = plain(n_bytes, device)
        if ws is not None:
            ws.fill_(0xFF)
        return ws

    monkeypatch.setattr(_ops, "_new_workspace", poisoned)
    return asked


def withhold_workspace(monkeypatch):
    """The backward gets no workspace, as when the device has no room for it: the call must work without."""
    from ops_rec import _ops

    monkeypatch.setattr(_ops, "_new_workspace", lambda n_bytes, device: None)


def small_case(seed=0, batch=3, heads=2, dim=32, lo=1, hi=40, dtype=torch.float32, std=1.0, rab=False, custom_mask=False,
               ctx=0, max_target=0, group=0, heads_k=None, dim_v=None, delta=False, index_dtype=torch.int32,
               alpha=None):  # fmt: skip
    """A small jagged batch; with ``delta`` the K/V sequences are longer than the Q sequences."""
    w = workloads.make("t", batch=batch, heads=heads, dim=dim, lo=lo, hi=hi, dtype=dtype, std=std,
                       rab_std=(0.5 if rab else None), num_context=ctx, max_target=max_target,
                       target_group_size=group, heads_k=heads_k, dim_v=dim_v, index_dtype=index_dtype, seed=seed,
                       alpha=alpha)  # fmt: skip
    g = torch.Generator().manual_seed(seed + 7)
    if delta:
        extra = torch.randint(0, 9, (len(w.lengths),), generator=g).tolist()
        len_k = [a + b for a, b in zip(w.lengths, extra)]
        total_k = sum(len_k)
        hk = heads_k or heads
        w.k = (torch.randn(total_k, hk, dim, generator=g) * std).to(dtype)
        w.v = (torch.randn(total_k, hk, dim_v or dim, generator=g) * std).to(dtype)
        offs = [0]
        for n in len_k:
            offs.append(offs[-1] + n)
        w.seq_offset_k = torch.tensor(offs, dtype=index_dtype)
        w.max_seq_len_k = max(len_k)
        if rab:
            w.attn_bias = (torch.randn(len(len_k), heads, w.max_seq_len, w.max_seq_len_k, generator=g) * 0.5).to(dtype)
    if custom_mask:
        mk = w.max_seq_len_k if w.max_seq_len_k is not None else w.max_seq_len
        w.mask = torch.randint(0, 2, (len(w.lengths), heads, w.max_seq_len, mk), generator=g).to(dtype)
        w.mask_type = 3
    return w


def reference_style_case(batch, heads, max_len, dim, dtype, *, enable_bias=False, silu_scale=0.0, mask_type=0,
                         group=0, ctx=0, tgt=0, heads_k=None, dim_v=None, min_len=1, repeat_offset=False,
                         index_dtype=torch.int32, delta=False, alpha=1.0, seed=0):  # fmt: skip
    """Inputs with the distributions of the reference's forward tests: q/k/v ~ U(-1, 1), bias ~ U(0, 1),
    lengths uniform in [min_len, max_len] (+ context + targets for the built-in mask), every sequence with the
    same num_context / num_target, a 0/1 random tensor as custom mask, max_seq_len = the longest sequence
    (hstu_forward_v1/test/pytest/test_hstu_jagged.py:41-104 and :755-800 for the delta form)."""
    g = torch.Generator().manual_seed(seed)
    heads_k = heads_k or heads
    dim_v = dim_v or dim
    lens = torch.randint(min_len, max_len + 1, (batch,), generator=g)
    if mask_type == 0:
        lens = lens + ctx + tgt
    lens_k = lens.clone()
    if delta:
        lens_k = lens + (torch.rand(batch, generator=g) * (int(lens.max()) - lens + 1)).long()
    lq, lk = lens.tolist(), lens_k.tolist()
    max_q, max_k = max(lq), max(lk)

    def offs(ls):
        o = [0]
        for n in ls:
            o.append(o[-1] + n)
        return o

    oq, ok = offs(lq), offs(lk)
    u = lambda *s: (torch.rand(*s, generator=g) * 2 - 1).to(dtype)  # noqa: E731
    q, k, v = u(oq[-1], heads, dim), u(ok[-1], heads_k, dim), u(ok[-1], heads_k, dim_v)
    bias = torch.rand(batch, heads, max_q, max_k, generator=g).to(dtype) if enable_bias else None
    mask = None
    if mask_type == 3:
        mask = torch.randint(0, 2, (batch, heads, max_q, max_k), generator=g).to(dtype)
    n_ctx = torch.full((batch,), ctx, dtype=index_dtype)
    n_tgt = torch.full((batch,), tgt, dtype=index_dtype)
    if repeat_offset:
        oq, ok = oq + oq[-1:], ok + ok[-1:]
        n_ctx, n_tgt = torch.cat([n_ctx, n_ctx[-1:]]), torch.cat([n_tgt, n_tgt[-1:]])
        if bias is not None:
            bias = torch.cat([bias, bias[-1:]])
        if mask is not None:
            mask = torch.cat([mask, mask[-1:]])
    return workloads.Workload(
        name="ref-style", q=q, k=k, v=v, seq_offset=torch.tensor(oq, dtype=index_dtype), max_seq_len=max_q,
        silu_scale=silu_scale, alpha=alpha, attn_bias=bias, mask=mask, mask_type=mask_type, num_context=n_ctx,
        num_target=n_tgt, target_group_size=group,
        seq_offset_k=(torch.tensor(ok, dtype=index_dtype) if delta else None), max_seq_len_k=(max_k if delta else None),
        lengths=lq,
    )  # fmt: skip


def paged_case(hist, prev, targets, page_size, heads=2, heads_k=None, dim=32, dtype=torch.float32, std=1.0, seed=0,
               index_dtype=torch.int32, shuffle_pages=True, spare_pages=2):
    """Inputs of ``hstu_paged`` in the way the reference's test builds them
    (hstu_forward_v1/test/pytest/test_hstu_paged.py:274-330): per sequence ``hist[b]`` new history tokens and
    ``targets[b]`` target tokens are the query rows; the cache holds ``prev[b] + hist[b]`` rows in pages of
    ``page_size``; physical pages are numbered in a shuffled order with unused spare pages in between."""
    g = torch.Generator().manual_seed(seed)
    heads_k = heads_k or heads
    batch = len(hist)
    q_lens = [h + t for h, t in zip(hist, targets)]
    k_lens = [p + h + t for p, h, t in zip(prev, hist, targets)]
    total = sum(q_lens)
    rnd = lambda *shape: (torch.randn(*shape, generator=g) * std).to(dtype)  # noqa: E731
    q, k, v = rnd(total, heads, dim), rnd(total, heads_k, dim), rnd(total, heads_k, dim)
    cached = [p + h for p, h in zip(prev, hist)]
    pages_per_seq = [(c + page_size - 1) // page_size for c in cached]
    n_pages = sum(pages_per_seq) + spare_pages
    order = torch.randperm(n_pages, generator=g).tolist() if shuffle_pages else list(range(n_pages))
    kv_cache = rnd(n_pages, 2, page_size, heads_k, dim)
    page_ids = order[: sum(pages_per_seq)]
    offs = lambda ls: torch.tensor([0] + list(np.cumsum(ls)), dtype=index_dtype)  # noqa: E731
    last = [c % page_size if c % page_size else (page_size if c else 0) for c in cached]
    return dict(
        q=q, k=k, v=v, kv_cache=kv_cache, seq_offset=offs(q_lens), seq_offset_k=offs(k_lens),
        seq_offset_t=offs(targets), page_offsets=offs(pages_per_seq), page_ids=torch.tensor(page_ids, dtype=index_dtype),
        last_page_len=torch.tensor(last, dtype=index_dtype), num_target=torch.tensor(targets, dtype=index_dtype),
        max_seq_len=max(q_lens), max_seq_len_k=max(k_lens),
    )  # fmt: skip
