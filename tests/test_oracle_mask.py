"""Pins the oracle's built-in mask (mask_type 0).

The closed form (``builtin_mask``, following the reference's test helper) is checked against two
independent statements: a per-point double loop written from the device-side rules
(``builtin_mask_pointwise``) and the predicate of the scalar C restatement.  Special cases that
reduce to textbook objects (tril, block-diagonal tril) anchor all three.
"""

import itertools

import numpy as np
import pytest

from oracle import bruteforce, hstu_oracle as O

CASES = [
    # (s_q, s_k, ctx, tgt, group) -- includes the sizes of the reference's own mask brute-force test
    # (seq 64, ctx 16, tgt 16, group 4: hstu_backward_v1/test/pytest/test_target_mask.py:260-286)
    (64, 64, 16, 16, 4),
    (64, 64, 0, 16, 1),
    (64, 64, 16, 0, 0),
    (1, 1, 0, 0, 0),
    (1, 1, 1, 1, 1),
    (7, 7, 3, 2, 5),
    (33, 33, 6, 30, 3),
    (33, 33, 6, 30, 1),
    (40, 40, 0, 30, 3),
    (16, 16, 255, 30, 1),  # context larger than the sequence (reference edge case ctx 255/256/257)
    (48, 48, 20, 47, 3),
    (20, 20, 4, 6, 0),  # group 0 switches the target rule off, context still stops before the targets
    (10, 14, 3, 4, 2),  # delta: more keys than queries
    (5, 9, 6, 3, 1),
    (12, 30, 0, 0, 0),
    (30, 12, 0, 0, 0),  # more queries than keys: the first rows see nothing
    (30, 12, 4, 3, 2),
    (4, 20, 2, 8, 3),  # more targets than query rows
]


@pytest.mark.parametrize("s_q,s_k,ctx,tgt,group", CASES)
def test_three_statements_agree(s_q, s_k, ctx, tgt, group):
    closed = O.builtin_mask(s_q, s_k, ctx, tgt, group)
    point = O.builtin_mask_pointwise(s_q, s_k, ctx, tgt, group)
    c_pred = bruteforce.mask(s_q, s_k, ctx, tgt, group)
    assert closed.shape == (s_q, s_k)
    np.testing.assert_array_equal(closed, point)
    np.testing.assert_array_equal(closed, c_pred)


def test_exhaustive_small():
    for s_q, s_k in itertools.product(range(1, 7), repeat=2):
        for ctx, tgt, group in itertools.product(range(0, 4), range(0, 4), range(0, 4)):
            if tgt > min(s_q, s_k):
                continue
            a = O.builtin_mask(s_q, s_k, ctx, tgt, group)
            np.testing.assert_array_equal(a, O.builtin_mask_pointwise(s_q, s_k, ctx, tgt, group))
            np.testing.assert_array_equal(a, bruteforce.mask(s_q, s_k, ctx, tgt, group))


@pytest.mark.parametrize("n", [1, 2, 17, 64])
def test_plain_causal_is_tril(n):
    np.testing.assert_array_equal(O.builtin_mask(n), np.tril(np.ones((n, n), dtype=np.float32)))


def test_delta_diagonal_offset():
    # with more keys than queries the triangle is aligned to the bottom-right corner
    m = O.builtin_mask(3, 5)
    np.testing.assert_array_equal(m, np.tril(np.ones((3, 5), dtype=np.float32), k=2))


def test_group_at_least_target_is_plain_causal():
    for g in (8, 9, 100):
        np.testing.assert_array_equal(O.builtin_mask(20, 20, 0, 8, g), np.tril(np.ones((20, 20), dtype=np.float32)))


def test_group_one_targets_see_history_and_self_only():
    n, t = 12, 5
    m = O.builtin_mask(n, n, 0, t, 1)
    h = n - t
    np.testing.assert_array_equal(m[:h], np.tril(np.ones((n, n), dtype=np.float32))[:h])
    np.testing.assert_array_equal(m[h:, :h], np.ones((t, h), dtype=np.float32))
    np.testing.assert_array_equal(m[h:, h:], np.eye(t, dtype=np.float32))


def test_target_block_is_block_diagonal_tril():
    n, t, g = 16, 8, 4
    blk = O.builtin_mask(n, n, 0, t, g)[n - t :, n - t :]
    expect = np.kron(np.eye(t // g), np.tril(np.ones((g, g)))).astype(np.float32)
    np.testing.assert_array_equal(blk, expect)


def test_context_rows_see_all_history_but_no_targets():
    n, c, t = 10, 3, 4
    m = O.builtin_mask(n, n, c, t, 2)
    np.testing.assert_array_equal(m[:c, : n - t], np.ones((c, n - t), dtype=np.float32))
    np.testing.assert_array_equal(m[:c, n - t :], np.zeros((c, t), dtype=np.float32))


def test_nnz_closed_form():
    # nnz of the plain triangle is L (L + 1) / 2; group 1 removes t (t - 1) / 2 pairs
    assert O.mask_nnz(37, 37) == 37 * 38 // 2
    assert O.mask_nnz(37, 37, 0, 9, 1) == 37 * 38 // 2 - 9 * 8 // 2
    # context rows add the pairs above the diagonal that stay before the target block
    n, c, t = 20, 4, 5
    extra = sum(max((n - t) - (i + 1), 0) for i in range(c))
    assert O.mask_nnz(n, n, c, t, 0) == n * (n + 1) // 2 + extra


def test_effective_batch_drops_trailing_repeats():
    assert O.effective_batch([0, 4, 10]) == 2
    assert O.effective_batch([0, 4, 10, 10]) == 2
    assert O.effective_batch([0, 4, 10, 10, 10]) == 2
    assert O.effective_batch([0, 4, 4, 10]) == 3  # an empty sequence in the middle is kept
    assert O.effective_batch([0, 0]) == 0
