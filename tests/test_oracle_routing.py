"""Pins of the routing oracle (CPU only): brute force, tie and known-answer cases."""

import numpy as np
import pytest
from scipy.special import softmax

from oracle import affine as ora
from oracle import routing as orr


def test_topk_is_the_sort_by_logit_then_id():
    rng = np.random.default_rng(0)
    l = rng.standard_normal((9, 129)).astype(np.float32)
    l[2, 5] = l[2, 90] = l[2].max() + 1                        # a tie at the top: the lower id first
    picks, wts = orr.topk_rows(l, 128, 6, shared=True)
    for r in range(9):
        want = sorted(range(128), key=lambda e: (-float(l[r, e]), e))[:6]
        assert picks[r, :6].tolist() == want and picks[r, 6] == 128
    assert picks[2, :2].tolist() == [5, 90]


def test_ties_known_answer():
    """All-equal logits select ids 0..k-1 (the reference's tests/cuda/test_nemotron_kernels.py:71-80)."""

    picks, wts = orr.topk_rows(np.zeros((3, 65), np.float32), 64, 6, shared=True)
    assert picks.tolist() == [[0, 1, 2, 3, 4, 5, 64]] * 3
    assert np.all(wts[:, :6] == ora.bf16(np.float32(1 / 6))) and np.all(wts[:, 6] == 0.5)


def test_weights_are_the_softmax_over_the_selected():
    rng = np.random.default_rng(1)
    l = rng.standard_normal((16, 513)).astype(np.float32)
    picks, wts = orr.topk_rows(l, 512, 10, shared=True)
    chosen = np.take_along_axis(l[:, :512], picks[:, :10].astype(np.int64), 1)
    want = softmax(chosen.astype(np.float64), axis=1)
    assert np.abs(wts[:, :10] - want).max() <= 2 ** -8                       # bf16-rounded
    assert np.array_equal(wts[:, :10], ora.bf16(wts[:, :10]))
    gate = 1 / (1 + np.exp(-ora.bf16(l[:, 512]).astype(np.float64)))
    assert np.abs(wts[:, 10] - gate).max() <= 2 ** -8
    p2, w2 = orr.topk_rows(l, 512, 10, shared=False)
    assert p2.shape == (16, 10) and np.array_equal(p2, picks[:, :10]) and np.array_equal(w2, wts[:, :10])


def brute_plan(picks, e, tile):
    flat = picks.reshape(-1).tolist()
    items, members = [], []
    for ex in range(e):
        pairs = [p for p, v in enumerate(flat) if v == ex]
        for j in range(0, len(pairs), tile):
            items.append([ex, len(members) + j, min(tile, len(pairs) - j)])
        members += pairs
    return items, members, len(set(flat))


@pytest.mark.parametrize("rows,tile", [(1, 16), (23, 16), (300, 64), (1500, 16), (700, 128)])
def test_plan_against_brute_force(rows, tile):
    rng = np.random.default_rng(rows)
    picks = np.stack([rng.permutation(50)[:7] for _ in range(rows)]).astype(np.int32)
    picks[:, 0] = 3
    items, members, distinct = orr.plan(picks, 50, tile)
    bi, bm, bd = brute_plan(picks, 50, tile)
    assert items.tolist() == bi and members.tolist() == bm and distinct == bd
    assert len(items) <= orr.max_items(picks.size, 50, tile)


def test_plan_known_answer():
    """37 rows on one expert: items of 16, 16 and 5 (the reference's tests/cuda/test_experts.py:91-104)."""

    items, members, distinct = orr.plan(np.full((37, 1), 4, np.int32), 9, 16)
    assert items.tolist() == [[4, 0, 16], [4, 16, 16], [4, 32, 5]] and members.tolist() == list(range(37))
    assert distinct == 1
