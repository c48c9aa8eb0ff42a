"""Oracle: per-row top-k routing and the grouping of (row, slot) pairs by expert.  Test infrastructure only."""

from __future__ import annotations

import numpy as np

from .affine import bf16


def topk_rows(logits: np.ndarray, experts: int, top_k: int, *, shared: bool = True) -> tuple[np.ndarray, np.ndarray]:
    """Row r's ``top_k`` experts by fp32 logit over columns [0, experts), largest first, the lower id among equals;
    weights bf16(exp(l_k - l_0) / sum) held as fp32.  With ``shared`` the last slot is expert id ``experts`` with
    weight bf16(sigmoid(bf16(logits[r, experts])))  (cuda/moe.py:58-85)."""

    l = np.asarray(logits, dtype=np.float32)
    rows = l.shape[0]
    slots = top_k + (1 if shared else 0)
    picks = np.zeros((rows, slots), dtype=np.int32)
    wts = np.zeros((rows, slots), dtype=np.float32)
    for r in range(rows):
        v = l[r, :experts].copy()
        top = v.max()
        total = np.float32(0)
        ex = np.zeros(top_k, dtype=np.float32)
        for k in range(top_k):
            m = v.max()
            idx = int(np.nonzero(v == m)[0][0])
            ex[k] = np.exp(np.float32(m - top), dtype=np.float32)
            total = np.float32(total + ex[k])
            picks[r, k] = idx
            v[idx] = -np.inf
        wts[r, :top_k] = bf16(ex / total)
        if shared:
            sg = bf16(l[r, experts:experts + 1])
            picks[r, top_k] = experts
            wts[r, top_k] = bf16(np.float32(1) / (np.float32(1) + np.exp(-sg, dtype=np.float32)))[0]
    return picks, wts


def plan(picks: np.ndarray, experts: int, tile: int) -> tuple[np.ndarray, np.ndarray, int]:
    """Pairs p = row * slots + slot grouped by expert id ascending, pair order kept within an expert; items
    (expert, first member, count <= tile) in expert order.  Returns (items [n, 3], members [P], distinct experts)
    (cuda/experts.cu:157-285; the spec the reference tests against is tests/cuda/test_experts.py:107-115)."""

    flat = np.asarray(picks, dtype=np.int64).reshape(-1)
    members = np.argsort(flat, kind="stable").astype(np.int32)
    counts = np.bincount(flat, minlength=experts)
    items = []
    first = 0
    for e in range(experts):
        c = int(counts[e])
        for j in range(0, c, tile):
            items.append((e, first + j, min(tile, c - j)))
        first += c
    return np.array(items, dtype=np.int32).reshape(-1, 3), members, int((counts > 0).sum())


def max_items(pairs: int, experts: int, tile: int) -> int:
    """Upper bound on a plan's items (cuda/experts.py:95-98)."""

    return min(pairs, experts) + pairs // tile
