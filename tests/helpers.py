"""Conversions between torch tensors and the oracle's numpy conventions, and the error measures the tests state."""

from __future__ import annotations

import numpy as np
import torch


def f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def bits16(t: torch.Tensor) -> np.ndarray:
    """bf16 / fp16 tensor -> its bit patterns as uint16."""

    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def u32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def rel_l2(got, want) -> float:
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def max_abs(got, want) -> float:
    return float(np.abs(np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)).max())
