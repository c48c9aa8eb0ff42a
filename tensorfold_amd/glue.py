"""Fused producers of the quantized matmuls' inputs: residual add, RMSNorm and the group sums in one launch.

Mirrors the reference's ``families/qwen3_5/cuda/glue.py:31-41`` (``add_rmsnorm``) and
``families/nemotron_h/cuda/glue.py:131-141`` (``add_moe_norm``): same arguments, same three results; each row's bits
depend on that row alone.  ``gs`` (the weights' group size, 64 in the reference) is the one extra argument.
"""

from __future__ import annotations

import torch

from . import _lib


def _check(x: torch.Tensor, w: torch.Tensor, gs: int) -> tuple[int, int]:
    if x.dim() != 2 or x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("add_norm: x must be a contiguous bf16 [rows, d]")
    rows, d = x.shape
    if w.dtype != torch.bfloat16 or tuple(w.shape) != (d,) or not w.is_contiguous():
        raise ValueError(f"add_norm: the norm weight must be a contiguous bf16 [{d}]")
    if gs not in (32, 64, 128) or d % gs or d > 16384 or rows < 1:
        raise ValueError(f"add_norm: rows of up to 16384 values in whole groups of 32, 64 or 128, not d={d}, gs={gs}")
    _lib.on_gpu(x, w)
    return rows, d


def add_rmsnorm(x: torch.Tensor, r: torch.Tensor | None, w: torch.Tensor, eps: float, gs: int = 64):
    """h = x + r (bf16; x itself when r is None), y = rmsnorm(h) * w (bf16), xs = y's group sums (fp32).
    Returns (h, y, xs)."""

    rows, d = _check(x, w, gs)
    if r is not None and (r.dtype != torch.bfloat16 or r.shape != x.shape or not r.is_contiguous() or not r.is_cuda):
        raise ValueError("add_rmsnorm: r must be a contiguous bf16 GPU tensor of x's shape")
    h = torch.empty_like(x) if r is not None else x
    y = torch.empty_like(x)
    xs = torch.empty((rows, d // gs), dtype=torch.float32, device=x.device)
    _lib.call("tf_add_norm", _lib.ptr(x), _lib.ptr(r), 0 if r is None else 1, None, 0, 0, _lib.ptr(w), float(eps),
              _lib.ptr(h) if r is not None else None, _lib.ptr(y), _lib.ptr(xs), rows, d, gs)
    return h, y, xs


def add_moe_norm(h: torch.Tensor, y: torch.Tensor, wt: torch.Tensor, w: torch.Tensor, eps: float, top_k: int,
                 gs: int = 64):
    """h [R, D] bf16, y [R * NS, D] fp32 or bf16 pair outputs, wt [R, NS] fp32 -> (h + delta, its RMSNorm, group sums),
    delta = bf16(sum of the first ``top_k`` slots' wt * y + sum of the other slots' y)."""

    rows, d = _check(h, w, gs)
    if wt.dim() != 2 or wt.shape[0] != rows or wt.dtype != torch.float32 or not wt.is_contiguous():
        raise ValueError("add_moe_norm: wt must be a contiguous fp32 [rows, slots]")
    slots = wt.shape[1]
    if y.dtype not in (torch.float32, torch.bfloat16) or tuple(y.shape) != (rows * slots, d) or not y.is_contiguous():
        raise ValueError(f"add_moe_norm: y must be a contiguous fp32 or bf16 [{rows * slots}, {d}]")
    if not 0 <= top_k <= slots:
        raise ValueError(f"add_moe_norm: top_k {top_k} outside 0..{slots}")
    _lib.on_gpu(y, wt)
    hn = torch.empty_like(h)
    out = torch.empty_like(h)
    xs = torch.empty((rows, d // gs), dtype=torch.float32, device=h.device)
    _lib.call("tf_add_norm", _lib.ptr(h), _lib.ptr(y), 3 if y.dtype == torch.bfloat16 else 2, _lib.ptr(wt), slots,
              int(top_k), _lib.ptr(w), float(eps), _lib.ptr(hn), _lib.ptr(out), _lib.ptr(xs), rows, d, gs)
    return hn, out, xs
