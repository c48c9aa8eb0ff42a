"""EXL3 prompt matmuls: W_q decoded once a chunk, then an fp16 MFMA GEMM whose epilogue rotates each 128-column block.

Mirrors the reference's ``cuda/exl3/prefill.py:15-95`` (``tiles``, ``Workspace``, ``matmul``): any M, a row's output
bits independent of the chunk it arrives in.  Differences: the decoded weight is kept as [K / 8, N, 8] (the order an
MFMA B operand is read in: 16 bytes a lane, a tile's columns side by side); the epilogue's Hadamard is an exact fp32
butterfly, not the reference's bf16 hi/lo split matmul.
"""

from __future__ import annotations

import torch

from .. import _lib
from .linear import CODEBOOK_IDS, Exl3Linear, _DTYPES


def tiles(k: int, n: int) -> tuple[int, int]:
    """(rows, columns) a workgroup takes: the shape's alone, so a row never depends on its chunk
    (exl3/prefill.py:47-50)."""

    return 128, 256


class Workspace:
    """One decoded W_q (as [K / 8, N, 8]) and one rotated input, grown to the largest call and reused: calls that share a
    workspace run in order on one stream (exl3/prefill.py:53-79)."""

    def __init__(self) -> None:
        self.w: torch.Tensor | None = None
        self.xh: torch.Tensor | None = None

    def _grow(self, name: str, numel: int, device: torch.device) -> torch.Tensor:
        t = getattr(self, name)
        if t is None or t.numel() < numel or t.device != device:
            t = torch.empty((numel,), dtype=torch.float16, device=device)
            setattr(self, name, t)
        return t

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w, self.xh) if t is not None)


def decode(layer: Exl3Linear, ws: Workspace) -> torch.Tensor:
    """W_q as fp16 [K / 8, N, 8] (``w8[o, c, i] = W_q[8 * o + i, c]``) into the workspace: once a chunk, or once for
    several calls on one layer."""

    k, n = layer.k, layer.n
    w8 = ws._grow("w", k * n, layer.words.device)[:k * n].view(k // 8, n, 8)
    _lib.call("tf_exl3_unpack_k8", _lib.ptr(layer.words), _lib.ptr(w8), k, n, *layer.strides, layer.k2,
              CODEBOOK_IDS[layer.codebook])
    return w8


def matmul(layer: Exl3Linear, x: torch.Tensor, out: torch.Tensor, ws: Workspace,
           wt: torch.Tensor | None = None) -> torch.Tensor:
    """out [M, N] (row stride free) = x [M, K] @ W + bias for any M, the prompt path's arithmetic
    (exl3/prefill.py:82-95).  ``wt`` brings a weight already decoded with ``decode``."""

    m, k, n = int(x.shape[0]), layer.k, layer.n
    if x.dim() != 2 or x.shape[1] != k or tuple(out.shape) != (m, n) or out.stride(1) != 1 or m < 1:
        raise ValueError(f"prefill matmul: x {tuple(x.shape)} and out {tuple(out.shape)} do not match K={k}, N={n}")
    if x.dtype not in _DTYPES or out.dtype not in _DTYPES:
        raise ValueError("prefill matmul: x and out must be fp16, bf16 or fp32")
    if out.stride(0) < n or out.stride(0) % 2 or out.data_ptr() % 8:
        raise ValueError("prefill matmul: out rows must be an even stride apart and 8-byte aligned")
    _lib.on_gpu(x, out)
    x = x.contiguous()
    xh = ws._grow("xh", m * k, x.device)[:m * k].view(m, k)
    _lib.call("tf_exl3_rot_in", _lib.ptr(x), _DTYPES[x.dtype], _lib.ptr(layer.suh), _lib.ptr(xh), m, k)
    if wt is None:
        wt = decode(layer, ws)
    elif wt.dtype != torch.float16 or tuple(wt.shape) != (k // 8, n, 8) or not wt.is_contiguous() or wt.device != x.device:
        raise ValueError(f"prefill matmul: wt must be the contiguous fp16 ({k // 8}, {n}, 8) that decode() returns")
    _lib.call("tf_exl3_gemm", _lib.ptr(xh), _lib.ptr(wt), _lib.ptr(layer.svh), _lib.ptr(layer.bias), _lib.ptr(out),
              _DTYPES[out.dtype], out.stride(0), m, k, n)
    return out
