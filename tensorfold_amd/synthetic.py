"""Seeded synthetic inputs in the shapes the benchmark configurations name (there are no checkpoints to load).

Everything is drawn on the CPU with ``torch.Generator().manual_seed`` / ``numpy.random.default_rng`` so that the
same seed gives the same tensors on any machine; callers move them to the GPU.  Used by the tests, ``bench.py`` and
the smoke check.
"""

from __future__ import annotations

import dataclasses

import numpy as np
import torch


def affine(n: int, k: int, gs: int, seed: int, lead: tuple[int, ...] = ()) -> tuple[torch.Tensor, ...]:
    """MLX 4-bit tensors: words int32 [*lead, n, k/8] (codes uniform 0..15), scales bf16 ~ U(0.002, 0.02),
    biases = -8 * scale (exact in bf16)."""

    g = torch.Generator().manual_seed(seed)
    words = torch.randint(-(2 ** 31), 2 ** 31, (*lead, n, k // 8), generator=g, dtype=torch.int64).to(torch.int32)
    scales = (torch.rand((*lead, n, k // gs), generator=g) * 0.018 + 0.002).to(torch.bfloat16)
    biases = (scales.float() * -8).to(torch.bfloat16)
    return words, scales, biases


def affine_general(n: int, k: int, gs: int, seed: int, lead: tuple[int, ...] = ()) -> tuple[torch.Tensor, ...]:
    """As ``affine`` with independent biases ~ N(0, 0.02) (the distribution the reference's kernel tests draw)."""

    g = torch.Generator().manual_seed(seed)
    words = torch.randint(-(2 ** 31), 2 ** 31, (*lead, n, k // 8), generator=g, dtype=torch.int64).to(torch.int32)
    scales = (torch.rand((*lead, n, k // gs), generator=g) * 0.02 + 0.001).to(torch.bfloat16)
    biases = (torch.randn((*lead, n, k // gs), generator=g) * 0.02).to(torch.bfloat16)
    return words, scales, biases


def activations(rows: int, k: int, seed: int, scale: float = 1.0, dtype=torch.bfloat16) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((rows, k), generator=g) * scale).to(dtype)


def logits(rows: int, columns: int, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randn((rows, columns), generator=g, dtype=torch.float32)


def zipf_picks(rows: int, experts: int, top_k: int, seed: int, s: float = 1.1) -> torch.Tensor:
    """Each row: ``top_k`` distinct experts drawn without replacement with p(e) ~ (e + 1)^-s; int32 [rows, top_k]."""

    g = torch.Generator().manual_seed(seed)
    p = (torch.arange(experts, dtype=torch.float64) + 1) ** -s
    return torch.multinomial(p.expand(rows, experts), top_k, replacement=False, generator=g).to(torch.int32)


def exl3_layer(k: int, n: int, bits: float, seed: int):
    """trellis int16 [k/16, n/16, 16 * bits] uniform; suh, svh fp16 ~ U(0.5, 2) with random signs."""

    rng = np.random.default_rng(seed)
    trellis = rng.integers(-2 ** 15, 2 ** 15, size=(k // 16, n // 16, int(16 * bits)), dtype=np.int64).astype(np.int16)

    def signed(size: int) -> np.ndarray:
        return (rng.uniform(0.5, 2.0, size) * rng.choice([-1.0, 1.0], size)).astype(np.float16)

    return torch.from_numpy(trellis), torch.from_numpy(signed(k)), torch.from_numpy(signed(n))


@dataclasses.dataclass(frozen=True)
class MoEShape:
    name: str
    hidden: int
    experts: int
    width: int
    top_k: int
    gs: int
    swiglu: bool
    shared: bool


C1 = MoEShape("decode MoE layer, 4-bit/g64, D=2688, 128 experts, NI=1856, relu^2, top-6", 2688, 128, 1856, 6, 64,
              False, False)
C2 = MoEShape("decode/verify MoE layer, 4-bit/g32, D=2048, 512 experts + shared, NI=512, SwiGLU, top-10", 2048, 512,
              512, 10, 32, True, True)
