"""Host-side facts of the EXL3 format that the GPU layer needs at load time: widths, codebook ids, tile sizes, the
packed sign words of older checkpoints.  (The format is ExLlamaV3's, MIT, Copyright (c) 2025 Turboderp; the
reference states it in src/tensorfold/cuda/exl3/format.py:14-110 and docs/recipes/exl3.md:43-74.)

Decoding itself happens on the GPU (``linear.py``); nothing here computes weights.
"""

from __future__ import annotations

import numpy as np

CODEBOOKS = ("3inst", "mcg", "mul1")
CODEBOOK_IDS = {name: i for i, name in enumerate(CODEBOOKS)}
BITS = (1, 1.5, 2, 2.5, 3, 3.5, 4, 5, 6, 7, 8)      # half widths exist with the mul1 codebook only
HAD = 128                                           # Hadamard block


def check_bits(bits: float) -> float:
    """``bits`` as a float if it is a width the format has, else ValueError."""

    b = float(bits)
    if b not in BITS:
        raise ValueError(f"EXL3 bits must be one of {', '.join(str(v) for v in BITS)}, got {bits}")
    return b


def tile_words(bits: float) -> int:
    """int16 words of one 16 x 16 tile."""

    return int(16 * check_bits(bits))


def bits_of(trellis_shape) -> float:
    """Bits per weight of a trellis from its last dimension (16 * bits int16 words a tile)."""

    last = int(tuple(trellis_shape)[-1])
    if last % 8:
        raise ValueError(f"EXL3 trellis tiles hold a multiple of 8 int16 words, got {last}")
    b = last / 16
    return check_bits(int(b) if b.is_integer() else b)


def check_pair(bits: float, codebook: str) -> None:
    """A width and codebook that exist together."""

    if codebook not in CODEBOOK_IDS:
        raise ValueError(f"unknown EXL3 codebook {codebook!r}")
    if not float(bits).is_integer() and codebook != "mul1":
        raise ValueError(f"{bits}-bit EXL3 tiles need the mul1 codebook")


def unpack_signs(packed) -> np.ndarray:
    """Sign words (su / sv of older checkpoints) int16 [n/16] -> fp16 [n] of +-1; bit b of word w set means element
    16 w + b is negative."""

    if hasattr(packed, "detach"):
        packed = packed.detach().cpu().numpy()
    words = np.ascontiguousarray(packed).view(np.uint16).reshape(-1, 1)
    neg = (words >> np.arange(16, dtype=np.uint16)) & 1
    return np.where(neg.reshape(-1) == 1, np.float16(-1), np.float16(1))
