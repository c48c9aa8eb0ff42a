"""Oracle: the EXL3 trellis format (codebooks, circular bitstream, tile permutation, Hadamard-128 layer) in numpy.

Test infrastructure only.  Restates cuda/exl3/format.py:31-180 and the prose of docs/recipes/exl3.md:43-74 with a
different decoder construction (an explicit bit array and gathered 16-bit windows), so that agreement with the C
bit-by-bit decoder in ``orc.c`` and with the pure-Python one in the tests is meaningful.
"""

from __future__ import annotations

import numpy as np

CODEBOOKS = ("3inst", "mcg", "mul1")
CODEBOOK_IDS = {"3inst": 0, "mcg": 1, "mul1": 2}
WIDTHS = (1, 1.5, 2, 2.5, 3, 3.5, 4, 5, 6, 7, 8)            # what checkpoints hold (x.5 with mul1 only)
# every half-bit count from 2 to 16: the bitstream rule is the same for all of them, and the reference's routed-expert
# kernels take any of them with any codebook (cuda/exl3/experts.py:15-16, decode.cuh:19-22)
EVERY_WIDTH = tuple(k2 / 2 for k2 in range(2, 17))

_tables: dict[str, np.ndarray] = {}


def _half(bits: np.ndarray) -> np.ndarray:
    return bits.astype(np.uint16).view(np.float16).astype(np.float64)


def codebook(name: str) -> np.ndarray:
    """fp16 value of each 16-bit state s, [65536]  (docs/recipes/exl3.md:55-59)."""

    if name in _tables:
        return _tables[name]
    if name not in CODEBOOKS:
        raise ValueError(f"unknown EXL3 codebook {name!r}")
    s = np.arange(1 << 16, dtype=np.uint64)
    two32 = np.uint64(0xFFFFFFFF)
    if name == "mul1":
        x = (s * np.uint64(0x83DCD12D)) & two32
        h = np.uint64(1024) + sum(((x >> np.uint64(8 * i)) & np.uint64(255)) for i in range(4))
        a = _half(np.array([0x1EEE]))[0]
        c = _half(np.array([0xC931]))[0]
        table = (h.astype(np.float64) * a + c).astype(np.float16)        # exact in float64: one rounding
    else:
        x = (s * np.uint64(89226354) + np.uint64(64248484)) & two32 if name == "3inst" \
            else (s * np.uint64(0xCBAC1FED)) & two32
        x = (x & np.uint64(0x8FFF8FFF)) ^ np.uint64(0x3B603B60)
        table = (_half(x & np.uint64(0xFFFF)) + _half(x >> np.uint64(16))).astype(np.float16)
    _tables[name] = table
    return table


def check_width(bits: float) -> float:
    b = float(bits)
    if b not in EVERY_WIDTH:
        raise ValueError(f"EXL3 bits must be one of {EVERY_WIDTH}, got {bits}")
    return b


def window_ends(bits: float) -> np.ndarray:
    """E(p), p = 0..255: one past the last stream bit of value p's window  (docs/recipes/exl3.md:48-52)."""

    b = check_width(bits)
    steps = np.full(256, int(b), dtype=np.int64)
    if not b.is_integer():
        steps[1::2] += 1                                  # the odd positions take the extra bit
    return np.cumsum(steps)


def positions() -> tuple[np.ndarray, np.ndarray]:
    """(row, col) inside the 16 x 16 tile of stream value p  (docs/recipes/exl3.md:61-63)."""

    p = np.arange(256)
    l, j = p >> 3, p & 7
    return 2 * (l & 3) + (j & 1) + 8 * ((j >> 1) & 1), (l >> 2) + 8 * (j >> 2)


def tile_states(trellis: np.ndarray, bits: float) -> np.ndarray:
    """int16 [..., 16*bits] -> the 256 16-bit states of each tile, uint32 [..., 256], in stream order."""

    t = np.ascontiguousarray(trellis)
    n16 = int(16 * check_width(bits))
    if t.dtype != np.int16 or t.shape[-1] != n16:
        raise ValueError(f"trellis must be int16 [..., {n16}], got {t.dtype} {t.shape}")
    lead = t.shape[:-1]
    u = t.view(np.uint16).reshape(-1, n16 // 2, 2).astype(np.uint32)
    words = u[..., 0] | (u[..., 1] << np.uint32(16))                       # little-endian int16 pairs
    be = words.astype(">u4").view(np.uint8).reshape(words.shape[0], -1)    # most significant byte first
    stream = np.unpackbits(be, axis=1)                                     # [tiles, R] bits, MSB of each word first
    r = stream.shape[1]
    idx = (window_ends(bits)[:, None] - 16 + np.arange(16)[None, :]) % r   # [256, 16]
    weights = (1 << np.arange(15, -1, -1)).astype(np.uint32)
    out = np.empty((stream.shape[0], 256), dtype=np.uint32)
    step = max(1, (1 << 22) // 4096)
    for a in range(0, stream.shape[0], step):
        out[a:a + step] = (stream[a:a + step][:, idx].astype(np.uint32) * weights).sum(-1)
    return out.reshape(*lead, 256)


def unpack(trellis: np.ndarray, bits: float, name: str) -> np.ndarray:
    """W_q [K, N] fp16 (rotated domain) from trellis int16 [K/16, N/16, 16*bits]."""

    t = np.ascontiguousarray(trellis)
    if t.ndim != 3:
        raise ValueError("trellis must be [K/16, N/16, 16 * bits]")
    kt, nt = t.shape[:2]
    vals = codebook(name)[tile_states(t, bits)]                            # [kt, nt, 256]
    rows, cols = positions()
    w = np.empty((kt, nt, 16, 16), dtype=np.float16)
    w[:, :, rows, cols] = vals
    return w.transpose(0, 2, 1, 3).reshape(kt * 16, nt * 16)


def unpack_signs(packed: np.ndarray) -> np.ndarray:
    """int16 sign words -> fp16 +-1: bit b of word w set <=> element 16 w + b is -1  (format.py:128-133)."""

    p = np.ascontiguousarray(packed).view(np.uint16).reshape(-1)
    bits = np.unpackbits(p.astype("<u2").view(np.uint8), bitorder="little")
    return np.where(bits == 1, -1.0, 1.0).astype(np.float16)


def hadamard(n: int = 128) -> np.ndarray:
    """Sylvester's construction: H_1 = [1], H_2n = [[H, H], [H, -H]]."""

    h = np.ones((1, 1))
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h


def rotate(x: np.ndarray, axis: int = -1) -> np.ndarray:
    """Each block of 128 along ``axis`` times H / sqrt(128), float64."""

    x = np.moveaxis(np.asarray(x, dtype=np.float64), axis, -1)
    if x.shape[-1] % 128:
        raise ValueError("the rotated dimension must be a multiple of 128")
    y = (x.reshape(*x.shape[:-1], -1, 128) @ (hadamard(128) / np.sqrt(128.0))).reshape(x.shape)
    return np.moveaxis(y, -1, axis)


def dequantize(trellis, suh, svh, bits: float, name: str) -> np.ndarray:
    """W = diag(suh) H_K W_q H_N diag(svh), float64 [K, N]."""

    w = rotate(unpack(trellis, bits, name).astype(np.float64), 0) * np.asarray(suh, dtype=np.float64)[:, None]
    return rotate(w, 1) * np.asarray(svh, dtype=np.float64)[None, :]


def forward(x, trellis, suh, svh, bits: float, name: str, bias=None, *, half_input: bool = False) -> np.ndarray:
    """y = ((((x * suh) H) W_q) H) * svh + bias in float64.  ``half_input`` rounds the rotated input to fp16 as the
    kernels do (cuda/exl3/linear.cu:110-124; tests/cuda/test_exl3_linear.py:32-39)."""

    xh = rotate(np.asarray(x, dtype=np.float64) * np.asarray(suh, dtype=np.float64), -1)
    if half_input:
        xh = xh.astype(np.float16).astype(np.float64)
    y = rotate(xh @ unpack(trellis, bits, name).astype(np.float64), -1) * np.asarray(svh, dtype=np.float64)
    return y if bias is None else y + np.asarray(bias, dtype=np.float64)


# -- routed experts (cuda/exl3/experts.py:173-202, experts.cu:96-237) --------------------------------------------------
#
# Pins (tests/test_oracle_exl3.py): without the fp16 input roundings the pair output equals the dense float64
# formula on dequantize()'s W (an independent path through the same decode); the clip and the bf16 roundings against
# hand-computed values; skipped picks contribute nothing; the combine is linear in the weights.

def swiglu_pair(g: np.ndarray, u: np.ndarray, limit: float = np.inf, act_bf16: bool = False) -> np.ndarray:
    """min(g, limit) * sigmoid(min(g, limit)) * clip(u, -limit, limit); with ``act_bf16`` g, u, the SiLU and the
    product are each rounded to bf16 first, in fp32 as the kernel computes them (experts.cu:141-151)."""

    if not act_bf16:
        gg = np.minimum(np.asarray(g, dtype=np.float64), limit)
        uu = np.clip(np.asarray(u, dtype=np.float64), -limit, limit)
        return gg / (1.0 + np.exp(-gg)) * uu
    from .affine import bf16

    gg = np.minimum(bf16(np.asarray(g, dtype=np.float32)), np.float32(min(limit, 3.0e38)))
    uu = np.clip(bf16(np.asarray(u, dtype=np.float32)), -np.float32(min(limit, 3.0e38)), np.float32(min(limit, 3.0e38)))
    silu = bf16((gg / (np.float32(1) + np.exp(-gg, dtype=np.float32))).astype(np.float32))
    return bf16((silu * uu).astype(np.float32)).astype(np.float64)


def routed(x, pick, wts, gate, up, down, name: str, *, limit: float = np.inf, act_bf16: bool = False,
           half_input: bool = True) -> tuple[np.ndarray, np.ndarray]:
    """Routed experts: ``gate``, ``up``, ``down`` are per-expert (trellis int16, suh, svh) triples, each trellis at
    its own width; pick [R, slots] int, wts [R, slots].  Pair (r, k) with 0 <= pick < E gives
    y[r, k] = down(swiglu(gate(x[r]), up(x[r]))), every projection a ``forward`` (``half_input`` rounds its rotated
    input to fp16 as the kernels do); other pairs are skipped (zeros).  Returns (y [R, slots, D], out [R, D] =
    sum over the routed slots of wts * y), float64."""

    x = np.asarray(x, dtype=np.float64)
    pick = np.asarray(pick)
    rows, slots = pick.shape
    n_exp = len(gate)
    y = np.zeros((rows, slots, x.shape[1]), dtype=np.float64)

    def lin(v, m):
        t, suh, svh = m
        return forward(v[None, :], np.asarray(t), np.asarray(suh), np.asarray(svh), t.shape[-1] / 16, name,
                       half_input=half_input)[0]

    for r in range(rows):
        for k in range(slots):
            e = int(pick[r, k])
            if e < 0 or e >= n_exp:
                continue
            a = swiglu_pair(lin(x[r], gate[e]), lin(x[r], up[e]), limit, act_bf16)
            y[r, k] = lin(a, down[e])
    out = (np.asarray(wts, dtype=np.float64)[:, :, None] * y).sum(axis=1)
    return y, out
