"""Oracle: MLX 4-bit affine weights, dequant-then-matmul and the expert epilogues, in numpy.  Test infrastructure only.

Conventions: bf16 tensors travel as float32 arrays whose values are bf16-representable (or as uint16 bit patterns
where a function says so); packed codes travel as uint32 arrays ``[..., K/8]``.
"""

from __future__ import annotations

import numpy as np


# -- bf16 ---------------------------------------------------------------------------------------------------------

def bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns (uint16), round to nearest even (what ``.to(torch.bfloat16)`` does)."""

    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    return ((u + bias) >> np.uint32(16)).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b).astype(np.uint32) << np.uint32(16)).view(np.float32)


def bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 values to bf16 and return them as float32."""

    return bf16_from_bits(bf16_bits(x))


# -- the format (families/qwen3_5/cuda/qmm.py:132-149; tests/cuda/test_qmm.py:22-26) ---------------------------------

def nibbles(words: np.ndarray) -> np.ndarray:
    """uint32 words [..., K/8] -> codes uint8 [..., K]: element 8 w + i is bits [4 i, 4 i + 4) of word w."""

    w = np.ascontiguousarray(words).view(np.uint32)
    q = (w[..., None] >> (np.arange(8, dtype=np.uint32) * np.uint32(4))) & np.uint32(15)
    return q.reshape(*w.shape[:-1], w.shape[-1] * 8).astype(np.uint8)


def words_from_nibbles(q: np.ndarray) -> np.ndarray:
    """The inverse of ``nibbles``."""

    q = np.ascontiguousarray(q).astype(np.uint32).reshape(*q.shape[:-1], q.shape[-1] // 8, 8)
    return (q << (np.arange(8, dtype=np.uint32) * np.uint32(4))).sum(-1, dtype=np.uint64).astype(np.uint32)


def dequantize(words: np.ndarray, scales: np.ndarray, biases: np.ndarray, gs: int) -> np.ndarray:
    """W[..., n, k] = scale[n, k // gs] * q[n, k] + bias[n, k // gs] in float32 (a product, then a sum)."""

    q = nibbles(words).astype(np.float32)
    s = np.repeat(np.asarray(scales, dtype=np.float32), gs, axis=-1)
    b = np.repeat(np.asarray(biases, dtype=np.float32), gs, axis=-1)
    return q * s + b


def prefill_weight(w: np.ndarray) -> np.ndarray:
    """The prompt form's one rounding of a dequantized weight.  The reference rounds to bf16
    (cuda/kernels/qmm_prefill.cu:1); this build's kernels round 256 w to fp16 (11 significant bits), which is what the
    tight prompt-form checks compare against; the bound that matters is the unrounded oracle's."""

    return ((w.astype(np.float64) * 256.0).astype(np.float16).astype(np.float32) / np.float32(256)).astype(np.float32)


def linear(x: np.ndarray, words: np.ndarray, scales: np.ndarray, biases: np.ndarray, gs: int, *,
           f32: bool = False, prefill: bool = False) -> np.ndarray:
    """(x.float() @ dequantize(...).T).to(bf16)  (families/qwen3_5/cuda/reference.py:11-15).

    ``prefill`` rounds each dequantized weight first (see ``prefill_weight``)."""

    w = dequantize(words, scales, biases, gs)
    if prefill:
        w = prefill_weight(w)
    y = np.asarray(x, dtype=np.float32) @ w.T
    return y if f32 else bf16(y)


def group_sums(x: np.ndarray, gs: int) -> np.ndarray:
    """xs[m, g] = sum of x[m, g*gs:(g+1)*gs] in float32 (cuda/kernels/qmm.py:139-154)."""

    x = np.asarray(x, dtype=np.float32)
    return x.reshape(x.shape[0], -1, gs).sum(-1, dtype=np.float32)


# -- expert epilogues (cuda/experts.cuh:53-103) -----------------------------------------------------------------------

def relu2(a: np.ndarray) -> np.ndarray:
    """bf16(max(bf16(a), 0)^2)."""

    u = np.maximum(bf16(a), np.float32(0))
    return bf16(u * u)


def swiglu(g: np.ndarray, u: np.ndarray, limit: float = 0.0) -> np.ndarray:
    """bf16(bf16(silu(g')) * u') on bf16 g and u; with limit > 0, g' = min(g, limit), u' = clip(u, -limit, limit)."""

    gv, uv = bf16(g), bf16(u)
    if limit > 0:
        gv = np.minimum(gv, np.float32(limit))
        uv = np.clip(uv, np.float32(-limit), np.float32(limit))
    silu = gv / (np.float32(1) + np.exp(-gv, dtype=np.float32))
    return bf16(bf16(silu.astype(np.float32)) * uv)


def expert_pairs(x: np.ndarray, picks: np.ndarray, up: list, down: tuple, gs: int, *, limit: float = 0.0,
                 prefill: bool = False, y_bf16: bool = False) -> tuple[np.ndarray, np.ndarray]:
    """Every (row, slot) pair through its expert: act [R*S, NI] (bf16 values) and y [R*S, D] (fp32, or bf16 values).

    ``up`` is [gate, up] (SwiGLU) or [up] (relu^2), each (words [E, NI, D/8], scales, biases); ``down`` likewise
    [E, D, NI/8].  Weights are dequantized per used expert; ``prefill`` rounds them first (``prefill_weight``)."""

    x = np.asarray(x, dtype=np.float32)
    rows, slots = picks.shape
    ni, d = up[0][0].shape[1], down[0].shape[1]
    act = np.zeros((rows * slots, ni), dtype=np.float32)
    y = np.zeros((rows * slots, d), dtype=np.float32)
    flat = picks.reshape(-1)

    def weight(m, e):
        w = dequantize(m[0][e], m[1][e], m[2][e], gs)
        return prefill_weight(w) if prefill else w

    for e in np.unique(flat):
        pairs = np.nonzero(flat == e)[0]
        xe = x[pairs // slots]
        projs = [xe @ weight(m, e).T for m in up]
        a = swiglu(projs[0], projs[1], limit) if len(up) == 2 else relu2(projs[0])
        act[pairs] = a
        ye = a @ weight(down, e).T
        y[pairs] = bf16(ye) if y_bf16 else ye
    return act, y


def combine(y: np.ndarray, wts: np.ndarray) -> np.ndarray:
    """out[r] = bf16(sum over slots, in slot order, of fp32 w[r, k] * y[r, k])  (cuda/moe.py:131-142)."""

    rows, slots, _ = y.shape
    acc = np.zeros((rows, y.shape[2]), dtype=np.float32)
    for k in range(slots):
        acc = acc + wts[:, k:k + 1].astype(np.float32) * y[:, k].astype(np.float32)
    return bf16(acc)


# -- fused producers: residual add, RMSNorm, group sums ---------------------------------------------------------------
#
# Pins (tests/test_oracle_affine.py): zero delta leaves h = x; the group sums equal sums of the returned y; a float64
# evaluation of the formulas agrees to bf16 rounding; moving one slot across the routed/shared boundary or dropping
# its weight changes the result (the routed slots are weighted, the rest are not).

def add_rmsnorm(x: np.ndarray, r: np.ndarray | None, w: np.ndarray, eps: float, gs: int = 64):
    """h = bf16(x + r) (x itself without r), y = bf16(h / sqrt(mean(h^2) + eps) * w), xs = y's sums over groups of
    ``gs`` columns in fp32.  x, r, w hold bf16 values as float32.  Returns (h, y, xs)
    (families/qwen3_5/cuda/glue.py:10-41)."""

    x = np.asarray(x, dtype=np.float32)
    h = bf16(x + np.asarray(r, dtype=np.float32)) if r is not None else x
    d = h.shape[1]
    ss = (h.astype(np.float64) ** 2).sum(axis=1, keepdims=True)
    inv = (np.float32(1) / np.sqrt((ss / d).astype(np.float32) + np.float32(eps), dtype=np.float32)).astype(np.float32)
    y = bf16((h * inv) * np.asarray(w, dtype=np.float32)[None, :])
    xs = y.reshape(y.shape[0], d // gs, gs).astype(np.float64).sum(axis=2).astype(np.float32)
    return h, y, xs


def moe_delta(y: np.ndarray, wts: np.ndarray, top_k: int) -> np.ndarray:
    """delta[r] = bf16(sum over the first ``top_k`` slots of w[r, k] * y[r, k] + sum of the remaining slots' y[r, k]),
    each sum in slot order in fp32, products rounded before they are added
    (families/nemotron_h/cuda/glue.py:111-118)."""

    rows, slots, d = y.shape
    routed = np.zeros((rows, d), dtype=np.float32)
    for k in range(top_k):
        routed = routed + wts[:, k:k + 1].astype(np.float32) * y[:, k].astype(np.float32)
    shared = np.zeros((rows, d), dtype=np.float32)
    for k in range(top_k, slots):
        shared = shared + y[:, k].astype(np.float32)
    return bf16(routed + shared)


def add_moe_norm(h: np.ndarray, y: np.ndarray, wts: np.ndarray, w: np.ndarray, eps: float, top_k: int, gs: int = 64):
    """(bf16(h + delta), its RMSNorm times w, the group sums) with ``delta = moe_delta(y, wts, top_k)``
    (families/nemotron_h/cuda/glue.py:103-141)."""

    return add_rmsnorm(h, moe_delta(y, wts, top_k), w, eps, gs)


# -- the FP8 prompt path (cuda/kernels/qmm.py:222-268, qmm_prefill8.cu:1-2,186-188) --------------------------------

def e4m3_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> OCP e4m3 (e4m3fn: bias 7, no infinities, largest 448) bit patterns, round to nearest even.  Values
    are taken within +-464 (nothing larger is asked of it: ``quantize_rows`` divides by the row's max / 448)."""

    v = np.ascontiguousarray(x, dtype=np.float32)
    a = np.abs(v).astype(np.float64)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -20)))
    e = np.clip(e, -6, 8)                                  # below 2^-6 the step stays 2^-9 (subnormals)
    step = 2.0 ** (e - 3)
    q = np.rint(a / step)                                  # ties to even; 16 steps of a binade carry into the next
    mag = q * step
    e2 = np.floor(np.log2(np.maximum(mag, 2.0 ** -20)))
    code = np.where(mag < 2.0 ** -6, np.rint(mag * 512.0),
                    (e2 + 7) * 8 + np.rint(mag / 2.0 ** (e2 - 3)) - 8).astype(np.int64)
    code = np.minimum(code, 0x7E)
    return (code | ((np.signbit(v)).astype(np.int64) << 7)).astype(np.uint8)


def e4m3_values(b: np.ndarray) -> np.ndarray:
    """e4m3 bit patterns -> float32 values."""

    b = np.ascontiguousarray(b).astype(np.int64)
    ex, man = (b >> 3) & 15, b & 7
    mag = np.where(ex == 0, man * 2.0 ** -9, (8 + man) * 2.0 ** (ex - 10))
    return np.where(b & 0x80, -mag, mag).astype(np.float32)


def quantize_rows(x: np.ndarray, gs: int):
    """``quantize_rows`` (kernels/qmm.py:222-255).  x float32 [M, K] of bf16 values -> (x8 uint8 [M, K] e4m3 bits in
    input order, xs float32 [M, K / gs] of bf16 values, a float32 [M]).  a = max|x| / 448 (1 for a row of zeros),
    x8 = e4m3(x / a), xs = bf16(sum of the group's inputs / a); the sum is taken an octet of inputs at a time, in order,
    and the octets' sums in order (the order the kernel fixes; the reference's Triton sum leaves it open)."""

    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    top = np.abs(x).max(axis=1)
    a = np.where(top > 0, top / np.float32(448), np.float32(1)).astype(np.float32)
    x8 = e4m3_bits(x / a[:, None])
    octets = np.cumsum(x.reshape(m, k // 8, 8), axis=2, dtype=np.float32)[:, :, -1]
    sums = np.cumsum(octets.reshape(m, k // gs, gs // 8), axis=2, dtype=np.float32)[:, :, -1]
    return x8, bf16(sums / a[:, None]), a


def prefill8(x8: np.ndarray, xs: np.ndarray, a: np.ndarray, words: np.ndarray, scales: np.ndarray,
             biases: np.ndarray, gs: int) -> np.ndarray:
    """``prefill_matmul8`` on ``quantize_rows`` output (qmm_prefill8.cu:1-2): per group, in order,
    acc = fma(P, s, acc) with P the group's sum of x8 * q (exact operands; taken in float64 here, the matrix unit's
    fp32 sum of the same exact products can differ in its last bit), then acc += xs . bias over the groups, then
    out = acc * a.  float32 [M, N]."""

    xv = e4m3_values(x8).astype(np.float64)
    q = nibbles(words).astype(np.float64)                               # [N, K]
    m, k = xv.shape
    s = np.asarray(scales, dtype=np.float32)
    b = np.asarray(biases, dtype=np.float32)
    acc = np.zeros((m, q.shape[0]), dtype=np.float32)
    for g in range(k // gs):
        part = (xv[:, g * gs:(g + 1) * gs] @ q[:, g * gs:(g + 1) * gs].T).astype(np.float32)
        acc = (part.astype(np.float64) * s[:, g].astype(np.float64)[None, :] + acc.astype(np.float64)).astype(np.float32)
    acc = (acc.astype(np.float64) + np.asarray(xs, dtype=np.float64) @ b.astype(np.float64).T).astype(np.float32)
    return acc * np.asarray(a, dtype=np.float32)[:, None]

