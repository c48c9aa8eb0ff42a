"""Pins of the EXL3 oracle (CPU only): hand-computed codebook values, three independent decoders (vectorised numpy,
C bit by bit, pure Python bit by bit) for all 27 codebook-and-width combinations, format invariants, the layer."""

import struct

import numpy as np
import pytest

from oracle import exl3 as ore
from oracle import native

COMBOS = [(cb, b) for cb in ore.CODEBOOKS for b in ore.EVERY_WIDTH]         # 45: every half-bit count, every codebook


def half(bits: int) -> float:
    """fp16 bit pattern -> value, by Python's own struct codec (not numpy)."""

    return struct.unpack("<e", struct.pack("<H", bits))[0]


def to_half_bits(v: float) -> int:
    return struct.unpack("<H", struct.pack("<e", v))[0]          # struct rounds to nearest even


def slow_value(s: int, cb: str) -> int:
    """The prose of docs/recipes/exl3.md:55-59 in Python integers; returns fp16 bits."""

    if cb == "mul1":
        x = (s * 0x83DCD12D) % 2 ** 32
        h = 1024 + sum((x >> (8 * i)) & 255 for i in range(4))
        return to_half_bits(h * half(0x1EEE) + half(0xC931))      # exact in float64, then one rounding
    x = (s * 0xCBAC1FED) % 2 ** 32 if cb == "mcg" else (s * 89226354 + 64248484) % 2 ** 32
    x = (x & 0x8FFF8FFF) ^ 0x3B603B60
    return to_half_bits(half(x & 0xFFFF) + half(x >> 16))


def slow_tile(words16, bits, cb):
    """One tile bit by bit, straight from the prose (docs/recipes/exl3.md:43-52)."""

    stream = []
    for j in range(0, len(words16), 2):
        word = (int(words16[j]) & 0xFFFF) | ((int(words16[j + 1]) & 0xFFFF) << 16)
        stream += [(word >> (31 - b)) & 1 for b in range(32)]
    n = len(stream)
    out, end = [], 0
    for p in range(256):
        end += int(bits) + (1 if (not float(bits).is_integer() and p % 2 == 1) else 0)
        s = 0
        for b in range(end - 16, end):
            s = (s << 1) | stream[b % n]
        out.append(slow_value(s, cb))
    assert end == n
    return out


def test_codebook_values_worked_by_hand():
    """3inst, s = 0: x = 64248484 = 0x03D45AA4; masked and flipped halves 0x38B4 and 0x31C4 are
    0.587890625 and 0.18017578125, whose sum 0.76806640625 is an fp16 value.
    mul1, s = 0: h = 1024, 1024 * fp16(0x1EEE) + fp16(0xC931) = 6.9296875 - 10.3828125 = -3.453125."""

    assert half(0x38B4) == 0.587890625 and half(0x31C4) == 0.18017578125
    assert float(ore.codebook("3inst")[0]) == 0.76806640625
    assert half(0x1EEE) * 1024 == 6.9296875 and half(0xC931) == -10.3828125
    assert float(ore.codebook("mul1")[0]) == -3.453125
    # mcg, s = 1: x = 0xCBAC1FED -> (0x8BAC ^ 0x3B60, 0x0FED ^ 0x3B60) = (0xB0CC, 0x348D)
    assert float(ore.codebook("mcg")[1]) == float(np.float16(half(0xB0CC) + half(0x348D)))


@pytest.mark.parametrize("cb", ore.CODEBOOKS)
def test_codebooks_three_ways(cb):
    table = ore.codebook(cb)
    assert table.dtype == np.float16 and table.shape == (65536,) and np.isfinite(table).all()
    assert 0.5 < float(np.std(table.astype(np.float64))) < 2.0        # unit-scale, Gaussian-like
    assert abs(float(np.mean(table.astype(np.float64)))) < 0.05
    assert np.array_equal(table.view(np.uint16), native.exl3_codebook(ore.CODEBOOK_IDS[cb]).view(np.uint16))
    rng = np.random.default_rng(0)
    for s in [0, 1, 2, 0x7FFF, 0x8000, 0xFFFF, *rng.integers(0, 65536, size=300).tolist()]:
        assert int(table.view(np.uint16)[s]) == slow_value(int(s), cb), (cb, s)
    with pytest.raises(ValueError):
        ore.codebook("2mad")


@pytest.mark.parametrize("cb,bits", COMBOS)
def test_decoders_agree_bit_by_bit(cb, bits):
    rng = np.random.default_rng(int(10 * bits) + len(cb))
    t = rng.integers(-2 ** 15, 2 ** 15, size=(2, 2, int(16 * bits)), dtype=np.int64).astype(np.int16)
    wq = ore.unpack(t, bits, cb)
    assert np.array_equal(wq.view(np.uint16), native.exl3_unpack(t, int(2 * bits), ore.CODEBOOK_IDS[cb]).view(np.uint16))
    rows, cols = ore.positions()
    for k in range(2):
        for n in range(2):
            tile = wq[16 * k:16 * k + 16, 16 * n:16 * n + 16].view(np.uint16)
            assert tile[rows, cols].tolist() == slow_tile(t[k, n], bits, cb), (k, n)


def test_stream_ends_and_the_tile():
    for bits in ore.EVERY_WIDTH:
        e = ore.window_ends(bits)
        assert e[-1] == 256 * bits and np.all(np.diff(e) >= 1)
        steps = np.diff(np.concatenate([[0], e]))
        if float(bits).is_integer():
            assert set(steps.tolist()) == {int(bits)}
        else:
            assert steps[0::2].tolist() == [int(bits)] * 128 and steps[1::2].tolist() == [int(bits) + 1] * 128
    for bad in (0, 9, 8.5, 0.5, 2.25):
        with pytest.raises(ValueError):
            ore.check_width(bad)
    rows, cols = ore.positions()
    assert sorted(zip(rows.tolist(), cols.tolist())) == [(r, c) for r in range(16) for c in range(16)]
    # a value's stream position from the prose: lane l holds 8 l .. 8 l + 7; value 8 l + j sits at
    assert (rows[8 * 5 + 3], cols[8 * 5 + 3]) == (2 * 1 + 1 + 8, 1)          # l = 5, j = 3
    assert (rows[8 * 31 + 7], cols[8 * 31 + 7]) == (15, 15)


def test_packed_signs_known_answer():
    """[0b1000_0000_0000_0101, 0] -> -1 at elements 0, 2 and 15 (the reference's tests/test_exl3_format.py:129-134)."""

    signs = np.array([0b1000_0000_0000_0101, 0], dtype=np.uint16).view(np.int16)
    want = np.ones(32, dtype=np.float16)
    want[[0, 2, 15]] = -1
    assert np.array_equal(ore.unpack_signs(signs), want)


def test_hadamard():
    h = ore.hadamard(128)
    i = np.arange(128)
    parity = np.array([bin(v).count("1") & 1 for v in range(128)])
    assert np.array_equal(h, np.where(parity[i[:, None] & i[None, :]] == 1, -1.0, 1.0))
    assert np.allclose((h / np.sqrt(128)) @ (h / np.sqrt(128)), np.eye(128), atol=1e-12)
    x = np.random.default_rng(1).standard_normal((3, 256))
    assert np.allclose(ore.rotate(ore.rotate(x)), x, atol=1e-12)


def test_weight_and_rotated_forward_agree():
    k, n = 256, 384
    rng = np.random.default_rng(3)
    for cb, bits in (("mul1", 2.5), ("mcg", 3), ("3inst", 6)):
        t = rng.integers(-2 ** 15, 2 ** 15, size=(k // 16, n // 16, int(16 * bits)), dtype=np.int64).astype(np.int16)
        suh = (rng.standard_normal(k) * 0.02).astype(np.float16)
        svh = (rng.standard_normal(n) * 0.5).astype(np.float16)
        bias = (rng.standard_normal(n) * 0.1).astype(np.float16)
        x = rng.standard_normal((5, k))
        w = ore.dequantize(t, suh, svh, bits, cb)
        y = ore.forward(x, t, suh, svh, bits, cb, bias)
        assert np.allclose(x @ w + bias.astype(np.float64), y, rtol=1e-12, atol=1e-12)
        xh = x.astype(np.float16)
        c = native.exl3_linear(xh, t, suh, svh, int(2 * bits), ore.CODEBOOK_IDS[cb], bias)
        want = ore.forward(xh, t, suh, svh, bits, cb, bias, half_input=True)
        assert np.abs(c - want).max() <= 1e-5 * np.abs(want).max()


# -- routed experts ----------------------------------------------------------------------------------------------------

def _experts(n_exp, d, width, cb, widths, seed):
    rng = np.random.default_rng(seed)

    def mat(k, n, bits, s_in, s_out):
        t = rng.integers(-2 ** 15, 2 ** 15, size=(k // 16, n // 16, int(16 * bits)), dtype=np.int64).astype(np.int16)
        return t, (rng.standard_normal(k) * s_in).astype(np.float16), (rng.standard_normal(n) * s_out).astype(np.float16)

    gate = [mat(d, width, widths[e % len(widths)], 1 / np.sqrt(d), 1.0) for e in range(n_exp)]
    up = [mat(d, width, widths[(e + 1) % len(widths)], 1 / np.sqrt(d), 1.0) for e in range(n_exp)]
    down = [mat(width, d, widths[(e + 2) % len(widths)], 1 / np.sqrt(width), 0.25) for e in range(n_exp)]
    return gate, up, down


def test_swiglu_pair_known_answers():
    """silu(0) = 0; silu(g) * u at g = ln 3: g / (1 + 1/3) = 0.75 g; the clip caps g from above only and u both ways;
    the bf16 mode rounds g, u, the SiLU and the product in turn."""

    g = np.array([0.0, np.log(3.0), 50.0, -50.0, 2.0])
    u = np.array([5.0, 2.0, -30.0, 30.0, 1.0])
    got = ore.swiglu_pair(g, u)
    assert np.allclose(got[:2], [0.0, 0.75 * np.log(3.0) * 2.0], atol=1e-15)
    clipped = ore.swiglu_pair(g, u, limit=10.0)
    assert np.isclose(clipped[2], 10.0 / (1 + np.exp(-10.0)) * -10.0)
    assert np.isclose(clipped[3], -50.0 / (1 + np.exp(50.0)) * 10.0)             # g is not clipped from below
    from oracle.affine import bf16
    b = ore.swiglu_pair(np.array([1.2345678]), np.array([0.7654321]), act_bf16=True)
    gg, uu = bf16(np.float32([1.2345678]))[0], bf16(np.float32([0.7654321]))[0]
    silu = bf16(np.float32([gg / (1 + np.exp(-np.float64(gg)))]))[0]
    assert b[0] == bf16(np.float32([silu * uu]))[0]


def test_routed_experts_against_the_dense_weights():
    """Without the fp16 input roundings a pair's output is the textbook MLP on dequantize()'s W; a pick outside
    [0, E) contributes nothing; the combine is the weighted sum."""

    n_exp, d, width = 5, 256, 128
    gate, up, down = _experts(n_exp, d, width, "mul1", (2, 2.5, 4), 21)
    rng = np.random.default_rng(22)
    x = rng.standard_normal((3, d))
    pick = np.array([[0, 3, 5], [4, 4, -1], [2, 1, 0]], dtype=np.int32)
    wts = rng.random((3, 3)) + 0.1
    y, out = ore.routed(x, pick, wts, gate, up, down, "mul1", half_input=False)
    for r in range(3):
        for k in range(3):
            e = int(pick[r, k])
            if not 0 <= e < n_exp:
                assert not y[r, k].any()
                continue
            w = [ore.dequantize(m[e][0], m[e][1], m[e][2], m[e][0].shape[-1] / 16, "mul1") for m in (gate, up, down)]
            g, u = x[r] @ w[0], x[r] @ w[1]
            want = (g / (1 + np.exp(-g)) * u) @ w[2]
            assert np.allclose(y[r, k], want, rtol=1e-9, atol=1e-9 * np.abs(want).max())
    assert np.allclose(out, np.einsum("rk,rkd->rd", wts, y))
    # the fp16 roundings of the rotated inputs move the result by about 2^-11 a value, not more
    y16, _ = ore.routed(x, pick, wts, gate, up, down, "mul1")
    assert 0 < np.abs(y16 - y).max() <= 4e-3 * np.abs(y).max()
