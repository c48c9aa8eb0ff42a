"""Pins of the affine-4-bit oracle (CPU only): hand-built words, the one-hot identity, three independent statements
(numpy, C, pure Python), float64 textbook products, closed forms of the epilogues."""

import math

import numpy as np
import pytest

from oracle import affine as ora
from oracle import native


def rng_tables(n, k, gs, seed, lead=()):
    rng = np.random.default_rng(seed)
    words = rng.integers(0, 2 ** 32, size=(*lead, n, k // 8), dtype=np.uint64).astype(np.uint32)
    scales = ora.bf16((rng.random((*lead, n, k // gs)) * 0.02 + 0.001).astype(np.float32))
    biases = ora.bf16((rng.standard_normal((*lead, n, k // gs)) * 0.02).astype(np.float32))
    return words, scales, biases


def test_nibble_order_known_answer():
    """Element 8 w + i is bits [4 i, 4 i + 4) of word w: 0x76543210 reads 0, 1, .. 7; 0xF0000001 reads 1, 0.., 15."""

    got = ora.nibbles(np.array([[0x76543210, 0xF0000001]], dtype=np.uint32))
    assert got.tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, 1, 0, 0, 0, 0, 0, 0, 15]]
    assert np.array_equal(ora.words_from_nibbles(got), np.array([[0x76543210, 0xF0000001]], dtype=np.uint32))


def test_bf16_rounding_known_answers():
    """Round to nearest even on the 16 dropped bits: 1 + 2^-8 is a tie and goes down to 1, 1 + 3 * 2^-8 goes up."""

    x = np.array([1.0, 1 + 2 ** -8, 1 + 2 ** -8 + 2 ** -20, 1 + 3 * 2 ** -8, -2.5, 3.140625], dtype=np.float32)
    assert ora.bf16(x).tolist() == [1.0, 1.0, 1.0078125, 1.015625, -2.5, 3.140625]
    assert ora.bf16_bits(np.array([1.0, -2.0], dtype=np.float32)).tolist() == [0x3F80, 0xC000]


def test_one_hot_rows_read_back_every_nibble():
    """eye(K) @ W.T with scale 1 and bias 0 is the table of codes (the reference's tests/cuda/test_qmm.py:98-111)."""

    words, _, _ = rng_tables(24, 128, 32, 1)
    ones, zeros = np.ones((24, 4), np.float32), np.zeros((24, 4), np.float32)
    y = ora.linear(np.eye(128, dtype=np.float32), words, ones, zeros, 32, f32=True)
    assert np.array_equal(y, ora.nibbles(words).astype(np.float32).T)
    assert set(np.unique(y).tolist()) == set(range(16))


@pytest.mark.parametrize("gs", [32, 64])
def test_three_statements_of_dequantize_agree(gs):
    words, scales, biases = rng_tables(10, 256, gs, 2)
    a = ora.dequantize(words, scales, biases, gs)
    b = native.affine_dequant(words, ora.bf16_bits(scales), ora.bf16_bits(biases), gs)
    assert np.array_equal(a, b)
    for n in range(10):                                        # pure Python, element by element
        for k in (0, 1, 7, 8, 63, 64, 200, 255):
            q = (int(words[n, k // 8]) >> (4 * (k % 8))) & 15
            want = np.float32(np.float32(q) * scales[n, k // gs]) + biases[n, k // gs]
            assert a[n, k] == want


def test_linear_is_the_textbook_product():
    words, scales, biases = rng_tables(48, 512, 64, 3)
    rng = np.random.default_rng(4)
    x = ora.bf16(rng.standard_normal((3, 512)).astype(np.float32))
    w64 = ora.nibbles(words).astype(np.float64) * np.repeat(scales, 64, -1) + np.repeat(biases, 64, -1)
    want = x.astype(np.float64) @ w64.T
    got = ora.linear(x, words, scales, biases, 64, f32=True)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    c = native.affine_linear(ora.bf16_bits(x), words, ora.bf16_bits(scales), ora.bf16_bits(biases), 64)
    assert np.abs(c - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(ora.linear(x, words, scales, biases, 64), ora.bf16(got))
    # prompt form: each weight rounded once first
    wp = ora.prefill_weight(ora.dequantize(words, scales, biases, 64)).astype(np.float64)
    cp = native.affine_linear(ora.bf16_bits(x), words, ora.bf16_bits(scales), ora.bf16_bits(biases), 64, prefill=True)
    assert np.abs(cp - x.astype(np.float64) @ wp.T).max() <= 1e-5 * np.abs(want).max()


def test_group_sums():
    x = np.arange(256, dtype=np.float32).reshape(2, 128)
    assert ora.group_sums(x, 64).tolist() == [[2016.0, 6112.0], [10208.0, 14304.0]]


def test_epilogue_closed_forms():
    """relu^2 on the bf16-rounded input; SwiGLU = bf16(bf16(silu(g)) * u), clipped first when a limit is set."""

    assert ora.relu2(np.array([-3.0, 0.0, 2.0, 1.00390625], np.float32)).tolist() == [0.0, 0.0, 4.0, 1.0]
    g, u = np.array([0.0, 1.0, -20.0, 12.0], np.float32), np.array([5.0, 2.0, 1.0, -30.0], np.float32)
    got = ora.swiglu(g, u)
    silu = [v / (1 + math.exp(-v)) for v in g.tolist()]
    want = [float(ora.bf16(np.float32(ora.bf16(np.float32(s)) * uu))) for s, uu in zip(silu, u.tolist())]
    assert got.tolist() == want and got[0] == 0.0 and abs(got[1] - 1.4609375) < 1e-6
    clipped = ora.swiglu(g, u, limit=10.0)
    assert clipped[3] == float(ora.bf16(np.float32(ora.bf16(np.float32(10 / (1 + math.exp(-10)))) * -10.0)))


def test_combine_is_slot_ordered():
    y = np.array([[[1.0, 2.0], [10.0, 20.0], [100.0, 200.0]]], np.float32)
    w = np.array([[0.5, 0.25, 2.0]], np.float32)
    assert ora.combine(y, w).tolist() == [[203.0, 406.0]]


@pytest.mark.parametrize("swiglu,gs", [(True, 32), (False, 64)])
def test_c_layer_agrees_with_the_numpy_pairs(swiglu, gs):
    """orc_moe_layer (C) against expert_pairs + combine (numpy): same rounding points, different code."""

    e, d, ni, rows, slots = 6, 256, 128, 4, 3
    up = [rng_tables(ni, d, gs, 10 + i, (e,)) for i in range(2 if swiglu else 1)]
    down = rng_tables(d, ni, gs, 20, (e,))
    rng = np.random.default_rng(5)
    x = ora.bf16((rng.standard_normal((rows, d)) * 0.5).astype(np.float32))
    picks = np.stack([rng.permutation(e)[:slots] for _ in range(rows)]).astype(np.int32)
    wts = rng.random((rows, slots)).astype(np.float32)
    act, y = ora.expert_pairs(x, picks, up, down, gs, limit=7.0 if swiglu else 0.0)
    want = ora.combine(y.reshape(rows, slots, d), wts)
    bits = lambda m: (m[0], ora.bf16_bits(m[1]), ora.bf16_bits(m[2]))
    out, act_c, y_c = native.moe_layer(ora.bf16_bits(x), picks, wts, bits(up[0]) if swiglu else None, bits(up[-1]),
                                       bits(down), gs, limit=7.0 if swiglu else 0.0, want_pairs=True)
    assert np.abs(y_c - y).max() <= 1e-4 * np.abs(y).max()
    a_c = ora.bf16_from_bits(act_c)
    assert np.abs(a_c - act).max() <= 2 ** -7 * np.abs(act).max()          # summation order may move a bf16 step
    assert np.abs(ora.bf16_from_bits(out) - want).max() <= 2 ** -7 * np.abs(want).max()


# -- fused producers (add_rmsnorm, add_moe_norm) ----------------------------------------------------------------------

def _norm_case(rows, d, slots, seed):
    rng = np.random.default_rng(seed)
    h = ora.bf16(rng.standard_normal((rows, d)).astype(np.float32))
    y = (rng.standard_normal((rows, slots, d)) * 0.5).astype(np.float32)
    wts = ora.bf16(rng.random((rows, slots)).astype(np.float32) * 0.5 + 0.05)
    w = ora.bf16((rng.random(d) + 0.5).astype(np.float32))
    return h, y, wts, w


def test_rmsnorm_closed_forms():
    """A row of +-c has mean square c^2: with eps = 0 and w = 1 the normed row is +-1 and every group of 64 sums to
    its count of +1 minus its count of -1; without a residual h is x itself."""

    d = 256
    sign = np.where(np.arange(d) % 3 == 0, -1.0, 1.0).astype(np.float32)
    x = (sign * np.float32(0.75))[None, :]
    h, y, xs = ora.add_rmsnorm(x, None, np.ones(d, dtype=np.float32), 0.0)
    assert h is x or np.array_equal(h, x)
    assert np.array_equal(y, sign[None, :])
    assert np.array_equal(xs[0], sign.reshape(4, 64).sum(axis=1))
    # eps enters under the root: x = 3, eps = 16 -> 3 / sqrt(9 + 16) = 0.6 -> bf16
    _, y, _ = ora.add_rmsnorm(np.full((1, 64), 3.0, dtype=np.float32), None, np.ones(64, dtype=np.float32), 16.0)
    assert np.array_equal(y, ora.bf16(np.full((1, 64), 0.6, dtype=np.float32)))


def test_add_rmsnorm_against_float64_and_its_own_outputs():
    h, y3, _, w = _norm_case(5, 384, 1, 11)
    r = ora.bf16(y3[:, 0])
    hn, out, xs = ora.add_rmsnorm(h, r, w, 1e-5, gs=64)
    assert np.array_equal(hn, ora.bf16(h + r))
    h64 = hn.astype(np.float64)
    want = h64 / np.sqrt((h64 ** 2).mean(axis=1, keepdims=True) + 1e-5) * w.astype(np.float64)
    assert np.abs(out - want).max() <= 2 ** -8 * np.abs(want).max()              # one bf16 step
    assert np.allclose(xs, out.reshape(5, 6, 64).sum(axis=2), rtol=1e-6, atol=1e-6)
    _, _, xs32 = ora.add_rmsnorm(h, r, w, 1e-5, gs=32)
    assert np.allclose(xs32.reshape(5, 6, 2).sum(axis=2), xs, rtol=1e-6, atol=1e-5)


def test_moe_delta_weights_the_routed_slots_only():
    """Slots below top_k are weighted, the rest are added as they are; with weights of one the split does not matter;
    moving the boundary or zeroing a routed weight changes the result by that slot's share."""

    h, y, wts, w = _norm_case(3, 128, 5, 12)
    want = (wts[:, :3, None].astype(np.float64) * y[:, :3]).sum(axis=1) + y[:, 3:].astype(np.float64).sum(axis=1)
    got = ora.moe_delta(y, wts, 3)
    assert np.abs(got - want).max() <= 2 ** -8 * np.abs(want).max()
    ones = np.ones_like(wts)
    assert np.array_equal(ora.moe_delta(y, ones, 0), ora.moe_delta(y, ones, 5))
    moved = ora.moe_delta(y, wts, 4)
    step = ((wts[:, 3, None] - 1).astype(np.float64) * y[:, 3])
    assert np.abs((moved - got) - step).max() <= 2 ** -6 * np.abs(want).max()
    assert np.abs(moved - got).max() > 0.05
    hn, out, xs = ora.add_moe_norm(h, y, wts, w, 1e-5, 3)
    assert np.array_equal(hn, ora.bf16(h + got))
    h2, out2, xs2 = ora.add_rmsnorm(h, got, w, 1e-5)
    assert np.array_equal(out, out2) and np.array_equal(xs, xs2) and np.array_equal(hn, h2)


# -- the FP8 prompt path's oracle -----------------------------------------------------------------------------------

def test_e4m3_against_an_independent_conversion_and_known_codes():
    """The numpy e4m3 rounding against torch's float8_e4m3fn (another implementation of the OCP format) over the whole
    range that quantize_rows produces, ties and subnormals included; the value table of all 256 codes; known codes."""

    import torch

    rng = np.random.default_rng(0)
    v = np.concatenate([rng.uniform(-448, 448, 20000), rng.uniform(-1, 1, 20000), rng.uniform(-2 ** -5, 2 ** -5, 20000),
                        [0, 448, -448, 2 ** -9, 2 ** -10, 3 * 2 ** -10, 15.5, 16.5, 17, 18, 232, 240, 248, 463.9]]
                       ).astype(np.float32)
    want = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ora.e4m3_bits(v), want)
    table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    mine = ora.e4m3_values(np.arange(256, dtype=np.uint8))
    assert np.array_equal(mine[~np.isnan(table)], table[~np.isnan(table)])
    assert ora.e4m3_bits(np.float32([1.0, 448.0, -0.5, 2 ** -9])).tolist() == [0x38, 0x7E, 0xB0, 0x01]
    # a 4-bit code in a byte is the e4m3 number code * 2^-9: what lets the packed nibbles be the matrix operand
    assert np.array_equal(ora.e4m3_values(np.arange(16, dtype=np.uint8)), np.arange(16, dtype=np.float32) * 2.0 ** -9)


def test_quantize_rows_closed_forms():
    """The largest magnitude of a row lands on +-448; a row of zeros keeps scale 1; the group sums are the inputs'
    sums over the scale; dequantizing x8 * a gives x back within e4m3's half step (2^-4 relative)."""

    rng = np.random.default_rng(1)
    x = ora.bf16(rng.standard_normal((5, 256)).astype(np.float32))
    x[3] = 0
    x[4, 7] = 50.0
    x8, xs, a = ora.quantize_rows(x, 64)
    v = ora.e4m3_values(x8)
    assert np.array_equal(np.abs(v).max(1)[[0, 1, 2, 4]], np.float32([448] * 4)) and not v[3].any() and a[3] == 1
    assert a[4] == np.float32(50.0) / np.float32(448)
    back = v * a[:, None]
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0 ** -4 + a[:, None] * 2.0 ** -10)
    want = x.reshape(5, 4, 64).astype(np.float64).sum(-1) / a[:, None]
    assert np.all(np.abs(xs - want) <= np.abs(want) * 2.0 ** -8 + 1e-3)


def test_prefill8_is_the_dequantized_product_of_the_quantized_rows():
    """prefill8 on exact inputs: with x already on the e4m3 grid times a power-of-two row scale the quantization is
    lossless, and the result must be the float64 dequant-then-matmul to fp32 rounding."""

    rng = np.random.default_rng(2)
    n, k, gs = 40, 128, 32
    words, scales, biases = rng_tables(n, k, gs, 3)
    grid = ora.e4m3_values(rng.integers(0, 0x7F, (6, k)).astype(np.uint8)) * np.where(rng.random((6, k)) < 0.5, -1, 1)
    grid[:, 0] = 448.0                                              # every row's scale is then 2^-3 exactly
    x = (grid * 0.125).astype(np.float32)
    assert np.array_equal(ora.bf16(x), x)
    x8, xs, a = ora.quantize_rows(x, gs)
    assert np.array_equal(ora.e4m3_values(x8), grid.astype(np.float32)) and np.all(a == 0.125)
    got = ora.prefill8(x8, xs, a, words, scales, biases, gs)
    dense = ora.dequantize(words, scales, biases, gs).astype(np.float64)
    # xs is rounded to bf16 (8 bits): the bias term carries that, so compare the scale term tightly and the whole loosely
    q = ora.nibbles(words).astype(np.float64)
    scale_term = (x.astype(np.float64)[:, None, :] * q[None] * np.repeat(scales.astype(np.float64), gs, 1)[None]).sum(-1)
    bias_term = (xs.astype(np.float64) * a[:, None]) @ biases.astype(np.float64).T
    assert np.allclose(got, scale_term + bias_term, rtol=1e-5, atol=1e-5)
    want = x.astype(np.float64) @ dense.T
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 5e-3
