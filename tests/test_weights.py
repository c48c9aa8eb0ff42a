"""The load-time steps between a checkpoint's tensors and ``pack`` that need no GPU: the affine dequantization of the
router rows at every stored width, the shared expert folded into two experts, and what ``triple`` refuses."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from tensorfold_amd import synthetic, weights


def slow_dequantize(words: np.ndarray, scales: np.ndarray, biases: np.ndarray, gs: int, bits: int) -> np.ndarray:
    """Element by element from the format's definition: element i of a row is bits [bits i, bits (i + 1)) of the
    row's words taken as one little-endian bit string."""

    n, k = scales.shape[0], scales.shape[1] * gs
    out = np.zeros((n, k), dtype=np.float32)
    for r in range(n):
        for i in range(k):
            at = bits * i
            q = (int(words[r, at // 32]) >> (at % 32)) & ((1 << bits) - 1)
            out[r, i] = np.float32(q) * np.float32(scales[r, i // gs]) + np.float32(biases[r, i // gs])
    return out


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("gs", [32, 64])
def test_dequantize_at_every_stored_width(bits, gs):
    rng = np.random.default_rng(bits * 100 + gs)
    n, k = 5, 2 * gs
    words = rng.integers(0, 2 ** 32, (n, k * bits // 32), dtype=np.uint32)
    scales = torch.from_numpy(rng.uniform(0.01, 0.1, (n, k // gs)).astype(np.float32)).to(torch.bfloat16)
    biases = torch.from_numpy(rng.standard_normal((n, k // gs)).astype(np.float32)).to(torch.bfloat16)
    got = weights.dequantize(torch.from_numpy(words), scales, biases, gs)
    want = slow_dequantize(words, scales.float().numpy(), biases.float().numpy(), gs, bits)
    assert got.dtype == torch.float32 and np.array_equal(got.numpy(), want)
    if bits == 4:
        assert np.array_equal(got.numpy(), ora.dequantize(words, scales.float().numpy(), biases.float().numpy(), gs))


def test_dequantize_keeps_leading_dimensions_and_refuses_odd_shapes():
    w, s, b = synthetic.affine(6, 128, 64, 3, lead=(4,))
    got = weights.dequantize(w, s, b)
    assert got.shape == (4, 6, 128)
    assert torch.equal(got[2], weights.dequantize(w[2], s[2], b[2]))
    with pytest.raises(ValueError):
        weights.dequantize(w[..., :15], s, b)


def test_triple_views_unsigned_words_and_checks_dtypes():
    w, s, b = synthetic.affine(4, 64, 64, 1)
    held = {"p.weight": w.view(torch.uint32), "p.scales": s, "p.biases": b}
    words, scales, biases = weights.triple(held.__getitem__, "p")
    assert words.dtype == torch.int32 and torch.equal(words, w) and scales is s and biases is b
    with pytest.raises(ValueError, match="32-bit"):
        weights.triple({**held, "p.weight": w.to(torch.int64)}.__getitem__, "p")
    with pytest.raises(ValueError, match="floating"):
        weights.triple({**held, "p.scales": s.to(torch.int32)}.__getitem__, "p")
    with pytest.raises(KeyError):
        weights.triple(held.__getitem__, "q")


def test_the_folded_halves_add_up_to_the_shared_expert():
    """Nemotron-H's shared expert is twice a routed expert's width.  As experts E and E + 1 (rows [0, W) and [W, 2 W)
    of its up projection, the matching input halves of its down projection) it gives the same output, in float64."""

    experts, width, d, gs = 3, 64, 128, 64
    fc1, fc2 = synthetic.affine_general(width, d, gs, 1, lead=(experts,)), synthetic.affine_general(d, width, gs, 2, lead=(experts,))
    up, down = synthetic.affine_general(2 * width, d, gs, 3), synthetic.affine_general(d, 2 * width, gs, 4)
    first, second = weights.fold_shared(fc1, fc2, up, down, width, gs)
    assert [tuple(t.shape) for t in first] == [(5, 64, 16), (5, 64, 2), (5, 64, 2)]
    assert [tuple(t.shape) for t in second] == [(5, 128, 8), (5, 128, 1), (5, 128, 1)]
    for t, src in zip(first + second, fc1 + fc2):
        assert torch.equal(t[:experts], src)                      # the routed experts are untouched

    x = synthetic.activations(2, d, 5).double()
    dq = lambda m, e=None: weights.dequantize(*(m if e is None else [t[e] for t in m]), gs).double()
    relu2 = lambda a: a.clamp(min=0) ** 2
    whole = relu2(x @ dq(up).T) @ dq(down).T
    halves = sum(relu2(x @ dq(first, e).T) @ dq(second, e).T for e in (experts, experts + 1))
    assert torch.allclose(whole, halves, rtol=1e-12, atol=1e-12)
    with pytest.raises(ValueError, match="fold"):
        weights.fold_shared(fc1, fc2, tuple(t[0] for t in fc1), down, width, gs)       # a shared expert of W rows
