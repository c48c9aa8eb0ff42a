"""EXL3 on the GPU: the device decoder against the oracle bit for bit (every codebook and width), the layer against
the float64 forward, row invariance, dtypes, layouts (properties after tests/cuda/test_exl3_linear.py)."""

import numpy as np
import pytest
import torch

from oracle import exl3 as ore
from oracle import native
from tensorfold_amd import synthetic
from tensorfold_amd.exl3 import format as fmt
from tensorfold_amd.exl3 import linear
from tests.helpers import rel_l2, max_abs

pytestmark = pytest.mark.gpu
COMBOS = [("3inst", b) for b in (1, 2, 3, 4, 5, 6, 7, 8)] + [("mcg", b) for b in (1, 2, 3, 4, 5, 6, 7, 8)] \
    + [("mul1", b) for b in (1, 1.5, 2, 2.5, 3, 3.5, 4, 5, 6, 7, 8)]
ROWS = (1, 2, 3, 16, 17, 64, 128)


def tensors(codebook, bits, kt=16, nt=8, seed=0):
    rng = np.random.default_rng(seed)
    trellis = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, size=(kt, nt, fmt.tile_words(bits))).astype(np.int16))
    k, n = 16 * kt, 16 * nt
    suh = torch.from_numpy((rng.standard_normal(k) * 0.05).astype(np.float16))
    svh = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float16))
    return trellis, suh, svh


@pytest.mark.parametrize("codebook,bits", COMBOS)
def test_decode_is_bit_exact(codebook, bits):
    trellis, _, _ = tensors(codebook, bits)
    w = linear.unpack_gpu(trellis, codebook)
    ref = ore.unpack(trellis.numpy(), bits, codebook)
    assert np.array_equal(w.cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_config4_decode_is_bit_exact_at_full_size():
    """benchmark configuration 4's gate/up trellis [320, 1088, 48] at 3 bits, all three codebooks, against the C decoder."""

    trellis, suh, svh = synthetic.exl3_layer(5120, 17408, 3, 4000)
    for cb in ("3inst", "mcg", "mul1"):
        layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, cb)
        got = layer.unpack().cpu().numpy().view(np.uint16)
        want = native.exl3_unpack(trellis.numpy(), 6, ore.CODEBOOK_IDS[cb]).view(np.uint16)
        assert np.array_equal(got, want), cb


@pytest.mark.parametrize("m", [1, 8])
@pytest.mark.parametrize("k,n", [(5120, 17408), (17408, 5120)])
def test_config4_projections(k, n, m):
    """benchmark configuration 4: 3.0 bpw, default codebook, fp16 in and out, tokens 1 and 8; rel-L2 <= 2e-3 against the
    float64 forward with the fp16-rounded rotated input (a 1,024-column slice of N for the CPU's sake)."""

    trellis, suh, svh = synthetic.exl3_layer(k, n, 3, 4100 + k // 1000)
    x = synthetic.activations(m, k, 4200 + m, dtype=torch.float16)
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, "3inst")
    y = layer(x.cuda())
    assert y.dtype == torch.float16 and y.shape == (m, n)
    cols = slice(0, 1024)
    want = native.exl3_linear(x.numpy(), trellis.numpy()[:, :64], suh.numpy(), svh.numpy()[cols], 6, 0)
    got = y[:, cols].float().cpu().numpy()
    err = rel_l2(got, want)
    print(f"config 4 K={k} N={n} M={m}: rel-L2 {err:.2e}, max-abs {max_abs(got, want):.3e}")
    assert err <= 2e-3


@pytest.mark.parametrize("codebook,bits", [("mul1", 2), ("mul1", 3), ("mul1", 6), ("3inst", 4), ("mcg", 8),
                                           ("mul1", 2.5)])
@pytest.mark.parametrize("split", [(1, 4), (2, 4), (8, 4), (2, 8), (1, 2)])
def test_row_invariance(codebook, bits, split):
    """Rows 1..128 identical in every window and under every split of K."""

    trellis, suh, svh = tensors(codebook, bits, kt=64)          # K = 1024
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, codebook)
    layer.split = split
    x = synthetic.activations(128, layer.k, 3, dtype=torch.float16).cuda()
    whole = layer(x)
    for m in ROWS:
        assert torch.equal(layer(x[:m]), whole[:m]), f"rows 1..{m}"
        for r in sorted({0, m // 2, m - 1}):
            assert torch.equal(layer(x[r:r + 1])[0], whole[r]), f"row {r} alone vs {m}-row window"
    assert int(layer.counters.abs().sum()) == 0                 # the arrival counters are left zero


@pytest.mark.parametrize("codebook,bits", [("mul1", 2), ("mul1", 4), ("mul1", 6), ("3inst", 8), ("mcg", 4),
                                           ("3inst", 3), ("mul1", 3.5)])
def test_matches_the_float64_reference(codebook, bits):
    trellis, suh, svh = tensors(codebook, bits)
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, codebook)
    x = synthetic.activations(17, layer.k, 5, dtype=torch.float16)
    got = layer(x.cuda(), out_dtype=torch.float32).cpu().numpy()
    want = ore.forward(x.numpy(), trellis.numpy(), suh.numpy(), svh.numpy(), bits, codebook, half_input=True)
    assert rel_l2(got, want) < 2e-3
    # the C statement of the same forward agrees
    c = native.exl3_linear(x.numpy(), trellis.numpy(), suh.numpy(), svh.numpy(), int(2 * bits),
                           ore.CODEBOOK_IDS[codebook])
    assert rel_l2(c, want) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_input_and_output_dtypes(dtype):
    trellis, suh, svh = tensors("mul1", 4)
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, "mul1")
    x = synthetic.activations(8, layer.k, 6, dtype=torch.float32).to(dtype).cuda()
    half = layer(x.half(), out_dtype=torch.float32)
    got = layer(x, out_dtype=torch.float32)
    assert torch.allclose(got, half, rtol=2e-3, atol=2e-3)
    assert layer(x).dtype == dtype and layer(x, out_dtype=torch.bfloat16).dtype == torch.bfloat16


def test_bias_and_the_sign_words_of_older_checkpoints():
    trellis, suh, svh = tensors("mcg", 4)
    bias = torch.from_numpy((np.random.default_rng(2).standard_normal(svh.numel()) * 0.05).astype(np.float16))
    plain = linear.Exl3Linear.from_tensors(trellis, suh, svh, "mcg")
    with_bias = linear.Exl3Linear.from_tensors(trellis, suh, svh, "mcg", bias=bias)
    x = synthetic.activations(3, plain.k, 7, dtype=torch.float16).cuda()
    assert torch.allclose((with_bias(x, out_dtype=torch.float32) - plain(x, out_dtype=torch.float32)).cpu(),
                          bias.float(), rtol=2e-2, atol=2e-2)

    def pack(scales):
        neg = (scales.numpy() < 0).reshape(-1, 16).astype(np.uint16)
        words = (neg * (1 << np.arange(16, dtype=np.uint16))).sum(1).astype(np.uint16)
        return torch.from_numpy(words.view(np.int16).copy())

    signs = linear.Exl3Linear.from_tensors(trellis, pack(suh), pack(svh), "mcg")
    assert torch.equal(signs.suh.cpu(), torch.from_numpy(ore.unpack_signs(pack(suh).numpy())))
    assert torch.equal(signs.svh.cpu(), torch.where(svh < 0, -1.0, 1.0).half())


def test_stored_layout_gives_the_same_bits():
    trellis, suh, svh = tensors("mul1", 3)
    a = linear.Exl3Linear.from_tensors(trellis, suh, svh, "mul1", layout="strips")
    b = linear.Exl3Linear.from_tensors(trellis, suh, svh, "mul1", layout="stored")
    assert a.words.shape != b.words.shape
    x = synthetic.activations(5, a.k, 8, dtype=torch.float16).cuda()
    assert torch.equal(a(x), b(x))
    assert torch.equal(a.unpack(), b.unpack())


def test_bad_arguments_raise():
    trellis, suh, svh = tensors("3inst", 3)
    with pytest.raises(ValueError):
        linear.Exl3Linear.from_tensors(trellis, suh, svh, "2mad")
    with pytest.raises(ValueError):
        linear.Exl3Linear.from_tensors(tensors("mul1", 2.5)[0], suh, svh, "3inst")
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, "3inst")
    with pytest.raises(ValueError):
        layer(torch.zeros((129, layer.k), dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError):
        layer(torch.zeros((1, layer.k + 128), dtype=torch.float16, device="cuda"))
