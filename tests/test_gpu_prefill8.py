"""The FP8 prompt path on the GPU (``qmm.quantize_rows`` + ``qmm.prefill_matmul8``) against the oracle's restatement of
cuda/kernels/qmm.py:222-268 and qmm_prefill8.cu: the quantized rows bit for bit, the matmul to fp32 rounding of the
same exact products, a row's bits whatever the chunking, and the reference's own bound against the float64
dequant-then-matmul (tests/cuda/test_qwen27_prefill.py:216-236: rows in chunks of 1, 7, 16, 64, 256 equal the whole,
relative error under 5e-2)."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from tensorfold_amd import qmm, synthetic
from tests.helpers import bits16, f32, rel_l2, u32

pytestmark = pytest.mark.gpu
DEV = "cuda"
ORDER = np.array([0, 4, 1, 5, 2, 6, 3, 7])          # where each byte of a stored octet comes from


def case(n, k, gs, seed, rows):
    words, scales, biases = synthetic.affine_general(n, k, gs, seed)
    q = qmm.pack(words.to(DEV), scales.to(DEV), biases.to(DEV), gs)
    x = synthetic.activations(rows, k, seed + 1)
    x[:, 5] *= 50                                                   # an outlier channel, as the reference's test has
    return q, x, (u32(words), f32(scales), f32(biases))


@pytest.mark.parametrize("gs", [64, 32])
def test_quantized_rows_are_the_oracles(gs):
    x = synthetic.activations(37, 512, 70 + gs, 3.0)
    x[3] = 0                                                        # a row of zeros keeps scale 1
    x[:, 9] *= 40
    x8, xs, a = qmm.quantize_rows(x.to(DEV), gs)
    want8, want_xs, want_a = ora.quantize_rows(f32(x), gs)
    assert np.array_equal(a.cpu().numpy(), want_a)
    stored = x8.cpu().numpy().reshape(37, -1, 8)
    assert np.array_equal(stored, want8.reshape(37, -1, 8)[:, :, ORDER])
    assert np.array_equal(bits16(xs), ora.bf16_bits(want_xs))
    # a strided view of a wider buffer gives the same
    wide = torch.zeros((37, 1024), dtype=torch.bfloat16, device=DEV)
    wide[:, :512] = x.to(DEV)
    again = qmm.quantize_rows(wide[:, :512], gs)
    assert all(torch.equal(p, r) for p, r in zip(again, (x8, xs, a)))


@pytest.mark.parametrize("f32_out", [True, False])
@pytest.mark.parametrize("n,k,gs,rows", [(1000, 1024, 64, 333), (1000, 1024, 32, 333), (192, 448, 32, 5),
                                         (520, 2048, 64, 130), (64, 64, 64, 1)])
def test_against_the_oracle_and_the_float64_product(n, k, gs, rows, f32_out):
    q, x, (words, scales, biases) = case(n, k, gs, 80 + gs + rows, rows)
    xq = qmm.quantize_rows(x.to(DEV), gs)
    got = f32(qmm.prefill_matmul8(xq, q, f32=f32_out))
    x8, xs, a = ora.quantize_rows(f32(x), gs)
    want = ora.prefill8(x8, xs, a, words, scales, biases, gs)
    if not f32_out:
        want = ora.bf16(want)
    # The same exact products, summed by the matrix unit where the oracle sums in float64.  The unit does not keep a
    # group's sum to fp32 precision: the 32 products of an instruction are aligned to the largest and about 13 bits
    # below it survive (one group of exact operands is off by up to 2^-12 of its largest product), which shows as
    # 2e-5 to 3e-5 relative L2 here.
    assert rel_l2(got, want) <= (1e-4 if f32_out else 2e-3)
    dense = ora.dequantize(words, scales, biases, gs).astype(np.float64)
    ref = f32(x).astype(np.float64) @ dense.T
    err = rel_l2(got, ref)
    print(f"prefill8 {rows}x{k}x{n} g{gs}: rel-L2 {err:.2e} against the float64 dequant-then-matmul")
    assert err < 5e-2


@pytest.mark.parametrize("gs", [64, 32])
def test_a_rows_bits_do_not_depend_on_the_chunking(gs):
    q, x, _ = case(1000, 1024, gs, 90 + gs, 333)
    xd = x.to(DEV)
    run = lambda rows, tile=0: qmm.prefill_matmul8(qmm.quantize_rows(rows.contiguous(), gs), q, f32=True, tile=tile)
    whole = run(xd)
    for tile in (1, 2):
        assert torch.equal(whole, run(xd, tile))
    for size in (1, 7, 16, 64, 256):
        assert torch.equal(whole, torch.cat([run(xd[a:a + size]) for a in range(0, 333, size)])), size


def test_what_the_path_refuses():
    q, x, _ = case(128, 256, 64, 99, 4)
    with pytest.raises(ValueError):
        qmm.quantize_rows(x.to(DEV)[:, :48], 32)                    # K not a multiple of the group
    with pytest.raises(ValueError):
        qmm.quantize_rows(x.to(DEV).float(), 64)                    # bf16 only
    xq = qmm.quantize_rows(x.to(DEV), 64)
    with pytest.raises(ValueError):
        qmm.prefill_matmul8((xq[0][:, :128], xq[1], xq[2]), q)      # inputs of another K
    with pytest.raises(ValueError):
        qmm.prefill_matmul8(qmm.quantize_rows(x.to(DEV), 32), q)    # sums of another group size
    with pytest.raises(ValueError):
        qmm.prefill_matmul8(xq, q, out=torch.empty((4, 128), dtype=torch.float32, device=DEV))    # bf16 asked, fp32 given
