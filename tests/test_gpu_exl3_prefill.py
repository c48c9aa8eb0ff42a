"""The EXL3 prompt matmul on the GPU (decode once, fp16 GEMM, rotated epilogue) against the float64 forward, the
decode-form layer and its own invariances (properties after the reference's tests/cuda/test_exl3_prefill.py: any M, a
row's bits independent of its chunk, either layout, strided output rows)."""

import numpy as np
import pytest
import torch

from oracle import exl3 as ore
from oracle import native
from tensorfold_amd import synthetic
from tensorfold_amd.exl3 import format as fmt
from tensorfold_amd.exl3 import linear, prefill
from tests.helpers import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"


def layer_of(codebook, bits, kt, nt, seed, bias=False, layout="strips"):
    rng = np.random.default_rng(seed)
    trellis = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, size=(kt, nt, fmt.tile_words(bits))).astype(np.int16))
    k, n = 16 * kt, 16 * nt
    suh = torch.from_numpy((rng.standard_normal(k) * 0.05).astype(np.float16))
    svh = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float16))
    b = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float16)) if bias else None
    return linear.Exl3Linear.from_tensors(trellis, suh, svh, codebook, bias=b, layout=layout), trellis, suh, svh, b


def test_the_operand_order_decode_is_the_decode():
    for codebook, bits in (("3inst", 3), ("mcg", 4), ("mul1", 2.5), ("mul1", 8)):
        layer, trellis, _, _, _ = layer_of(codebook, bits, 16, 24, 3)
        wt = prefill.decode(layer, prefill.Workspace())
        assert wt.shape == (layer.k // 8, layer.n, 8)
        plain = wt.permute(0, 2, 1).reshape(layer.k, layer.n)
        assert torch.equal(plain, layer.unpack())
        want = ore.unpack(trellis.numpy(), bits, codebook)
        assert np.array_equal(plain.cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("codebook,bits,kt,nt,m,bias", [("3inst", 3, 32, 16, 1, False), ("3inst", 3, 32, 16, 200, True),
                                                        ("mcg", 4, 8, 8, 17, False), ("mul1", 2.5, 24, 40, 130, True),
                                                        ("mul1", 6, 16, 8, 128, False), ("3inst", 8, 8, 16, 129, False)])
def test_matches_the_float64_forward(codebook, bits, kt, nt, m, bias):
    layer, trellis, suh, svh, b = layer_of(codebook, bits, kt, nt, 11 + m, bias)
    x = synthetic.activations(m, layer.k, 20 + m, dtype=torch.float16)
    out = torch.empty((m, layer.n), dtype=torch.float32, device=DEV)
    prefill.matmul(layer, x.to(DEV), out, prefill.Workspace())
    want = ore.forward(x.numpy(), trellis.numpy(), suh.numpy(), svh.numpy(), bits, codebook,
                       bias=None if b is None else b.numpy(), half_input=True)
    err = rel_l2(out.cpu().numpy(), want)
    print(f"exl3 prompt matmul {codebook} {bits} bpw K={layer.k} N={layer.n} M={m}: rel-L2 {err:.2e}")
    assert err < 2e-3
    # and close to the decode-form layer on the same rows (different summation order, same operands)
    rows = slice(0, min(m, 128))
    dec = layer(x[rows].to(DEV), out_dtype=torch.float32)
    assert rel_l2(out[rows].cpu().numpy(), dec.cpu().numpy()) < 1e-3


def test_a_row_does_not_depend_on_its_chunk():
    layer, _, _, _, _ = layer_of("3inst", 3, 40, 16, 5, bias=True)
    ws = prefill.Workspace()
    x = synthetic.activations(300, layer.k, 6, dtype=torch.float16).to(DEV)
    whole = prefill.matmul(layer, x, torch.empty((300, layer.n), dtype=torch.float16, device=DEV), ws).clone()
    wt = prefill.decode(layer, ws)
    for m in (1, 2, 127, 128, 129, 256, 299):
        part = prefill.matmul(layer, x[:m], torch.empty((m, layer.n), dtype=torch.float16, device=DEV), ws, wt=wt)
        assert torch.equal(part, whole[:m]), m
    for r in (0, 77, 128, 299):
        one = prefill.matmul(layer, x[r:r + 1], torch.empty((1, layer.n), dtype=torch.float16, device=DEV), ws, wt=wt)
        assert torch.equal(one[0], whole[r]), r


def test_layouts_dtypes_and_strided_output():
    a, trellis, suh, svh, _ = layer_of("mul1", 3, 16, 16, 9, layout="strips")
    b = linear.Exl3Linear.from_tensors(trellis, suh, svh, "mul1", layout="stored")
    ws = prefill.Workspace()
    x = synthetic.activations(40, a.k, 10, dtype=torch.float32).to(DEV)
    ya = prefill.matmul(a, x.half(), torch.empty((40, a.n), dtype=torch.float32, device=DEV), ws).clone()
    yb = prefill.matmul(b, x.half(), torch.empty((40, a.n), dtype=torch.float32, device=DEV), ws).clone()
    assert torch.equal(ya, yb)                                   # either stored order decodes to the same weight
    for dtype in (torch.bfloat16, torch.float32):
        y = prefill.matmul(a, x.to(dtype), torch.empty((40, a.n), dtype=dtype, device=DEV), ws)
        assert y.dtype == dtype and rel_l2(y.float().cpu().numpy(), ya.cpu().numpy()) < 1e-2
    wide = torch.zeros((40, a.n + 64), dtype=torch.float16, device=DEV)
    prefill.matmul(a, x.half(), wide[:, :a.n], ws)                # rows a.n + 64 elements apart
    assert torch.equal(wide[:, :a.n].float(), ya.half().float()) and float(wide[:, a.n:].abs().sum()) == 0.0
    assert ws.nbytes() >= 2 * a.k * a.n


def test_config4_gate_projection_chunk():
    """benchmark configuration 4's gate/up shape (K 5120, N 17408, 3.0 bpw) on a 512-row chunk: a 1,024-column slice and 12
    sampled rows against the C forward; the rest against the decode-form layer's rows."""

    trellis, suh, svh = synthetic.exl3_layer(5120, 17408, 3, 4100)
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, "3inst")
    x = synthetic.activations(512, 5120, 4300, dtype=torch.float16)
    out = torch.empty((512, 17408), dtype=torch.float16, device=DEV)
    prefill.matmul(layer, x.to(DEV), out, prefill.Workspace())
    rows = list(range(0, 512, 43))
    cols = slice(0, 1024)
    want = native.exl3_linear(x[rows].numpy(), trellis.numpy()[:, :64], suh.numpy(), svh.numpy()[cols], 6, 0)
    err = rel_l2(out[rows][:, cols].float().cpu().numpy(), want)
    print(f"config 4 gate projection, 512-row chunk: rel-L2 {err:.2e}")
    assert err < 2e-3
    dec = layer(x[:64].to(DEV))
    assert rel_l2(out[:64].float().cpu().numpy(), dec.float().cpu().numpy()) < 2e-3


def test_bad_arguments_raise():
    layer, _, _, _, _ = layer_of("mcg", 4, 8, 16, 1)
    ws = prefill.Workspace()
    x = torch.zeros((4, layer.k), dtype=torch.float16, device=DEV)
    with pytest.raises(ValueError):
        prefill.matmul(layer, x[:, :64], torch.empty((4, layer.n), dtype=torch.float16, device=DEV), ws)
    with pytest.raises(ValueError):
        prefill.matmul(layer, x, torch.empty((5, layer.n), dtype=torch.float16, device=DEV), ws)
    with pytest.raises(ValueError):
        prefill.matmul(layer, x, torch.empty((4, layer.n), dtype=torch.float16, device=DEV), ws,
                       wt=torch.empty((layer.k, layer.n), dtype=torch.float16, device=DEV))
    with pytest.raises(ValueError):
        prefill.matmul(layer, x, torch.empty((4, layer.n), dtype=torch.int32, device=DEV), ws)
