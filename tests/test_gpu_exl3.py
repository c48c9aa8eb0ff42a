"""The EXL3 linear on the GPU.  Bit-exact: the device decoder against the oracle's bit-by-bit decoder for every codebook
at every width the linear takes, and at benchmark configuration 4's full size against the C decoder.  Within 2e-3: the layer
against the float64 forward that rounds the rotated input to fp16 as the rotation kernel does.  Bit-equal among
themselves: a row alone, in any window of rows, under any split of K, in either stored layout.  (The properties the
reference's tests/cuda/test_exl3_linear.py asks of its kernels.)"""

import dataclasses

import numpy as np
import pytest
import torch

from oracle import exl3 as ore
from oracle import native
from tensorfold_amd import synthetic
from tensorfold_amd.exl3 import format as fmt
from tensorfold_amd.exl3 import linear
from tests.helpers import max_abs, rel_l2

pytestmark = pytest.mark.gpu
WINDOWS = (1, 2, 3, 16, 17, 64, 128)


@dataclasses.dataclass
class Group:
    """A synthetic quantized group: random trellis words, small signed input and output scales."""

    codebook: str
    bits: float
    trellis: torch.Tensor
    suh: torch.Tensor
    svh: torch.Tensor

    @classmethod
    def draw(cls, codebook, bits, k=256, n=128, seed=0):
        rng = np.random.default_rng(seed)
        words = rng.integers(-2 ** 15, 2 ** 15, size=(k // 16, n // 16, fmt.tile_words(bits))).astype(np.int16)
        scale = lambda size: torch.from_numpy((rng.standard_normal(size) * 0.05).astype(np.float16))
        return cls(codebook, bits, torch.from_numpy(words), scale(k), scale(n))

    def layer(self, **kw):
        return linear.Exl3Linear.from_tensors(self.trellis, self.suh, self.svh, self.codebook, **kw)

    def float64(self, x):
        return ore.forward(x.numpy(), self.trellis.numpy(), self.suh.numpy(), self.svh.numpy(), self.bits,
                           self.codebook, half_input=True)


@pytest.mark.parametrize("codebook", list(ore.CODEBOOK_IDS))
def test_every_width_decodes_bit_exactly(codebook):
    """Every width the linear takes: whole bits with any codebook, 1.5 / 2.5 / 3.5 bits with mul1.  (The routed experts
    take every half-bit width with every codebook; tests/test_gpu_exl3_experts.py decodes those.)"""

    for bits in fmt.BITS:
        if codebook != "mul1" and not float(bits).is_integer():
            continue
        g = Group.draw(codebook, bits, seed=int(2 * bits))
        got = linear.unpack_gpu(g.trellis, codebook).cpu().numpy().view(np.uint16)
        assert np.array_equal(got, ore.unpack(g.trellis.numpy(), bits, codebook).view(np.uint16)), bits


def test_config4_decode_is_bit_exact_at_full_size():
    """benchmark configuration 4's gate/up trellis [320, 1088, 48] at 3 bits, all three codebooks, against the C decoder."""

    trellis, suh, svh = synthetic.exl3_layer(5120, 17408, 3, 4000)
    for cb, cb_id in ore.CODEBOOK_IDS.items():
        got = linear.Exl3Linear.from_tensors(trellis, suh, svh, cb).unpack().cpu().numpy().view(np.uint16)
        assert np.array_equal(got, native.exl3_unpack(trellis.numpy(), 6, cb_id).view(np.uint16)), cb


@pytest.mark.parametrize("m", [1, 8])
@pytest.mark.parametrize("k,n", [(5120, 17408), (17408, 5120)])
def test_config4_projections(k, n, m):
    """benchmark configuration 4: 3.0 bpw, default codebook, fp16 in and out, tokens 1 and 8; rel-L2 <= 2e-3 against the
    float64 forward with the fp16-rounded rotated input (a 1,024-column slice of N for the CPU's sake)."""

    trellis, suh, svh = synthetic.exl3_layer(k, n, 3, 4100 + k // 1000)
    x = synthetic.activations(m, k, 4200 + m, dtype=torch.float16)
    y = linear.Exl3Linear.from_tensors(trellis, suh, svh, "3inst")(x.cuda())
    assert y.dtype == torch.float16 and y.shape == (m, n)
    want = native.exl3_linear(x.numpy(), trellis.numpy()[:, :64], suh.numpy(), svh.numpy()[:1024], 6, 0)
    got = y[:, :1024].float().cpu().numpy()
    err = rel_l2(got, want)
    print(f"config 4 K={k} N={n} M={m}: rel-L2 {err:.2e}, max-abs {max_abs(got, want):.3e}")
    assert err <= 2e-3


@pytest.mark.parametrize("split", [(1, 4), (2, 4), (8, 4), (2, 8), (1, 2)])
@pytest.mark.parametrize("codebook,bits", [("mul1", 2), ("mul1", 3), ("mul1", 6), ("3inst", 4), ("mcg", 8), ("mul1", 2.5)])
def test_a_rows_bits_do_not_depend_on_its_window_or_the_split(codebook, bits, split):
    layer = Group.draw(codebook, bits, k=1024).layer()
    layer.split = split
    x = synthetic.activations(max(WINDOWS), layer.k, 3, dtype=torch.float16).cuda()
    whole = layer(x)
    for m in WINDOWS:
        assert torch.equal(layer(x[:m]), whole[:m]), f"the first {m} rows as a window"
        for r in {0, m // 2, m - 1}:
            assert torch.equal(layer(x[r:r + 1])[0], whole[r]), f"row {r} by itself"
    assert not layer.counters.any()                 # the arrival counters of the K splits are left at zero


@pytest.mark.parametrize("codebook,bits", [("mul1", 2), ("mul1", 4), ("mul1", 6), ("3inst", 8), ("mcg", 4),
                                           ("3inst", 3), ("mul1", 3.5)])
def test_the_layer_against_the_float64_forward(codebook, bits):
    g = Group.draw(codebook, bits)
    x = synthetic.activations(17, 256, 5, dtype=torch.float16)
    want = g.float64(x)
    assert rel_l2(g.layer()(x.cuda(), out_dtype=torch.float32).cpu().numpy(), want) < 2e-3
    # the C statement of the same forward agrees with the numpy one
    c = native.exl3_linear(x.numpy(), g.trellis.numpy(), g.suh.numpy(), g.svh.numpy(), int(2 * bits),
                           ore.CODEBOOK_IDS[codebook])
    assert rel_l2(c, want) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_activations_of_any_float_type(dtype):
    layer = Group.draw("mul1", 4).layer()
    x = synthetic.activations(8, layer.k, 6, dtype=torch.float32).to(dtype).cuda()
    as_half = layer(x.half(), out_dtype=torch.float32)
    assert torch.allclose(layer(x, out_dtype=torch.float32), as_half, rtol=2e-3, atol=2e-3)
    assert layer(x).dtype == dtype                                  # the output follows the input unless told
    assert layer(x, out_dtype=torch.bfloat16).dtype == torch.bfloat16


def test_a_bias_is_added_after_the_output_scales():
    g = Group.draw("mcg", 4)
    bias = torch.from_numpy((np.random.default_rng(2).standard_normal(g.svh.numel()) * 0.05).astype(np.float16))
    x = synthetic.activations(3, 256, 7, dtype=torch.float16).cuda()
    delta = g.layer(bias=bias)(x, out_dtype=torch.float32) - g.layer()(x, out_dtype=torch.float32)
    assert torch.allclose(delta.cpu(), bias.float().expand_as(delta), rtol=2e-2, atol=2e-2)


def test_older_checkpoints_store_only_the_signs():
    """int16 words, bit b of word w set when element 16 w + b is negative: they load as vectors of +-1."""

    g = Group.draw("mcg", 4)
    words = lambda v: torch.from_numpy(np.packbits((v.numpy() < 0).reshape(-1, 16), axis=1, bitorder="little")
                                       .view(np.int16).reshape(-1).copy())
    layer = linear.Exl3Linear.from_tensors(g.trellis, words(g.suh), words(g.svh), "mcg")
    for got, scales in ((layer.suh, g.suh), (layer.svh, g.svh)):
        assert torch.equal(got.cpu(), torch.where(scales < 0, -1.0, 1.0).half())
    assert torch.equal(layer.suh.cpu(), torch.from_numpy(ore.unpack_signs(words(g.suh).numpy())))


def test_both_stored_layouts_give_the_same_bits():
    g = Group.draw("mul1", 3)
    strips, stored = g.layer(layout="strips"), g.layer(layout="stored")
    assert strips.words.shape != stored.words.shape
    x = synthetic.activations(5, 256, 8, dtype=torch.float16).cuda()
    assert torch.equal(strips(x), stored(x)) and torch.equal(strips.unpack(), stored.unpack())


@pytest.mark.parametrize("codebook,bits,split", [("3inst", 3, (7, 4)), ("mul1", 2.5, (1, 2)), ("mcg", 4, (3, 8)), ("mul1", 6, (2, 2))])
def test_a_stack_of_layers_gives_each_layer_its_own_bits(codebook, bits, split):
    """Gate and up of an MLP read the same input: stacked, they take one rotation launch and one linear launch, and
    every layer's rows are those of its own call, at any row count."""

    groups = [Group.draw(codebook, bits, k=1024, n=256, seed=40 + i) for i in range(3)]
    bias = torch.from_numpy((np.random.default_rng(3).standard_normal(256) * 0.05).astype(np.float16))
    layers = [groups[0].layer(), groups[1].layer(bias=bias), groups[2].layer()]
    for layer in layers:
        layer.split = split
    stack = linear.Exl3Stack.of(layers)
    assert len(stack) == 3 and stack.split == split and stack.bias is not None
    for m in (1, 8, 17, 128):
        x = synthetic.activations(m, 1024, 50 + m, dtype=torch.float16).cuda()
        got = stack(x)
        assert got.shape == (3, m, 256) and got.dtype == torch.float16
        for i, layer in enumerate(layers):
            assert torch.equal(got[i], layer(x)), (m, i)
            assert torch.equal(stack.layer(i)(x), got[i]), (m, i)
        assert torch.equal(stack(x, out_dtype=torch.float32)[1], layers[1](x, out_dtype=torch.float32))
    assert not stack.counters.any()
    with pytest.raises(ValueError):
        linear.Exl3Stack.of([layers[0], Group.draw(codebook, bits, k=1024, n=128).layer()])
    with pytest.raises(ValueError):
        stack(x, out=torch.empty((2, 128, 256), dtype=torch.float16, device="cuda"))


@pytest.mark.parametrize("codebook,bits,split,mid", [("3inst", 3, (7, 4), torch.float16), ("mul1", 2.5, (1, 2), torch.bfloat16),
                                                     ("mcg", 4, (3, 8), torch.float16), ("mul1", 6, (2, 2), torch.float32)])
def test_an_mlp_in_three_launches(codebook, bits, split, mid):
    """``Exl3MLP``: the workgroups of the gate and up launch apply the SwiGLU and the down projection's rotation
    themselves.  Gate's and up's outputs, the rotated activations and the result have the bits of the stack, the
    producer run as a launch of its own, and the down layer's linear launch; against torch's silu and product on the
    same outputs the result stays within 2e-3; twice in a row on one scratch, rows 1 to 33."""

    from tensorfold_amd import _lib

    k, n = 1024, 768
    gate, up, down = Group.draw(codebook, bits, k=k, n=n, seed=71), Group.draw(codebook, bits, k=k, n=n, seed=72), \
        Group.draw(codebook, bits, k=n, n=k, seed=73)
    bias = torch.from_numpy((np.random.default_rng(5).standard_normal(n) * 0.05).astype(np.float16))
    layers = [gate.layer(), up.layer(bias=bias), down.layer()]
    layers[0].split = layers[1].split = split
    mlp = linear.Exl3MLP.of(*layers)
    stack, dl = linear.Exl3Stack.of(layers[:2]), layers[2]
    for m in (1, 5, 16, 33):
        x = synthetic.activations(m, k, 80 + m, dtype=torch.float16).cuda()
        scratch = mlp.scratch(m)
        y2 = stack(x, out_dtype=mid)
        hh = linear.swiglu_rot_in(y2, dl.suh)
        want = torch.empty((m, k), dtype=torch.float16, device="cuda")
        dsk, dwk = dl.split
        z = torch.empty((dsk * m * k,), dtype=torch.float32, device="cuda")
        _lib.call("tf_exl3_linear", _lib.ptr(hh), _lib.ptr(dl.words), *dl.strides, _lib.ptr(dl.svh), _lib.ptr(dl.bias),
                  _lib.ptr(want), linear._DTYPES[want.dtype], _lib.ptr(z), _lib.ptr(dl.counters), m, dl.k, dl.n, dl.k2,
                  linear.CODEBOOK_IDS[dl.codebook], dsk, dwk)
        for _ in range(2):
            kept = torch.empty((2, m, n), dtype=mid, device="cuda")
            got = mlp(x, mid_dtype=mid, scratch=scratch, mid=kept)
            assert torch.equal(kept, y2) and torch.equal(scratch["hh"][:m], hh) and torch.equal(got, want), m
            assert torch.equal(mlp(x, mid_dtype=mid, scratch=scratch), want), m            # without keeping gate and up
        act = (torch.nn.functional.silu(y2[0].float()).to(mid).float() * y2[1].float()).to(mid)
        ref = dl(act)
        assert rel_l2(got.float().cpu().numpy(), ref.float().cpu().numpy()) <= 2e-3, m
    assert not mlp.gate_up.counters.any() and not dl.counters.any()
    with pytest.raises(ValueError):
        linear.Exl3MLP.of(layers[0], layers[1], layers[0])


@pytest.mark.parametrize("m", [1, 8])
def test_config4_mlp_at_full_size(m):
    """benchmark configuration 4's whole MLP (5120 -> 17408 -> 5120, 3.0 bpw, default codebook, the splits the layers
    choose for themselves) through ``Exl3MLP``, the three launches the benchmark times, straight against the oracle:
    gate and up in full on the CPU, SwiGLU with the roundings of fp16 tensors, then a 1,024-column slice of the down
    projection; rel-L2 <= 2e-3.  ``Exl3Stack`` on the same layers has gate's and up's bits (checked too)."""

    d, width = 5120, 17408
    tg, sug, svg = synthetic.exl3_layer(d, width, 3, 4301)
    tu, suu, svu = synthetic.exl3_layer(d, width, 3, 4302)
    td, sud, svd = synthetic.exl3_layer(width, d, 3, 4303)
    layers = [linear.Exl3Linear.from_tensors(tg, sug, svg, "3inst"), linear.Exl3Linear.from_tensors(tu, suu, svu, "3inst"),
              linear.Exl3Linear.from_tensors(td, sud, svd, "3inst")]
    mlp = linear.Exl3MLP.of(*layers)
    assert mlp.gate_up.split == (7, 4) and mlp.down.split == linear.Exl3Linear.from_tensors(td, sud, svd, "3inst").split
    x = synthetic.activations(m, d, 4310 + m, 0.02, dtype=torch.float16)
    kept = torch.empty((2, m, width), dtype=torch.float16, device="cuda")
    got = mlp(x.cuda(), mid=kept)
    assert torch.equal(linear.Exl3Stack.of(layers[:2])(x.cuda()), kept)
    f16 = lambda a: a.astype(np.float16)
    g = f16(native.exl3_linear(x.numpy(), tg.numpy(), sug.numpy(), svg.numpy(), 6, 0))
    u = f16(native.exl3_linear(x.numpy(), tu.numpy(), suu.numpy(), svu.numpy(), 6, 0))
    assert rel_l2(kept[0].float().cpu().numpy(), g.astype(np.float64)) <= 2e-3
    assert rel_l2(kept[1].float().cpu().numpy(), u.astype(np.float64)) <= 2e-3
    g32 = g.astype(np.float32)
    act = f16(f16(g32 / (1.0 + np.exp(-g32))).astype(np.float32) * u.astype(np.float32))
    assert np.isfinite(act).all() and float(np.abs(act).max()) > 1.0
    want = native.exl3_linear(act, td.numpy()[:, :64], sud.numpy(), svd.numpy()[:1024], 6, 0)
    out = got[:, :1024].float().cpu().numpy()
    err = rel_l2(out, want)
    print(f"config 4 MLP M={m}: rel-L2 {err:.2e}, max-abs {max_abs(out, want):.3e}")
    assert err <= 2e-3


def test_what_the_layer_refuses():
    g = Group.draw("3inst", 3)
    with pytest.raises(ValueError):                                  # no such codebook
        linear.Exl3Linear.from_tensors(g.trellis, g.suh, g.svh, "2mad")
    with pytest.raises(ValueError):                                  # the linear kernel has half-bit widths for mul1 only
        linear.Exl3Linear.from_tensors(Group.draw("mul1", 2.5).trellis, g.suh, g.svh, "3inst")
    layer = g.layer()
    for shape in ((129, layer.k), (1, layer.k + 128)):               # more rows than a decode call takes; a wrong K
        with pytest.raises(ValueError):
            layer(torch.zeros(shape, dtype=torch.float16, device="cuda"))
