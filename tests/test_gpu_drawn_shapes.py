"""Drawn shapes through every kernel family: sizes off the benchmark's grid (odd column counts, K that is not whole
steps of 64, one expert, one row, many rows) against the CPU oracle, with the invariances the reference's tests ask for
(rows alone equal rows in a batch; every item size gives the same bits; every K split stays inside the bound)."""

import random

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import exl3 as ore
from oracle import native
from oracle import routing as orr
from tensorfold_amd import experts, moe, qmm, synthetic
from tensorfold_amd.exl3 import format as fmt
from tensorfold_amd.exl3 import linear
from tests.helpers import bits16, f32, rel_l2, u32
from tests.test_gpu_moe import layer_tables

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3


@pytest.mark.parametrize("seed", range(10))
def test_dense_projection(seed):
    rnd = random.Random(1000 + seed)
    gs = rnd.choice([32, 64])
    n = rnd.choice([1, 7, 32, 48, 64, 100, 128, 200, 256, 513, 1000, 1536])
    k = gs * rnd.randint(1, 60)
    m = rnd.choice([1, 2, 3, 7, 8, 9, 16, 17, 33, 64, 65, 100, 129, 257])
    w = synthetic.affine_general(n, k, gs, 7000 + seed)
    x = synthetic.activations(m, k, 8000 + seed)
    q = qmm.pack(*(t.to(DEV) for t in w), gs)
    ref = native.affine_linear(bits16(x), u32(w[0]), bits16(w[1]), bits16(w[2]), gs)
    xd = x.to(DEV)
    ran = 0
    for sk in (None, 1, 2, 16):
        try:
            y = qmm.matmul(xd, q, f32=True, sk=sk)
        except (ValueError, RuntimeError):
            continue                            # K does not cut into that many slices of whole groups
        ran += 1
        assert rel_l2(f32(y), ref) <= TOL, sk
    assert ran >= 2                             # the shape's own split and one slice always run
    yp = qmm.prefill_matmul(xd, q, f32=True)
    assert rel_l2(f32(yp), ref) <= TOL
    r = rnd.randrange(m)
    assert torch.equal(qmm.prefill_matmul(xd[r:r + 1].contiguous(), q, f32=True)[0], yp[r])
    assert torch.equal(qmm.matmul(xd[r:r + 1].contiguous(), q, f32=True)[0], qmm.matmul(xd, q, f32=True)[r])


@pytest.mark.parametrize("seed", range(10))
def test_routed_experts_both_forms(seed):
    rnd = random.Random(2000 + seed)
    gs = rnd.choice([32, 64])
    hidden, width = 32 * rnd.randint(1, 24), 32 * rnd.randint(1, 20)
    if gs == 64:
        hidden, width = (hidden + 63) // 64 * 64, (width + 63) // 64 * 64
    ne = rnd.choice([1, 2, 5, 16, 33, 64])
    top_k = rnd.randint(1, min(6, ne))
    swiglu = rnd.random() < 0.5
    rows = rnd.choice([1, 5, 16, 40, 130, 300, 700])
    shape = synthetic.MoEShape(f"drawn{seed}", hidden, ne, width, top_k, gs, swiglu, False)
    up, down = layer_tables(shape, 9000 + seed, ne)
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), gs)
    x = synthetic.activations(rows, hidden, 9500 + seed)
    picks = (synthetic.zipf_picks(rows, ne, top_k, 9600 + seed) if ne > 1
             else torch.zeros((rows, top_k), dtype=torch.int32)).contiguous()
    wts = torch.softmax(synthetic.logits(rows, top_k, 9700 + seed), 1).bfloat16().float().contiguous()
    outs = {}
    for tile, form in ((16, "prompt"), (64, "prompt"), (128, "prompt"), (16, "decode")):
        plan = experts.Plan(rows, top_k, ne, DEV, prefill=form == "prompt")
        experts.route(picks.to(DEV), plan, tile)
        items, members, _ = orr.plan(picks.numpy(), ne, tile)
        assert np.array_equal(plan.members.cpu().numpy(), members)
        assert np.array_equal(plan.items[:int(plan.counts[0])].cpu().numpy(), items)
        act = torch.empty((rows * top_k, width), dtype=torch.bfloat16, device=DEV)
        y = torch.empty((rows * top_k, hidden), dtype=torch.float32, device=DEV)
        experts.gate_up(x.to(DEV), ex, plan, act, rows)
        experts.down(act, ex, plan, y, rows)
        outs[(tile, form)] = moe.combine(y.view(rows, -1, hidden), wts.to(DEV)).clone()
    assert torch.equal(outs[(16, "prompt")], outs[(64, "prompt")])
    assert torch.equal(outs[(64, "prompt")], outs[(128, "prompt")])
    sample = sorted(rnd.sample(range(rows), min(rows, 6)))
    t = lambda m: (u32(m[0]), bits16(m[1]), bits16(m[2]))
    def want(form):
        return ora.bf16_from_bits(native.moe_layer(bits16(x[sample]), picks[sample].numpy(), wts[sample].numpy(),
                                                   t(up[0]) if swiglu else None, t(up[1]) if swiglu else t(up[0]),
                                                   t(down), gs, prefill=form))
    # a relu^2 layer's prompt form is the reference's bf16 arithmetic (weights rounded to bf16 once, the oracle's
    # form 2), which by itself sits past the bound from the unrounded weights; everything else against those
    for key, o in outs.items():
        bf16_form = key[1] == "prompt" and ex.arith == experts.ARITH_BF16
        assert rel_l2(f32(o[sample]), want(2 if bf16_form else 0)) <= TOL, key


@pytest.mark.parametrize("seed", range(10))
def test_exl3_layer(seed):
    rnd = random.Random(500 + seed)
    cb = rnd.choice(["3inst", "mcg", "mul1"])
    bits = rnd.choice([1, 2, 3, 4, 5, 6, 7, 8] + ([1.5, 2.5, 3.5] if cb == "mul1" else []))
    k, n = 128 * rnd.randint(1, 24), 128 * rnd.randint(1, 6)
    m = rnd.choice([1, 2, 3, 8, 16, 17, 31, 64, 100, 128])
    rng = np.random.default_rng(seed)
    trellis = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15,
                                            size=(k // 16, n // 16, fmt.tile_words(bits))).astype(np.int16))
    suh = torch.from_numpy((rng.standard_normal(k) * 0.05).astype(np.float16))
    svh = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float16))
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, cb)
    x = synthetic.activations(m, k, 600 + seed, dtype=torch.float16)
    xd = x.to(DEV)
    want = native.exl3_linear(x.numpy(), trellis.numpy(), suh.numpy(), svh.numpy(), int(2 * bits),
                              ore.CODEBOOK_IDS[cb])
    ran = 0
    for split in (layer.split, (1, 4), (1, 2), (2, 4), (4, 2), (8, 4), (16, 4), (2, 8)):
        layer.split = split
        try:
            got = layer(xd, out_dtype=torch.float32)
        except (ValueError, RuntimeError):
            continue                            # K's tile pairs do not divide over that many waves
        ran += 1
        assert rel_l2(got.cpu().numpy(), want) < TOL, split
        r = rnd.randrange(m)
        assert torch.equal(layer(xd[r:r + 1], out_dtype=torch.float32)[0], got[r]), split
        assert int(layer.counters.abs().sum()) == 0
    assert ran >= 2


@pytest.mark.parametrize("seed", range(8))
def test_drawn_exl3_prompt_matmuls(seed):
    """Shapes off the benchmark's grid through the decode-once GEMM: any M, N of 1 to 5 blocks of 128 (part-filled
    256-column tiles), K down to one block, every codebook."""

    from tensorfold_amd.exl3 import prefill

    rng = np.random.default_rng(900 + seed)
    codebook = ("3inst", "mcg", "mul1")[seed % 3]
    bits = (2, 3, 4, 5, 6, 8)[int(rng.integers(6))] if codebook != "mul1" else (1.5, 2.5, 3.5, 4)[int(rng.integers(4))]
    kt, nt, m = 8 * int(rng.integers(1, 6)), 8 * int(rng.integers(1, 6)), int(rng.integers(1, 300))
    trellis = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, size=(kt, nt, int(16 * bits))).astype(np.int16))
    k, n = 16 * kt, 16 * nt
    suh = torch.from_numpy((rng.standard_normal(k) * 0.05).astype(np.float16))
    svh = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float16))
    layer = linear.Exl3Linear.from_tensors(trellis, suh, svh, codebook)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float16))
    out = torch.full((m + 1, n + 2), 7.0, dtype=torch.float32, device=DEV)          # strided rows, a guard row below
    prefill.matmul(layer, x.to(DEV), out[:m, :n], prefill.Workspace())
    want = ore.forward(x.numpy(), trellis.numpy(), suh.numpy(), svh.numpy(), bits, codebook, half_input=True)
    assert rel_l2(out[:m, :n].cpu().numpy(), want) < TOL, (codebook, bits, k, n, m)
    assert (out[m] == 7.0).all() and (out[:, n:] == 7.0).all()
