"""The committed fixtures (tests/golden/fixtures.json) replayed: known answers the reference's tests hold against the
oracle (numpy and C), regression vectors against the oracle on the CPU and against the kernels on the GPU."""

import json
import pathlib

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import exl3 as ore
from oracle import native
from oracle import routing as orr

FIX = json.loads((pathlib.Path(__file__).parent / "golden" / "fixtures.json").read_text())
KA, REG = FIX["known_answers"], FIX["regression"]


def test_known_answers_of_the_reference_tests():
    s = KA["packed_signs"]
    signs = ore.unpack_signs(np.array(s["words"], dtype=np.uint16).view(np.int16))
    assert signs.shape == (s["length"],)
    assert sorted(np.nonzero(signs < 0)[0].tolist()) == s["negative_at"] and set(np.abs(signs).tolist()) == {1.0}
    p = KA["plan_one_expert"]
    items, members, distinct = orr.plan(np.full((p["rows"], 1), p["expert"], np.int32), p["experts"], p["tile"])
    assert items[:, 2].tolist() == p["item_counts"] and set(items[:, 0].tolist()) == {p["expert"]} and distinct == 1
    assert members.tolist() == list(range(p["rows"]))
    t = KA["ties"]
    picks, wts = orr.topk_rows(np.zeros((2, t["experts"]), np.float32), t["experts"], t["top_k"], shared=False)
    assert picks.tolist() == [t["ids"]] * 2
    assert np.all(wts == ora.bf16(np.float32(t["weight"])))
    n = KA["nibble_order"]
    assert ora.nibbles(np.array([n["word"]], dtype=np.uint32)).tolist() == n["codes"]
    assert native.affine_dequant(np.array([[n["word"]] * 8], np.uint32), ora.bf16_bits(np.ones((1, 1), np.float32)),
                                 ora.bf16_bits(np.zeros((1, 1), np.float32)), 64)[0, :8].tolist() == n["codes"]


def test_regression_vectors_on_the_cpu():
    a = REG["affine"]
    words = np.array(a["words"], dtype=np.uint32)
    s_bits, b_bits = np.array(a["scales_bits"], np.uint16), np.array(a["biases_bits"], np.uint16)
    x_bits = np.array(a["x_bits"], np.uint16)
    y = ora.linear(ora.bf16_from_bits(x_bits), words, ora.bf16_from_bits(s_bits), ora.bf16_from_bits(b_bits), a["gs"])
    assert ora.bf16_bits(y).tolist() == a["y_bits"]
    yc = native.affine_linear(x_bits, words, s_bits, b_bits, a["gs"])
    assert np.abs(yc - ora.bf16_from_bits(np.array(a["y_bits"], np.uint16))).max() <= 2 ** -7 * np.abs(yc).max()
    r = REG["routing"]
    picks, wts = orr.topk_rows(np.array(r["logits"], np.float32), r["experts"], r["top_k"], shared=True)
    assert picks.tolist() == r["picks"] and wts.astype(np.float64).tolist() == r["weights"]
    items, members, distinct = orr.plan(picks, r["experts"] + 1, 16)
    assert items.tolist() == r["items"] and members.tolist() == r["members"] and distinct == r["distinct"]
    for cb, e in REG["exl3"].items():
        trellis = np.array(e["trellis"], np.int16).reshape(1, 1, -1)
        assert ore.unpack(trellis, e["bits"], cb).view(np.uint16).reshape(-1).tolist() == e["values_fp16_bits"]
        got = native.exl3_unpack(trellis, int(2 * e["bits"]), ore.CODEBOOK_IDS[cb])
        assert got.view(np.uint16).reshape(-1).tolist() == e["values_fp16_bits"]


@pytest.mark.gpu
def test_regression_vectors_on_the_gpu():
    from tensorfold_amd import experts, moe, qmm
    from tensorfold_amd.exl3 import linear

    dev = "cuda"
    a = REG["affine"]
    as_bf16 = lambda bits: torch.from_numpy(np.array(bits, np.uint16).view(np.int16)).view(torch.bfloat16)
    words = torch.from_numpy(np.array(a["words"], dtype=np.uint32).view(np.int32))
    q = qmm.pack(words.to(dev), as_bf16(a["scales_bits"]).to(dev), as_bf16(a["biases_bits"]).to(dev), a["gs"])
    y = qmm.matmul(as_bf16(a["x_bits"]).to(dev), q)
    want = ora.bf16_from_bits(np.array(a["y_bits"], np.uint16))
    got = y.float().cpu().numpy()
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max()       # one bf16 step: a different fp32 order
    r = REG["routing"]
    cfg = type("c", (), dict(num_experts_per_tok=r["top_k"], num_experts=r["experts"], moe_intermediate_size=32,
                             hidden_size=32))
    buf = moe.MoEBuffers(4, cfg, dev, shared=True)
    moe.select(torch.tensor(r["logits"], dtype=torch.float32, device=dev), buf, r["top_k"], r["experts"],
               tile=experts.TILE)
    assert buf.pick.cpu().tolist() == r["picks"]
    assert buf.wts.cpu().double().tolist() == r["weights"]
    n = int(buf.plan.counts[0])
    assert buf.plan.items[:n].cpu().tolist() == r["items"] and buf.plan.members.cpu().tolist() == r["members"]
    for cb, e in REG["exl3"].items():
        # the kernels take whole 128 x 128 blocks: the tile repeated 8 x 8 times must decode to 64 copies
        trellis = torch.from_numpy(np.array(e["trellis"], np.int16).reshape(1, 1, -1)).repeat(8, 8, 1)
        w = linear.unpack_gpu(trellis, cb).cpu().view(torch.int16).numpy().view(np.uint16)
        want = np.array(e["values_fp16_bits"], np.uint16).reshape(16, 16)
        assert np.array_equal(w.reshape(8, 16, 8, 16), np.broadcast_to(want[None, :, None, :], (8, 16, 8, 16)))
