"""EXL3 routed experts on the GPU (a width per expert, any codebook) against the float64 restatement, and their own
invariances (after the reference's tests/cuda/test_exl3_experts.py: the kernels' decode bit for bit, mixed widths, rows
independent of the window, the fused down + combine equal to the separate launches, graph replay)."""

import numpy as np
import pytest
import torch

from oracle import exl3 as ore
from tensorfold_amd import experts as grouped
from tensorfold_amd.exl3 import experts
from tests.helpers import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3


def make_layer(n_exp, d, width, cb, widths, seed):
    """widths: e -> (gate, up, down) bits.  Returns (Exl3RoutedExperts, numpy triples for the oracle)."""

    rng = np.random.default_rng(seed)

    def mat(k, n, bits, s_in, s_out):
        t = rng.integers(-2 ** 15, 2 ** 15, size=(k // 16, n // 16, int(16 * bits)), dtype=np.int64).astype(np.int16)
        return t, (rng.standard_normal(k) * s_in).astype(np.float16), (rng.standard_normal(n) * s_out).astype(np.float16)

    gate, up, down = [], [], []
    for e in range(n_exp):
        bg, bu, bd = widths(e)
        gate.append(mat(d, width, bg, 1 / np.sqrt(d), 1.0))
        up.append(mat(d, width, bu, 1 / np.sqrt(d), 1.0))
        down.append(mat(width, d, bd, 1 / np.sqrt(width), 0.25))

    def dev(ms):
        return [tuple(torch.from_numpy(a).to(DEV) for a in m) for m in ms]

    return experts.prepare(dev(gate), dev(up), dev(down), cb), (gate, up, down)


def picks(n_exp, rows, k, seed, shared=False):
    g = torch.Generator().manual_seed(seed)
    sel = torch.stack([torch.randperm(n_exp, generator=g)[:k] for _ in range(rows)]).to(torch.int32)
    w = torch.rand((rows, k), generator=g) * 0.2 + 0.05
    if shared:
        sel = torch.cat([sel, torch.full((rows, 1), n_exp, dtype=torch.int32)], 1)
        w = torch.cat([w, torch.ones((rows, 1))], 1)
    return sel.to(DEV).contiguous(), w.float().to(DEV).contiguous()


MIXED = [
    ("mul1", lambda e: (2 + (e % 3), 2 + (e % 3), 2 + ((e + 1) % 3))),
    ("mul1", lambda e: ((1, 1.5, 2.5, 3, 3.5, 4, 5, 6, 7, 8)[e % 10],) * 2 + ((1.5, 2.5, 3.5, 4, 8)[e % 5],)),
    ("mcg", lambda e: ((1, 2, 3, 4, 5, 6, 7, 8)[e % 8],) * 2 + ((2, 3, 4)[e % 3],)),
    ("3inst", lambda e: ((1, 2, 3, 4, 5, 6, 7, 8)[(e + 3) % 8],) * 2 + ((4, 3, 8)[e % 3],)),
    # the half-bit widths past 3.5 and half-bit widths off the mul1 codebook (the reference's experts take every count)
    ("3inst", lambda e: ((4.5, 5.5, 6.5, 7.5, 1.5, 2.5, 3.5)[e % 7],) * 2 + ((4.5, 7.5, 2.5)[e % 3],)),
    ("mcg", lambda e: ((7.5, 6.5, 5.5, 4.5)[e % 4],) * 2 + ((5.5, 6.5)[e % 2],)),
    ("mul1", lambda e: ((4.5, 5.5, 6.5, 7.5)[e % 4],) * 2 + ((7.5, 4.5, 6.5)[e % 3],)),
]


def test_the_kernels_decode_is_the_bitstream():
    rng = np.random.default_rng(5)
    for cb in ("3inst", "mcg", "mul1"):
        for k2 in experts.K2_SUPPORTED[experts.codebook_id(cb)]:
            t = rng.integers(-2 ** 15, 2 ** 15, size=(8, 16, 8 * k2), dtype=np.int64).astype(np.int16)
            got = experts.dequant(torch.from_numpy(t).to(DEV), cb).cpu().numpy()
            want = ore.unpack(t, k2 / 2, cb)
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (cb, k2)


@pytest.mark.parametrize("cb,widths", MIXED, ids=[m[0] + str(i) for i, m in enumerate(MIXED)])
def test_mixed_widths_match_the_oracle_and_rows_are_independent(cb, widths):
    n_exp, d, width, top_k, rows = 24, 512, 256, 6, 40
    ex, mats = make_layer(n_exp, d, width, cb, widths, 11)
    x = torch.randn((rows, d), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(DEV)
    sel, w = picks(n_exp, rows, top_k, 4, shared=True)
    scratch = experts.Scratch(ex, rows, top_k + 1)

    def run(idx):
        scratch.y.zero_()
        return experts.routed(x[idx], sel[idx].contiguous(), w[idx].contiguous(), ex, scratch, None, len(idx)).clone()

    full = run(list(range(rows)))
    assert torch.isfinite(full).all()
    for n in (1, 2, 3, 16, 17, 40):
        for start in (0, rows - n):
            idx = list(range(start, start + n))
            assert torch.equal(run(idx), full[idx]), (cb, n, start)
    # the float64 restatement with the kernels' fp16 rounding points, on the first rows (the shared slot's y is zero)
    nref = 5
    _, want = ore.routed(x[:nref].float().cpu().numpy(), sel[:nref].cpu().numpy(), w[:nref].cpu().numpy(), *mats, cb)
    got = full[:nref].double().cpu().numpy()
    err = rel_l2(got, want)
    print(f"{cb}: rel-L2 {err:.2e}, max-abs/max {np.abs(got - want).max() / np.abs(want).max():.2e}")
    assert err <= TOL


@pytest.mark.parametrize("act_mode,limit", [(experts.ACT_F32, 0.75), (experts.ACT_BF16, 0.75), (experts.ACT_BF16, float("inf"))])
def test_clip_and_bf16_activation(act_mode, limit):
    n_exp, d, width = 6, 256, 384
    ex, mats = make_layer(n_exp, d, width, "mcg", lambda e: (4, 4, 4), 31)
    x = (torch.randn((4, d), generator=torch.Generator().manual_seed(8)) * 2).to(torch.bfloat16).to(DEV)
    sel, w = picks(n_exp, 4, 3, 9)
    scratch = experts.Scratch(ex, 4, 3)
    y = experts.routed(x, sel, None, ex, scratch, None, 4, limit=limit, act_mode=act_mode).clone()
    want, _ = ore.routed(x.float().cpu().numpy(), sel.cpu().numpy(), w.cpu().numpy(), *mats, "mcg", limit=limit,
                         act_bf16=act_mode == experts.ACT_BF16)
    got = y.view(4, 3, d).double().cpu().numpy()
    # bf16 activations sit on rounding boundaries: a flipped bf16 step of one activation moves an output by its share
    tol = TOL if act_mode == experts.ACT_F32 else 4e-3
    assert rel_l2(got, want) <= tol
    unclipped, _ = ore.routed(x.float().cpu().numpy(), sel.cpu().numpy(), w.cpu().numpy(), *mats, "mcg")
    if limit < 1:
        assert rel_l2(got, unclipped) > 0.05                   # the clip is live in this case


@pytest.mark.parametrize("slots", [1, 3, 9, 33])
def test_fused_down_and_combine_equal_the_separate_steps(slots):
    n_exp, d, width, rows = 40, 256, 128, 5
    ex, _ = make_layer(n_exp, d, width, "3inst", lambda e: (3, 3, 4), 41)
    x = torch.randn((rows, d), generator=torch.Generator().manual_seed(2)).to(torch.float16).to(DEV)
    sel, w = picks(n_exp, rows, slots - 1, 6, shared=True) if slots > 1 else picks(n_exp, rows, 1, 6)
    scratch = experts.Scratch(ex, rows, slots)
    scratch.y.fill_(7.0)                                                           # the shared slot's rows are the caller's
    y = experts.routed(x, sel, None, ex, scratch, None, rows).clone().view(rows, slots, d)
    if slots > 1:
        assert (y[:, -1] == 7.0).all()
    # the fma chain from zero in slot order: a product of two fp32 is exact in float64, so one rounding of
    # float64(w) * float64(y) + float64(acc) to fp32 is the fused multiply-add (but for a double rounding too rare to meet)
    acc = np.zeros((rows, d), dtype=np.float32)
    wn, yn = w.cpu().numpy(), y.cpu().numpy()
    for k in range(slots):
        acc = (wn[:, k:k + 1].astype(np.float64) * yn[:, k].astype(np.float64) + acc.astype(np.float64)).astype(np.float32)
    scratch.y.fill_(7.0)
    out = experts.routed(x, sel, w, ex, scratch, None, rows, group=False)
    assert np.array_equal(out.cpu().numpy(), acc)


@pytest.mark.parametrize("cb,rows,slots", [("mcg", 1, 9), ("3inst", 8, 9), ("mul1", 37, 5), ("mcg", 16, 64)])
def test_grouping_in_the_rotations_launch(cb, rows, slots):
    """The launch that groups and rotates at once leaves the plan and the rotated inputs of the two separate launches
    (``group=False`` after a ``route`` of one's own takes those), and so the same outputs; with slots that are not
    routed and a row that has none."""

    n_exp, d, width = 70, 384, 256
    ex, _ = make_layer(n_exp, d, width, cb, lambda e: ((2, 3.5, 4, 5)[e % 4],) * 2 + ((3, 4)[e % 2],), 91)
    gen = torch.Generator().manual_seed(rows)
    x = torch.randn((rows, d), generator=gen).to(torch.bfloat16).to(DEV)
    sel, w = picks(n_exp, rows, slots - 1, 17 + rows, shared=True)
    sel[rows // 2, 0] = -3
    if rows > 2:
        sel[rows - 2] = n_exp + 1
    mine = torch.randn((rows * slots, d), generator=gen).to(DEV)
    one, two = experts.Scratch(ex, rows, slots), experts.Scratch(ex, rows, slots)
    for n in (rows, max(1, rows - 3)):
        one.y.copy_(mine), two.y.copy_(mine)
        a = experts.routed(x[:n], sel[:n].contiguous(), w[:n].contiguous(), ex, one, None, n, limit=1.5).clone()
        grouped.route(sel[:n].contiguous(), two.plan)
        b = experts.routed(x[:n], sel[:n].contiguous(), w[:n].contiguous(), ex, two, None, n, limit=1.5, group=False)
        torch.cuda.synchronize()
        k = int(two.plan.counts[0])
        assert torch.equal(one.plan.counts, two.plan.counts) and torch.equal(one.plan.items[:k], two.plan.items[:k])
        assert torch.equal(one.plan.members, two.plan.members)
        assert torch.equal(one.xg, two.xg) and torch.equal(one.xu, two.xu) and torch.equal(one.y, two.y)
        assert torch.equal(a, b), n


def test_graph_replay_equals_eager():
    n_exp, d, width, top_k = 16, 512, 256, 4
    ex, _ = make_layer(n_exp, d, width, "mul1", lambda e: (2.5, 3, 4), 51)
    for rows in (1, 2, 8):
        scratch = experts.Scratch(ex, rows, top_k)
        x = torch.randn((rows, d), generator=torch.Generator().manual_seed(rows)).to(torch.bfloat16).to(DEV)
        sel, w = picks(n_exp, rows, top_k, 60 + rows)
        out = torch.empty((rows, d), dtype=torch.float32, device=DEV)
        eager = experts.routed(x, sel, w, ex, scratch, None, rows).clone()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            experts.routed(x, sel, w, ex, scratch, out, rows)
        for _ in range(3):
            out.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
        # new picks and inputs through the same graph
        sel2, w2 = picks(n_exp, rows, top_k, 90 + rows)
        x2 = torch.randn((rows, d), generator=torch.Generator().manual_seed(100 + rows)).to(torch.bfloat16).to(DEV)
        want = experts.routed(x2, sel2, w2, ex, scratch, None, rows).clone()
        x.copy_(x2), sel.copy_(sel2), w.copy_(w2)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_bad_arguments_raise():
    ex, _ = make_layer(4, 256, 128, "mcg", lambda e: (4, 4, 4), 61)
    scratch = experts.Scratch(ex, 2, 2)
    x = torch.zeros((2, 256), dtype=torch.bfloat16, device=DEV)
    sel, w = picks(4, 2, 2, 1)
    with pytest.raises(ValueError):
        experts.routed(x, sel, w, ex, scratch, None, 3)
    with pytest.raises(ValueError):
        experts.routed(x[:, :128], sel, w, ex, scratch, None, 2)
    with pytest.raises(ValueError):
        experts.routed(x, sel.long(), w, ex, scratch, None, 2)
    with pytest.raises(ValueError):
        experts.routed(x, sel, w.double(), ex, scratch, None, 2)
    with pytest.raises(ValueError):
        experts.routed(x, sel, w, ex, scratch, None, 2, act_mode=5)
    v = torch.ones(256, dtype=torch.float16, device=DEV)
    for last in (16 * 3 + 4, 8 * 17, 8):                # not whole half-bits; 8.5 bits; half a bit
        t = torch.zeros((16, 8, last), dtype=torch.int16, device=DEV)
        with pytest.raises(ValueError):
            experts.prepare([(t, v, v[:128])], [(t, v, v[:128])], [(t.reshape(8, 16, -1), v[:128], v)], "mcg")
    with pytest.raises(ValueError):
        experts.prepare([], [], [], "mcg")
    with pytest.raises(ValueError):
        experts.codebook_id("nope")


def test_more_than_1024_pairs():
    """Past 1,024 pairs the pair sort runs on several workgroups and an expert's pairs span many items of 16."""

    n_exp, d, width, top_k, rows = 12, 256, 128, 7, 160
    ex, mats = make_layer(n_exp, d, width, "mcg", lambda e: (2 + e % 3, 3, 4), 71)
    x = torch.randn((rows, d), generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(DEV)
    sel, w = picks(n_exp, rows, top_k, 6, shared=True)
    scratch = experts.Scratch(ex, rows, top_k + 1)
    scratch.y.zero_()
    full = experts.routed(x, sel, w, ex, scratch, None, rows).clone()
    small = experts.Scratch(ex, 3, top_k + 1)
    for r0 in (0, 77, rows - 3):
        part = experts.routed(x[r0:r0 + 3], sel[r0:r0 + 3].contiguous(), w[r0:r0 + 3].contiguous(), ex, small, None, 3)
        assert torch.equal(part, full[r0:r0 + 3])
    _, want = ore.routed(x[:3].float().cpu().numpy(), sel[:3].cpu().numpy(), w[:3].cpu().numpy(), *mats, "mcg")
    assert rel_l2(full[:3].double().cpu().numpy(), want) <= TOL


def test_no_routed_pick_at_all():
    """Every slot outside [0, E): nothing is grouped, y stays the caller's and the combine is its weighted sum."""

    n_exp, d, width, rows, slots = 5, 256, 128, 3, 4
    ex, _ = make_layer(n_exp, d, width, "mcg", lambda e: (4, 4, 4), 81)
    x = torch.randn((rows, d), generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(DEV)
    sel = torch.tensor([[5, 7, -1, 5]] * rows, dtype=torch.int32, device=DEV)
    w = torch.rand((rows, slots), generator=torch.Generator().manual_seed(2)).to(DEV)
    scratch = experts.Scratch(ex, rows, slots)
    mine = torch.randn((rows * slots, d), generator=torch.Generator().manual_seed(3)).to(DEV)
    scratch.y.copy_(mine)
    out = experts.routed(x, sel, w, ex, scratch, None, rows)
    assert torch.equal(scratch.y, mine)
    want = np.zeros((rows, d), dtype=np.float32)
    wn, yn = w.cpu().numpy(), mine.view(rows, slots, d).cpu().numpy()
    for k in range(slots):
        want = (wn[:, k:k + 1].astype(np.float64) * yn[:, k].astype(np.float64) + want.astype(np.float64)).astype(np.float32)
    assert np.array_equal(out.cpu().numpy(), want)
