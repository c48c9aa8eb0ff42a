"""Routed-expert kernels on the GPU, decode and prefill forms, against the CPU oracle (properties after the
reference's tests/cuda/test_experts.py; tensors are seeded on the CPU so the oracle sees the same bits)."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import routing as orr
from tensorfold_amd import experts, synthetic
from tests.helpers import f32, max_abs, rel_l2, u32

pytestmark = pytest.mark.gpu
DEV = "cuda"

# (group size, SwiGLU, limit, experts incl. shared, D, NI, shared slots)
CASES = [(32, True, 0.0, 41, 256, 96, 1), (64, True, 10.0, 19, 512, 128, 1), (64, False, 0.0, 12, 384, 192, 2)]


def build(case, seed):
    gs, swiglu, limit, e, d, ni, _ = case
    up = [synthetic.affine_general(ni, d, gs, seed + i, (e,)) for i in range(2 if swiglu else 1)]
    down = synthetic.affine_general(d, ni, gs, seed + 7, (e,))
    # a relu^2 layer is made for the bf16 prompt form unless told (its activations' range is not the tables' to
    # know); these cases' activations are small, and the fp16 form is the one they pin
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), gs, limit=limit,
                      arith=experts.ARITH_F16)
    return ex, up, down


def picks_for(rows, case, seed, hot=None):
    """Each row: distinct routed experts (the first ones when ``hot``, so every row shares them), then the shared."""

    e, shared = case[3], case[6]
    routed = e - shared
    k = min(6, routed)
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(rows):
        r = torch.arange(k) if hot is not None else torch.randperm(routed, generator=g)[:k]
        out.append(torch.cat([r, torch.arange(routed, e)]))
    return torch.stack(out).to(torch.int32)


def run(ex, x, picks, prefill=False, y_dtype=torch.float32, tile=None):
    rows, slots = picks.shape
    plan = experts.Plan(rows, slots, ex.count, DEV, prefill=prefill)
    experts.route(picks.to(DEV).contiguous(), plan, *(() if tile is None else (tile,)))
    act = torch.empty((rows * slots, ex.width), dtype=torch.bfloat16, device=DEV)
    y = torch.empty((rows * slots, ex.dims), dtype=y_dtype, device=DEV)
    experts.gate_up(x, ex, plan, act, rows)
    experts.down(act, ex, plan, y, rows)
    return act, y, plan


def np_tables(ms):
    return [(u32(w), f32(s), f32(b)) for (w, s, b) in ms]


@pytest.mark.parametrize("gs", [32, 64])
def test_pack_round_trip(gs):
    w = tuple(t.to(DEV) for t in synthetic.affine_general(96, 256, gs, 61, (3,)))
    blocks = experts.pack(*w, gs)
    assert blocks.shape == (3, 3, 256 // gs, experts.block_words(gs))
    back = experts.unpack(blocks, gs)
    assert all(torch.equal(a, b) for a, b in zip(back, w))
    stacked = torch.stack([blocks, blocks.flip(0)], dim=3)             # one matrix of a stacked table, as a view
    back = experts.unpack(stacked[1:2, :, :, 0], gs)
    assert all(torch.equal(a, b[1:2]) for a, b in zip(back, w))


@pytest.mark.parametrize("rows,prefill,tile", [(1, False, 64), (23, False, 64), (23, True, 64), (300, False, 64),
                                              (300, True, 64), (1500, True, 64), (1500, True, 16), (1500, True, 128)])
def test_plan_groups_pairs_by_expert(rows, prefill, tile):
    """Bit-exact members, items and counts against the oracle: one workgroup up to 1,024 pairs, several past it."""

    slots, e = 7, 50
    g = torch.Generator().manual_seed(9)
    picks = torch.stack([torch.randperm(e, generator=g)[:slots] for _ in range(rows)]).to(torch.int32)
    picks[:, 0] = 3                                            # one expert with a pair in every row
    plan = experts.Plan(rows, slots, e, DEV, prefill=prefill)
    experts.route(picks.to(DEV), plan, tile)
    assert plan.tile == (tile if prefill else experts.TILE)
    items, members, distinct = orr.plan(picks.numpy(), e, plan.tile)
    n = int(plan.counts[0])
    assert n == len(items) and int(plan.counts[1]) == distinct
    assert n <= experts.max_items(rows * slots, e, plan.tile)
    assert np.array_equal(plan.items[:n].cpu().numpy(), items)
    assert np.array_equal(plan.members.cpu().numpy(), members)


@pytest.mark.parametrize("gs", [32, 64])
def test_the_sums_a_wave_takes_from_its_inputs(gs):
    """The affine form needs the sum of every group of inputs; each wave takes it from the inputs it streams.  A table
    whose codes and scales are zero and whose bias is 1 in one group a column and 0 elsewhere makes every output
    that group's sum itself: out[p, n] = sum of x[p, group n % KG], which pins the sums (a dropped chunk, a lane
    left out of the row's tree or a wrong group would each show) for one and for two rows a pass."""

    d, k, e = 7 * gs, 6 * 64, 3                      # 7 or 14 column blocks (7: a half-empty pair), K of 12 or 6 groups
    kg = k // gs
    words = torch.zeros((e, d, k // 8), dtype=torch.int32)
    scales = torch.zeros((e, d, kg), dtype=torch.bfloat16)
    biases = torch.zeros((e, d, kg), dtype=torch.bfloat16)
    cols = torch.arange(d)
    biases[:, cols, cols % kg] = 1.0
    down = tuple(t.to(DEV) for t in (words, scales, biases))
    ex = experts.make([tuple(t.to(DEV) for t in synthetic.affine_general(k, d, gs, 3, (e,)))], down, gs)
    assert ex.width == k and ex.dims == d
    for rows, picks in ((1, [[2]]), (5, [[0], [0], [1], [0], [1]])):          # items of 1, of 3 (passes of 2 + 1), of 2
        picks = torch.tensor(picks, dtype=torch.int32, device=DEV)
        act = synthetic.activations(rows, k, 91 + rows, 1.0).to(DEV)
        plan = experts.Plan(rows, 1, e, DEV)
        experts.route(picks, plan)
        y = torch.empty((rows, d), dtype=torch.float32, device=DEV)
        experts.down(act, ex, plan, y, rows)
        want = act.float().view(rows, kg, gs).double().sum(-1)[:, cols % kg]
        assert (y.double().cpu() - want.cpu()).abs().max() <= 1e-5 * float(act.float().abs().sum(-1).max())
        # every output of a group's columns holds the same bits: the sum does not depend on the lane or the wave
        for g in range(kg):
            same = y[:, g::kg]
            assert torch.equal(same, same[:, :1].expand_as(same)), g


def test_an_expert_shared_by_many_rows_makes_items_of_16():
    picks = torch.full((37, 1), 5, dtype=torch.int32)
    plan = experts.Plan(37, 1, 8, DEV)
    experts.route(picks.to(DEV), plan)
    assert int(plan.counts[0]) == 3 and int(plan.counts[1]) == 1
    assert plan.items[:3].cpu().tolist() == [[5, 0, 16], [5, 16, 16], [5, 32, 5]]


@pytest.mark.parametrize("prefill", [False, True])
@pytest.mark.parametrize("case", CASES)
def test_matches_the_oracle(case, prefill):
    """act and y of every pair against dequant-then-matmul with the reference's rounding points (prefill: weights
    rounded to bf16 first).  Bounds: the reference's own (act 2^-6, y 1e-5 of the largest value) and rel-L2 2e-3."""

    gs, swiglu, limit = case[0], case[1], case[2]
    ex, up, down = build(case, 31)
    rows = 5
    x = synthetic.activations(rows, ex.dims, 77, 0.5)
    picks = picks_for(rows, case, 6)
    act, y, _ = run(ex, x.to(DEV), picks, prefill=prefill)
    act_ref, _ = ora.expert_pairs(f32(x), picks.numpy(), np_tables(up), np_tables([down])[0], gs, limit=limit,
                                  prefill=prefill)
    assert max_abs(f32(act), act_ref) <= 2 ** -6 * np.abs(act_ref).max()
    assert rel_l2(f32(act), act_ref) <= 2e-3
    # down from the GPU's own activations, so that only the down matmul is measured
    slots = picks.shape[1]
    pe = picks.reshape(-1).numpy()
    wd = ora.dequantize(u32(down[0]), f32(down[1]), f32(down[2]), gs)
    if prefill:
        wd = ora.prefill_weight(wd)
    y_ref = np.einsum("pk,pnk->pn", f32(act).astype(np.float64), wd[pe].astype(np.float64))
    assert max_abs(f32(y), y_ref) <= 1e-5 * np.abs(y_ref).max()
    assert rel_l2(f32(y), y_ref) <= 1e-5
    assert slots == picks.shape[1]


@pytest.mark.parametrize("case", CASES)
def test_pairs_do_not_depend_on_the_window(case):
    ex, _, _ = build(case, 11)
    rows = 40
    x = synthetic.activations(rows, ex.dims, 5, 0.5).to(DEV)
    picks = picks_for(rows, case, 3)
    slots = picks.shape[1]
    act, y, _ = run(ex, x, picks)
    alone = [run(ex, x[r:r + 1], picks[r:r + 1]) for r in range(rows)]
    assert torch.equal(act, torch.cat([a[0] for a in alone])) and torch.equal(y, torch.cat([a[1] for a in alone]))
    for m in (2, 3, 8, 9, 16, 17, 33):
        a_m, y_m, _ = run(ex, x[:m], picks[:m])
        assert torch.equal(a_m, act[:m * slots]) and torch.equal(y_m, y[:m * slots]), m
    perm = torch.randperm(rows, generator=torch.Generator().manual_seed(5))
    a_p, y_p, _ = run(ex, x[perm.to(DEV)], picks[perm])
    idx = (perm[:, None] * slots + torch.arange(slots)).reshape(-1).to(DEV)
    assert torch.equal(a_p, act[idx]) and torch.equal(y_p, y[idx])


@pytest.mark.parametrize("case", CASES)
def test_an_expert_shared_by_many_rows(case):
    """Every row picks the same experts: items of 16 pairs, several an expert, same bits as alone."""

    ex, _, _ = build(case, 21)
    rows = 37
    x = synthetic.activations(rows, ex.dims, 8, 0.5).to(DEV)
    picks = picks_for(rows, case, 4, hot=0)
    _, y, plan = run(ex, x, picks)
    slots = picks.shape[1]
    alone = torch.cat([run(ex, x[r:r + 1], picks[r:r + 1])[1] for r in range(rows)])
    assert torch.equal(y, alone)
    assert int(plan.counts[1]) == slots and int(plan.counts[0]) == slots * 3


@pytest.mark.parametrize("case", CASES)
def test_a_pairs_bits_never_depend_on_its_item(case):
    """A prompt plan grouped in items of 16, 64 and 128 pairs gives every pair the same bits."""

    ex, _, _ = build(case, 31)
    rows = 300
    x = synthetic.activations(rows, ex.dims, 12, 0.5).to(DEV)
    picks = picks_for(rows, case, 6)
    got = {t: run(ex, x, picks, prefill=True, y_dtype=torch.bfloat16, tile=t) for t in (16, 64, 128)}
    for t in (64, 128):
        assert torch.equal(got[16][0], got[t][0]) and torch.equal(got[16][1], got[t][1]), t
    assert int(got[128][2].counts[0]) <= int(got[64][2].counts[0]) < int(got[16][2].counts[0])


@pytest.mark.parametrize("case", CASES)
def test_prefill_rows_do_not_depend_on_the_chunk(case):
    """Prefill form past 1,024 pairs: any chunk or row order keeps each row's bits; bf16 down is fp32 rounded."""

    ex, _, _ = build(case, 71)
    rows = 200
    x = synthetic.activations(rows, ex.dims, 15, 0.5).to(DEV)
    picks = picks_for(rows, case, 13)
    slots = picks.shape[1]
    assert rows * slots > experts.SMALL
    act, y, _ = run(ex, x, picks, prefill=True)
    for a, b in ((0, 1), (77, 78), (199, 200), (0, 7), (5, 22), (0, 64), (100, 200)):
        a1, y1, _ = run(ex, x[a:b], picks[a:b], prefill=True)
        assert torch.equal(a1, act[a * slots:b * slots]) and torch.equal(y1, y[a * slots:b * slots]), (a, b)
    perm = torch.randperm(rows, generator=torch.Generator().manual_seed(5))
    a_p, y_p, _ = run(ex, x[perm.to(DEV)], picks[perm], prefill=True)
    idx = (perm[:, None] * slots + torch.arange(slots)).reshape(-1).to(DEV)
    assert torch.equal(a_p, act[idx]) and torch.equal(y_p, y[idx])
    _, y16, _ = run(ex, x, picks, prefill=True, y_dtype=torch.bfloat16)
    assert torch.equal(y16, y.to(torch.bfloat16))


def test_graph_replay_follows_the_picks():
    """A captured route + gate_up + down replays on new picks (no host reads of the plan); replayed three times with
    eager work in between."""

    case = CASES[1]
    ex, _, _ = build(case, 41)
    rows = 9
    picks = picks_for(rows, case, 7).to(DEV).contiguous()
    slots = picks.shape[1]
    plan = experts.Plan(rows, slots, ex.count, DEV)
    x = synthetic.activations(rows, ex.dims, 2, 0.5).to(DEV)
    act = torch.empty((rows * slots, ex.width), dtype=torch.bfloat16, device=DEV)
    y = torch.empty((rows * slots, ex.dims), dtype=torch.float32, device=DEV)

    def step():
        experts.route(picks, plan)
        experts.gate_up(x, ex, plan, act, rows)
        experts.down(act, ex, plan, y, rows)

    step()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        step()
    for seed in (8, 9, 10):
        picks.copy_(picks_for(rows, case, seed))
        g.replay()
        torch.cuda.synchronize()
        _, want, _ = run(ex, x, picks.cpu())
        assert torch.equal(y, want), seed


def test_many_units_keep_the_bits():
    """Far more workgroups than the chip holds at once, against rows alone."""

    case = (64, True, 0.0, 257, 2048, 128, 1)
    ex, _, _ = build(case, 81)
    rows = 64
    x = synthetic.activations(rows, ex.dims, 4, 0.5).to(DEV)
    g = torch.Generator().manual_seed(12)
    picks = torch.stack([torch.cat([torch.randperm(256, generator=g)[:8], torch.tensor([256])])
                         for _ in range(rows)]).to(torch.int32)
    _, y, plan = run(ex, x, picks)
    assert int(plan.counts[0]) * (ex.dims // experts.COLS) > 8192
    for r in (0, 31, 63):
        assert torch.equal(run(ex, x[r:r + 1], picks[r:r + 1])[1], y[9 * r:9 * r + 9]), r


@pytest.mark.parametrize("used,rows,d,ni", [(3, 80, 512, 256), (400, 96, 512, 256), (600, 640, 512, 256),
                                            (600, 200, 576, 320)])
def test_prompt_units_walked_by_workgroups_that_stay(used, rows, d, ni):
    """Past two units a compute unit (by the host's bound on the items) the prompt form is one workgroup a compute
    unit walking the units by ticket: with fewer units than workgroups, with between one and two each, and with
    several each, the bits are those of the 16-row items (one workgroup a unit, never walked), and the plan's ticket
    word is back at zero after every launch.  The last case has an odd number of 64-input steps (576 inputs) and
    part-filled last units (320 and 576 columns: 10 and 18 blocks of 32 where a unit holds 8 or 16)."""

    case = (32, True, 0.0, 601, d, ni, 1)
    ex, _, _ = build(case, 91)
    x = synthetic.activations(rows, ex.dims, 5, 0.5).to(DEV)
    g = torch.Generator().manual_seed(13)
    picks = torch.stack([torch.cat([torch.randperm(used, generator=g)[:6], torch.tensor([600])])
                         for _ in range(rows)]).to(torch.int32)
    assert experts.max_items(rows * 7, ex.count, 128) > 2 * torch.cuda.get_device_properties(0).multi_processor_count
    act, y, plan = run(ex, x, picks, prefill=True, tile=128)
    units = int(plan.counts[0])                       # the up launch: an item is one unit of 256 columns a matrix
    assert plan.counts.cpu().tolist()[2:] == [0, 0]
    want_act, want, _ = run(ex, x, picks, prefill=True, tile=16)
    assert torch.equal(act, want_act) and torch.equal(y, want), units
    # again on the same plan: the ticket word was left ready
    experts.gate_up(x, ex, plan, act.zero_(), rows)
    experts.down(act, ex, plan, y.zero_(), rows)
    assert torch.equal(act, want_act) and torch.equal(y, want) and plan.counts.cpu().tolist()[2:] == [0, 0]


def test_bad_arguments_raise():
    w = tuple(t.to(DEV) for t in synthetic.affine_general(96, 256, 64, 1, (2,)))
    with pytest.raises(ValueError):
        experts.pack(*w, 16)
    with pytest.raises(ValueError):
        experts.pack(w[0], w[1][:, :, :2], w[2], 64)
    plan = experts.Plan(4, 3, 8, DEV)
    with pytest.raises(ValueError):
        experts.route(torch.zeros((5, 3), dtype=torch.int32, device=DEV), plan)
    with pytest.raises(ValueError):
        experts.make([w, w, w], w, 64)


def test_prompt_experts_beyond_the_range_of_fp16():
    """A layer whose scales do not fit the fp16 prompt form is made for the bf16 form (the reference's arithmetic) and
    its prompt plan runs in it: against the oracle with the same once-rounded weights, every item size the same bits."""

    from oracle import native
    from tests.helpers import bits16

    gs, e, d, ni, rows = 32, 9, 256, 128, 150
    g = torch.Generator().manual_seed(17)

    def table(n, k, lo):
        words = synthetic.affine_general(n, k, gs, n + k, (e,))[0]
        scales = (torch.rand((e, n, k // gs), generator=g) * lo + lo).bfloat16()
        return words, scales, (scales.float() * -7.5).bfloat16()

    up, down = [table(ni, d, 150.0)], table(d, ni, 0.01)                 # only the up table is out of range
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), gs)
    assert ex.arith == experts.ARITH_BF16
    small = tuple(t.to(DEV) for t in down)
    fits = experts.make([small, small], tuple(t.to(DEV) for t in table(ni, ni, 0.01)), gs)
    assert fits.arith == experts.ARITH_F16
    # the same tables as a relu^2 layer: the bf16 form, whatever the tables (its activations are unbounded)
    assert experts.make([small], tuple(t.to(DEV) for t in table(ni, ni, 0.01)), gs).arith == experts.ARITH_BF16
    x = (synthetic.activations(rows, d, 18).float() * 300).bfloat16()
    picks = torch.stack([torch.randperm(e, generator=g)[:3] for _ in range(rows)]).to(torch.int32)
    wts = torch.full((rows, 3), 1 / 3)
    got = {t: run(ex, x.to(DEV), picks, prefill=True, tile=t) for t in (16, 64, 128)}
    for t in (64, 128):
        assert torch.equal(got[16][0], got[t][0]) and torch.equal(got[16][1], got[t][1]), t
    act, y, _ = got[128]
    assert torch.isfinite(y).all()
    tab = lambda m: (u32(m[0]), bits16(m[1]), bits16(m[2]))
    _, act_ref, y_ref = native.moe_layer(bits16(x), picks.numpy(), wts.numpy(), None, tab(up[0]), tab(down), gs,
                                         prefill=2, want_pairs=True)
    assert rel_l2(f32(act), ora.bf16_from_bits(act_ref)) <= 2e-3          # relu^2 on bf16 roundings: a few flipped steps
    assert rel_l2(f32(y), y_ref) <= 2e-3
    print(f"bf16 prompt form: act rel-L2 {rel_l2(f32(act), ora.bf16_from_bits(act_ref)):.2e}, "
          f"y rel-L2 {rel_l2(f32(y), y_ref):.2e}, max-abs {max_abs(f32(y), y_ref):.3e}")


def test_a_group_whose_weights_pass_256_takes_the_bf16_form():
    """The fp16 prompt form holds fp16(256 (q s + b)): scales of 20 to 100 with small biases pass every test of the
    scales and biases alone, but 15 s + b reaches 1,500 and 256 times that is past fp16.  Such a table must be made
    for the bf16 form and its prompt outputs must be finite and the oracle's."""

    from oracle import native
    from tests.helpers import bits16

    gs, e, d, ni, rows = 32, 5, 256, 128, 70
    g = torch.Generator().manual_seed(29)

    def table(n, k, lo, hi):
        words = synthetic.affine_general(n, k, gs, n + k + 1, (e,))[0]
        scales = (torch.rand((e, n, k // gs), generator=g) * (hi - lo) + lo).bfloat16()
        return words, scales, (torch.rand((e, n, k // gs), generator=g) - 0.5).bfloat16()

    wide, small = table(ni, d, 20.0, 100.0), table(d, ni, 0.002, 0.02)
    assert not experts.fits_f16(wide[1], wide[2]) and experts.fits_f16(small[1], small[2])
    assert not experts.fits_f16(torch.tensor([30.0]), torch.tensor([-100.0]))          # 15 s + b = 350
    assert experts.fits_f16(torch.tensor([30.0]), torch.tensor([-240.0]))              # weights in [-240, 210]
    dev = lambda m: tuple(t.to(DEV) for t in m)
    ex = experts.make([dev(wide), dev(wide)], dev(small), gs)
    assert ex.arith == experts.ARITH_BF16
    from tensorfold_amd import qmm
    q = qmm.pack(wide[0][0].to(DEV), wide[1][0].to(DEV), wide[2][0].to(DEV), gs)
    assert q.arith == experts.ARITH_BF16
    x = synthetic.activations(rows, d, 5, 0.02)
    yq = qmm.prefill_matmul(x.to(DEV), q, f32=True)
    assert torch.isfinite(yq).all()
    picks = torch.stack([torch.randperm(e, generator=g)[:2] for _ in range(rows)]).to(torch.int32)
    act, y, _ = run(ex, x.to(DEV), picks, prefill=True)
    assert torch.isfinite(y).all() and torch.isfinite(act.float()).all()
    tab = lambda m: (u32(m[0]), bits16(m[1]), bits16(m[2]))
    wts = torch.full((rows, 2), 0.5)
    _, act_ref, y_ref = native.moe_layer(bits16(x), picks.numpy(), wts.numpy(), tab(wide), tab(wide), tab(small), gs,
                                         prefill=2, want_pairs=True)
    assert rel_l2(f32(y), y_ref) <= 2e-3


def test_relu2_prompt_activations_past_fp16():
    """A relu^2 layer made without a word about its arithmetic (as the loader makes Nemotron-H's): up outputs beyond
    256 square to activations beyond fp16's 65,504, and the prompt layer must carry them unclamped through the down
    projection and the pair outputs: ``moe.run(prefill=True)`` against the oracle's bf16 prompt form."""

    from oracle import native
    from tensorfold_amd import moe
    from tests.helpers import bits16

    gs, ne, d, ni, rows, k = 64, 8, 256, 128, 48, 2
    up = synthetic.affine(ni, d, gs, 41, (ne + 1,))               # expert `ne` is the shared one
    down = synthetic.affine(d, ni, gs, 42, (ne + 1,))
    dev = lambda m: tuple(t.to(DEV) for t in m)
    ex = experts.make([dev(up)], dev(down), gs)
    assert ex.arith == experts.ARITH_BF16
    g = torch.Generator().manual_seed(43)
    rr = (torch.randn((ne + 1, d), generator=g) * 0.0005).bfloat16()
    x = (synthetic.activations(rows, d, 44).float() * 4000).bfloat16()
    layer = moe.Routed(rr.to(DEV), ex, k)
    out = moe.run(x.to(DEV), layer, prefill=True)
    assert torch.isfinite(out.float()).all()
    logits = moe.router(x.to(DEV), rr.to(DEV)).cpu().numpy()
    picks, wts = orr.topk_rows(logits, ne, k, shared=True)
    tab = lambda m: (u32(m[0]), bits16(m[1]), bits16(m[2]))
    want, act_ref, y_ref = native.moe_layer(bits16(x), picks, wts, None, tab(up), tab(down), gs, prefill=2,
                                            want_pairs=True)
    big = float(ora.bf16_from_bits(act_ref).max())
    assert big > 4 * 65504, big                                   # the case is the one the test is named for
    assert float(np.abs(y_ref).max()) > 65504                     # and pair outputs that fp16 could not hold either
    err = rel_l2(f32(out), ora.bf16_from_bits(want))
    print(f"relu^2 prompt layer past fp16: largest activation {big:.3g}, rel-L2 {err:.2e}")
    assert err <= 2e-3
