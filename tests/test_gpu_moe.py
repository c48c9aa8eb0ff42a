"""The MoE layer on the GPU (router, top-k, plan, experts, combine) against the CPU oracle, at the benchmark shapes
(configs 1 and 2) and in small; ids are checked bit for bit."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import native
from oracle import routing as orr
from tensorfold_amd import experts, moe, synthetic
from tests.helpers import bits16, f32, max_abs, rel_l2, u32

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3


class Cfg:
    def __init__(self, shape):
        self.num_experts_per_tok, self.num_experts = shape.top_k, shape.experts
        self.moe_intermediate_size, self.hidden_size = shape.width, shape.hidden


def test_topk_ids_are_bit_exact_and_weights_are_the_softmax():
    for rows, ne, k, shared in ((1, 128, 6, False), (8, 128, 6, False), (32, 512, 10, True), (5, 1000, 8, True),
                                (3, 64, 64, False)):
        l = synthetic.logits(rows, ne + int(shared), 100 + rows)
        buf = moe.MoEBuffers(rows, type("c", (), dict(num_experts_per_tok=k, num_experts=ne, moe_intermediate_size=32,
                                                      hidden_size=32)), DEV, shared=shared)
        moe.select_rows(l.to(DEV), buf, k, ne)
        picks, wts = orr.topk_rows(l.numpy(), ne, k, shared=shared)
        assert np.array_equal(buf.pick.cpu().numpy(), picks)
        # brute force, independent of the oracle's loop: sort by (-logit, id)
        for r in range(rows):
            order = sorted(range(ne), key=lambda e: (-float(l[r, e]), e))[:k]
            assert buf.pick[r, :k].cpu().tolist() == order
        got = buf.wts.cpu().numpy()
        assert np.abs(got - wts).max() <= 2 ** -8 * np.abs(wts).max()      # bf16-rounded values: at most one step
        assert (got == wts).mean() > 0.9
        assert np.allclose(got[:, :k].sum(1), 1.0, atol=2e-2)


def test_ties_go_to_the_lower_expert():
    l = torch.zeros((3, 129), dtype=torch.float32)
    buf = moe.MoEBuffers(3, type("c", (), dict(num_experts_per_tok=6, num_experts=128, moe_intermediate_size=32,
                                               hidden_size=32)), DEV)
    moe.select_rows(l.to(DEV), buf, 6, 128)
    assert buf.pick.cpu().tolist() == [[0, 1, 2, 3, 4, 5, 128]] * 3
    w = buf.wts.cpu()
    assert torch.equal(w[:, :6], torch.full((3, 6), 1 / 6).bfloat16().float()) and torch.all(w[:, 6] == 0.5)


def test_router_logits():
    g = torch.Generator().manual_seed(4)
    x = synthetic.activations(37, 2048, 1)
    rows = (torch.randn((513, 2048), generator=g) * 0.02).bfloat16()
    got = f32(moe.router(x.to(DEV), rows.to(DEV)))
    want = f32(x).astype(np.float64) @ f32(rows).astype(np.float64).T
    assert rel_l2(got, want) < 1e-5


def test_combine_is_the_slot_ordered_sum():
    g = torch.Generator().manual_seed(5)
    y = torch.randn((9, 7, 2688), generator=g)
    w = torch.rand((9, 7), generator=g)
    want = ora.combine(y.numpy(), w.numpy())
    got = f32(moe.combine(y.to(DEV), w.to(DEV)))
    assert max_abs(got, want) <= 2 ** -7 * np.abs(want).max() and rel_l2(got, want) < 1e-3
    got16 = f32(moe.combine(y.bfloat16().to(DEV), w.to(DEV)))
    want16 = ora.combine(f32(y.bfloat16()), w.numpy())
    assert rel_l2(got16, want16) < 1e-3
    # many rows take the kernel with 16-byte loads: the same bits a row as the narrow one
    y2 = torch.randn((80, 7, 2688), generator=g).to(DEV)
    w2 = torch.rand((80, 7), generator=g).to(DEV)
    wide = moe.combine(y2, w2)
    for r in (0, 41, 79):
        assert torch.equal(moe.combine(y2[r:r + 1].contiguous(), w2[r:r + 1].contiguous())[0], wide[r]), r


def layer_tables(shape, seed, experts_built):
    """MLX tensors of the first ``experts_built`` experts (a full table is hundreds of MB; ids are drawn below it)."""

    e = experts_built + int(shape.shared)
    up = [synthetic.affine(shape.width, shape.hidden, shape.gs, seed + i, (e,)) for i in range(2 if shape.swiglu else 1)]
    down = synthetic.affine(shape.hidden, shape.width, shape.gs, seed + 5, (e,))
    return up, down


def run_layer(shape, up, down, x, l, ne, prefill=False):
    """The layer through the host API on logits ``l`` ([R, ne (+1)])."""

    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), shape.gs)
    rows = x.shape[0]
    cfg = type("c", (), dict(num_experts_per_tok=shape.top_k, num_experts=ne, moe_intermediate_size=shape.width,
                             hidden_size=shape.hidden))
    buf = moe.MoEBuffers(rows, cfg, DEV, prefill=prefill, shared=shape.shared)
    moe.select(l.to(DEV), buf, shape.top_k, ne)
    xd = x.to(DEV)
    experts.gate_up(xd, ex, buf.plan, buf.act.view(-1, ex.width), rows)
    experts.down(buf.act.view(-1, ex.width), ex, buf.plan, buf.y.view(-1, ex.dims), rows)
    return moe.combine(buf.y, buf.wts), buf


@pytest.mark.parametrize("tokens", [1, 4, 8])
def test_config1_decode_layer(tokens):
    """benchmark configuration 1: D 2688, NI 1856, relu^2, top-6, g64, tokens 1 / 4 / 8 (ids drawn over the first 24 of the
    128 experts so the CPU oracle's table stays small; every other shape is the config's)."""

    shape, ne = synthetic.C1, 24
    up, down = layer_tables(shape, 1100, ne)
    x = synthetic.activations(tokens, shape.hidden, 1101)
    l = synthetic.logits(tokens, ne, 1102)
    out, buf = run_layer(shape, up, down, x, l, ne)
    picks, wts = orr.topk_rows(l.numpy(), ne, shape.top_k, shared=False)
    assert np.array_equal(buf.pick.cpu().numpy(), picks)
    want_bits, act_bits, y_ref = native.moe_layer(
        bits16(x), picks, buf.wts.cpu().numpy(), None, (u32(up[0][0]), bits16(up[0][1]), bits16(up[0][2])),
        (u32(down[0]), bits16(down[1]), bits16(down[2])), shape.gs, want_pairs=True)
    want = ora.bf16_from_bits(want_bits)
    err = rel_l2(f32(out), want)
    print(f"config 1, {tokens} tokens: rel-L2 {err:.2e}, max-abs {max_abs(f32(out), want):.3e}")
    assert err <= TOL
    assert rel_l2(f32(buf.act).reshape(-1, shape.width), ora.bf16_from_bits(act_bits)) <= TOL
    assert rel_l2(f32(buf.y).reshape(-1, shape.hidden), y_ref) <= TOL


@pytest.mark.parametrize("prefill", [False, True])
def test_config2_verify_layer(prefill):
    """benchmark configuration 2: D 2048, NI 512, SwiGLU, top-10 + shared, g32, 32 rows (8 lanes x 4 draft tokens); ids over
    the first 48 experts.  Both arithmetic forms: decode, and the prefill form the reference runs this window in."""

    shape, ne = synthetic.C2, 48
    up, down = layer_tables(shape, 1200, ne)
    x = synthetic.activations(32, shape.hidden, 1201)
    l = synthetic.logits(32, ne + 1, 1202)
    out, buf = run_layer(shape, up, down, x, l, ne, prefill=prefill)
    picks, wts = orr.topk_rows(l.numpy(), ne, shape.top_k, shared=True)
    assert np.array_equal(buf.pick.cpu().numpy(), picks)
    items, members, distinct = orr.plan(picks, ne + 1, buf.plan.tile)
    n = int(buf.plan.counts[0])
    assert np.array_equal(buf.plan.items[:n].cpu().numpy(), items)
    assert np.array_equal(buf.plan.members.cpu().numpy(), members)
    want_bits = native.moe_layer(bits16(x), picks, buf.wts.cpu().numpy(),
                                 (u32(up[0][0]), bits16(up[0][1]), bits16(up[0][2])),
                                 (u32(up[1][0]), bits16(up[1][1]), bits16(up[1][2])),
                                 (u32(down[0]), bits16(down[1]), bits16(down[2])), shape.gs)
    want = ora.bf16_from_bits(want_bits)
    err = rel_l2(f32(out), want)
    print(f"config 2 ({'prefill' if prefill else 'decode'} form): rel-L2 {err:.2e}, max-abs {max_abs(f32(out), want):.3e}")
    assert err <= TOL


def test_config3_prefill_chunk_small():
    """benchmark configuration 3 in small: Zipf(1.1) picks over 64 experts, 512 tokens, SwiGLU g32, bf16 MFMA path, items of
    64 and 128; weighted scatter-add back to token order.  Sort permutation bit-exact, output within 2e-3."""

    shape, ne, rows = synthetic.C2, 64, 512
    up, down = layer_tables(shape, 1300, ne)
    x = synthetic.activations(rows, shape.hidden, 1301)
    ids = synthetic.zipf_picks(rows, ne, shape.top_k, 1302)
    sel = synthetic.logits(rows, shape.top_k + 1, 1303)
    # weights: softmax over the chosen ten (bf16-rounded), shared slot sigmoid-gated, as the reference's rule
    wts = torch.cat([torch.softmax(sel[:, :-1], 1).bfloat16().float(),
                     torch.sigmoid(sel[:, -1:].bfloat16().float()).bfloat16().float()], 1).contiguous()
    picks = torch.cat([ids, torch.full((rows, 1), ne, dtype=torch.int32)], 1).contiguous()
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), shape.gs)
    outs = {}
    for tile in (64, 128):
        plan = experts.Plan(rows, picks.shape[1], ne + 1, DEV, prefill=True)
        experts.route(picks.to(DEV), plan, tile)
        items, members, _ = orr.plan(picks.numpy(), ne + 1, tile)
        assert np.array_equal(plan.members.cpu().numpy(), members)
        assert np.array_equal(plan.items[:int(plan.counts[0])].cpu().numpy(), items)
        act = torch.empty((rows * picks.shape[1], shape.width), dtype=torch.bfloat16, device=DEV)
        y = torch.empty((rows * picks.shape[1], shape.hidden), dtype=torch.float32, device=DEV)
        experts.gate_up(x.to(DEV), ex, plan, act, rows)
        experts.down(act, ex, plan, y, rows)
        outs[tile] = moe.combine(y.view(rows, -1, shape.hidden), wts.to(DEV))
    assert torch.equal(outs[64], outs[128])
    # the reference's prompt form keeps bf16 pair outputs (cuda/moe.py:99): the same kernels into a bf16 buffer
    y16 = torch.empty((rows * picks.shape[1], shape.hidden), dtype=torch.bfloat16, device=DEV)
    experts.down(act, ex, plan, y16, rows)
    assert torch.equal(y16, y.bfloat16())
    outs["y_bf16"] = moe.combine(y16.view(rows, -1, shape.hidden), wts.to(DEV))
    # fp16 pair outputs: half the bytes as well, three more bits than bf16
    yh = torch.empty((rows * picks.shape[1], shape.hidden), dtype=torch.float16, device=DEV)
    experts.down(act, ex, plan, yh, rows)
    assert torch.equal(yh, y.half())
    outs["y_f16"] = moe.combine(yh.view(rows, -1, shape.hidden), wts.to(DEV))
    sample = list(range(0, rows, 37))
    want_bits = native.moe_layer(bits16(x[sample]), picks[sample].numpy(), wts[sample].numpy(),
                                 (u32(up[0][0]), bits16(up[0][1]), bits16(up[0][2])),
                                 (u32(up[1][0]), bits16(up[1][1]), bits16(up[1][2])),
                                 (u32(down[0]), bits16(down[1]), bits16(down[2])), shape.gs)
    want = ora.bf16_from_bits(want_bits)
    err = rel_l2(f32(outs[64][sample]), want)
    print(f"config 3 (small): rel-L2 {err:.2e}, max-abs {max_abs(f32(outs[64][sample]), want):.3e}")
    assert err <= TOL
    err16 = rel_l2(f32(outs["y_bf16"][sample]), want)
    print(f"config 3 (small, bf16 pair outputs): rel-L2 {err16:.2e}, max-abs {max_abs(f32(outs['y_bf16'][sample]), want):.3e}")
    assert err16 <= 2 * TOL          # measured 2.7e-3: over the bound, which is why fp32 pair outputs are this build's default
    errh = rel_l2(f32(outs["y_f16"][sample]), want)
    print(f"config 3 (small, fp16 pair outputs): rel-L2 {errh:.2e}, max-abs {max_abs(f32(outs['y_f16'][sample]), want):.3e}")
    assert errh <= TOL


def test_moe_run_rows_do_not_depend_on_the_window():
    shape = synthetic.MoEShape("small", 512, 16, 128, 4, 32, True, True)
    up, down = layer_tables(shape, 7, 16)
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), 32)
    g = torch.Generator().manual_seed(3)
    rr = (torch.randn((17, 512), generator=g) * 0.05).bfloat16().to(DEV)
    layer = moe.Routed(rr, ex, 4)
    x = synthetic.activations(8, 512, 9).to(DEV)
    whole = moe.run(x, layer)
    for r in range(8):
        assert torch.equal(moe.run(x[r:r + 1], layer)[0], whole[r]), r
    for m in (2, 3, 5):
        assert torch.equal(moe.run(x[:m], layer), whole[:m]), m
    whole_p = moe.run(x, layer, prefill=True)
    for r in (0, 7):
        assert torch.equal(moe.run(x[r:r + 1], layer, prefill=True)[0], whole_p[r]), r
    assert rel_l2(f32(whole_p), f32(whole)) < 1e-2


def test_a_prompts_pair_outputs_in_fp16():
    """``run`` keeps a prompt's pair outputs in fp16 for a layer on the fp16 prompt arithmetic and in fp32 for one
    made with ARITH_BF16; fp16 pair outputs are the fp32 ones rounded once, those beyond fp16's range stored as
    +-65504; decode buffers take fp32 only."""

    shape = synthetic.MoEShape("small", 512, 16, 128, 4, 32, True, True)
    up, down = layer_tables(shape, 7, 16)
    tables = [tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down)
    rr = (torch.randn((17, 512), generator=torch.Generator().manual_seed(3)) * 0.05).bfloat16().to(DEV)
    x = synthetic.activations(40, 512, 9).to(DEV)
    kept = {}
    for arith in (experts.ARITH_F16, experts.ARITH_BF16):
        layer = moe.Routed(rr, experts.make(*tables, 32, arith=arith), 4)
        out = moe.run(x, layer, prefill=True)
        kept[arith] = {b.y.dtype for key, b in moe._pool.items() if key[6] and key[0] == 64 and key[3] == 128}
        buf = moe.MoEBuffers(40, moe._Dims(layer), DEV, prefill=True)            # fp32 pair outputs, by hand
        moe.moe(x, layer.router, layer.experts, buf, 4, 16)
        assert rel_l2(f32(out), f32(moe.combine(buf.y, buf.wts))) < 1.5e-3
    assert torch.float16 in kept[experts.ARITH_F16] and torch.float32 in kept[experts.ARITH_BF16]
    with pytest.raises(ValueError):
        moe.MoEBuffers(8, moe._Dims(layer), DEV, y_dtype=torch.float16)

    # 64 inputs of 1e4 against weights of 1.5 (code 15, scale 0.1, bias 0): 9.6e5 a pair output
    ones = lambda n, k: (torch.full((1, n, k // 8), -1, dtype=torch.int32), torch.full((1, n, k // 32), 0.1).bfloat16(),
                         torch.zeros((1, n, k // 32)).bfloat16())
    ex = experts.make([tuple(t.to(DEV) for t in ones(64, 64))], tuple(t.to(DEV) for t in ones(64, 64)), 32)
    plan = experts.Plan(2, 1, 1, DEV, prefill=True)
    experts.route(torch.zeros((2, 1), dtype=torch.int32, device=DEV), plan, 64)
    act = torch.tensor([[1e4] * 64, [-2.0] * 64], device=DEV).bfloat16()
    y32, y16 = torch.empty((2, 64), device=DEV), torch.empty((2, 64), device=DEV, dtype=torch.float16)
    experts.down(act, ex, plan, y32, 2)
    experts.down(act, ex, plan, y16, 2)
    assert float(y32[0, 0]) > 9e5 and torch.all(y16[0] == 65504) and torch.equal(y16[1], y32[1].half())


@pytest.mark.parametrize("shape,ne,rows", [(synthetic.C1, 24, 1), (synthetic.C1, 24, 8), (synthetic.C2, 48, 32),
                                           (synthetic.MoEShape("small", 512, 16, 128, 4, 32, True, True), 16, 5),
                                           (synthetic.MoEShape("small64", 384, 12, 192, 3, 64, False, False), 12, 19),
                                           # short K under a full down launch: 6 groups for 16 slices and an odd
                                           # number of column pairs; 8 groups of 64
                                           (synthetic.MoEShape("short32", 448, 16, 192, 6, 32, True, True), 16, 64),
                                           (synthetic.MoEShape("short64", 1024, 40, 512, 8, 64, False, False), 40, 24)])
@pytest.mark.parametrize("path", ["route_up", "topk_then_up", "route_then_up", "one_launch", "sliced", "topk_then_sliced"])
def test_the_fused_decode_layer_equals_the_separate_kernels(shape, ne, rows, path, monkeypatch):
    """The forms of ``decode`` (routing inside the up launch; a top-k launch, then the plan inside the up launch; a
    routing launch, then up, down, combine from its item descriptors; a routing launch and one launch for up + down +
    combine): ids, plan and output bits equal those of select + gate_up + down + combine; twice in a row on
    different inputs."""

    monkeypatch.setattr(moe, "FUSED_DECODE", path == "one_launch")
    monkeypatch.setattr(moe, "ROUTING_LAUNCH", path == "route_then_up")
    monkeypatch.setattr(moe, "ROUTE_UP_LOGITS", 0 if path.startswith("topk_then") else 1 << 30)
    monkeypatch.setattr(moe, "SLICED_DECODE", path.endswith("sliced"))
    monkeypatch.setattr(moe, "SLICED_ROWS", 64)

    up, down = layer_tables(shape, 1500, ne)
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), shape.gs)
    cfg = type("c", (), dict(num_experts_per_tok=shape.top_k, num_experts=ne, moe_intermediate_size=shape.width,
                             hidden_size=shape.hidden))
    fused = moe.MoEBuffers(rows, cfg, DEV, shared=shape.shared)
    for seed in (1, 2):
        x = synthetic.activations(rows, shape.hidden, 1501 + seed).to(DEV)
        l = synthetic.logits(rows, ne + int(shape.shared), 1510 + seed).to(DEV)
        ref = moe.MoEBuffers(rows, cfg, DEV, shared=shape.shared)
        moe.select(l, ref, shape.top_k, ne)
        experts.gate_up(x, ex, ref.plan, ref.act.view(-1, ex.width), rows)
        experts.down(ref.act.view(-1, ex.width), ex, ref.plan, ref.y.view(-1, ex.dims), rows)
        want = moe.combine(ref.y, ref.wts)
        got = moe.decode(x, l, ex, fused, shape.top_k, ne)
        torch.cuda.synchronize()
        fused.check()
        assert torch.equal(fused.pick, ref.pick) and torch.equal(fused.wts, ref.wts)
        n = int(ref.plan.counts[0])
        assert torch.equal(fused.plan.counts, ref.plan.counts) and torch.equal(fused.plan.items[:n], ref.plan.items[:n])
        assert torch.equal(fused.plan.members, ref.plan.members)
        assert torch.equal(fused.act, ref.act) and torch.equal(fused.y, ref.y)
        assert torch.equal(got, want), seed


def test_decode_replays_in_a_graph_with_new_logits_and_inputs():
    """``decode`` captured once and replayed on changed logits and activations (in place): every replay equals the
    eager result, so the arrival counters the routing launch clears are right on every pass, not only the first."""

    shape, ne, rows = synthetic.C1, 24, 8
    up, down = layer_tables(shape, 1600, ne)
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), shape.gs)
    cfg = type("c", (), dict(num_experts_per_tok=shape.top_k, num_experts=ne, moe_intermediate_size=shape.width,
                             hidden_size=shape.hidden))
    buf, ref = moe.MoEBuffers(rows, cfg, DEV, shared=False), moe.MoEBuffers(rows, cfg, DEV, shared=False)
    x = synthetic.activations(rows, shape.hidden, 1601).to(DEV)
    l = synthetic.logits(rows, ne, 1602).to(DEV)
    out = torch.empty((rows, shape.hidden), dtype=torch.bfloat16, device=DEV)
    moe.decode(x, l, ex, buf, shape.top_k, ne, out)              # warm-up: scratch is allocated outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        moe.decode(x, l, ex, buf, shape.top_k, ne, out)
    for seed in (1, 2, 3):
        x.copy_(synthetic.activations(rows, shape.hidden, 1610 + seed).to(DEV))
        l.copy_(synthetic.logits(rows, ne, 1620 + seed).to(DEV))
        g.replay()
        torch.cuda.synchronize()
        want = moe.decode(x, l, ex, ref, shape.top_k, ne).clone()
        torch.cuda.synchronize()
        assert torch.equal(out, want), seed
    with pytest.raises(RuntimeError):
        moe.decode(x[:, :64], l, ex, buf, shape.top_k, ne)           # not the table's K
    with pytest.raises(ValueError):
        moe.decode(torch.cat([x, x]), torch.cat([l, l]), ex, buf, shape.top_k, ne)      # more rows than the buffers hold


def check_decode_forms(shape, ne, rows, seed, oracle=True, levels=0):
    """Every form of ``decode`` gives the bits of the separate kernels (twice in a row), ids equal the oracle's, and
    the output is within 2e-3 of the CPU oracle's layer."""

    gs, top_k, shared, swiglu, hidden, width = shape.gs, shape.top_k, shape.shared, shape.swiglu, shape.hidden, shape.width
    up, down = layer_tables(shape, 3000 + seed, ne)
    ex = experts.make([tuple(t.to(DEV) for t in m) for m in up], tuple(t.to(DEV) for t in down), gs)
    cfg = type("c", (), dict(num_experts_per_tok=top_k, num_experts=ne, moe_intermediate_size=width,
                             hidden_size=hidden))
    x = synthetic.activations(rows, hidden, 4000 + seed).to(DEV)
    l = synthetic.logits(rows, ne + int(shared), 5000 + seed)
    if levels:
        l = torch.round(l * levels) / levels          # few distinct values: ties inside every row
    l = l.to(DEV)
    ref = moe.MoEBuffers(rows, cfg, DEV, shared=shared)
    moe.select(l, ref, top_k, ne)
    experts.gate_up(x, ex, ref.plan, ref.act.view(-1, ex.width), rows)
    experts.down(ref.act.view(-1, ex.width), ex, ref.plan, ref.y.view(-1, ex.dims), rows)
    want = moe.combine(ref.y, ref.wts)
    saved = moe.FUSED_DECODE, moe.ROUTE_UP_LOGITS, moe.ROUTING_LAUNCH, moe.SLICED_DECODE, moe.SLICED_ROWS
    try:
        for path in ("route_up", "topk_then_up", "route_then_up", "one_launch", "sliced", "topk_then_sliced"):
            moe.FUSED_DECODE = path == "one_launch"
            moe.ROUTING_LAUNCH = path == "route_then_up"
            moe.ROUTE_UP_LOGITS = 0 if path.startswith("topk_then") else 1 << 30
            moe.SLICED_DECODE, moe.SLICED_ROWS = path.endswith("sliced"), 1024
            buf = moe.MoEBuffers(rows, cfg, DEV, shared=shared)
            for _ in range(2):
                got = moe.decode(x, l, ex, buf, top_k, ne)
                torch.cuda.synchronize()
                buf.check()
                assert torch.equal(buf.pick, ref.pick) and torch.equal(buf.wts, ref.wts), path
                assert torch.equal(buf.plan.members, ref.plan.members), path
                assert torch.equal(buf.act, ref.act) and torch.equal(buf.y, ref.y), path
                assert torch.equal(got, want), path
    finally:
        moe.FUSED_DECODE, moe.ROUTE_UP_LOGITS, moe.ROUTING_LAUNCH, moe.SLICED_DECODE, moe.SLICED_ROWS = saved
    picks, _ = orr.topk_rows(l.cpu().numpy(), ne, top_k, shared=shared)
    assert np.array_equal(ref.pick.cpu().numpy(), picks)
    if oracle:
        t = lambda m: (u32(m[0]), bits16(m[1]), bits16(m[2]))
        want_bits = native.moe_layer(bits16(x.cpu()), picks, ref.wts.cpu().numpy(), t(up[0]) if swiglu else None,
                                     t(up[1]) if swiglu else t(up[0]), t(down), gs)
        assert rel_l2(f32(want), ora.bf16_from_bits(want_bits)) <= TOL


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_of_the_decode_layer(seed):
    """Drawn shapes (hidden, width, experts, slots, group size, activation, rows) through ``check_decode_forms``."""

    import random

    rnd = random.Random(seed)
    gs = rnd.choice([32, 64])
    hidden, width = 64 * rnd.randint(1, 12), 64 * rnd.randint(1, 10)
    ne = rnd.choice([2, 3, 5, 8, 17, 33, 64, 100, 128, 130, 200])
    shared = rnd.random() < 0.4
    top_k = rnd.randint(1, min(8, ne))
    swiglu = rnd.random() < 0.5
    rows = rnd.choice([1, 2, 3, 5, 8, 13, 16, 17, 24, 33, 40])
    check_decode_forms(synthetic.MoEShape(f"drawn{seed}", hidden, ne, width, top_k, gs, swiglu, shared), ne, rows, seed)


@pytest.mark.parametrize("hidden,width,ne,top_k,gs,swiglu,shared,rows", [
    (64, 64, 256, 8, 64, False, False, 128),          # 1,024 pairs
    (128, 64, 64, 63, 32, True, True, 16),            # 64 slots a row
    (64, 128, 1023, 4, 64, False, True, 2),           # the most experts
    (64, 64, 1, 1, 32, False, False, 1024),           # one expert takes every pair
])
def test_the_decode_layer_at_its_limits(hidden, width, ne, top_k, gs, swiglu, shared, rows):
    check_decode_forms(synthetic.MoEShape("limit", hidden, ne, width, top_k, gs, swiglu, shared), ne, rows, 99)


@pytest.mark.parametrize("ne,top_k,shared,rows,levels", [(128, 6, False, 8, 2), (40, 8, True, 13, 1), (300, 5, False, 6, 2),
                                                         (16, 16, False, 64, 1), (700, 3, True, 2, 1)])
def test_tied_logits_through_the_decode_layer(ne, top_k, shared, rows, levels):
    """Logits on a grid of a few values, so every row holds runs of equal logits across its top-k boundary: a
    workgroup that finds its item from its pair's own row and a rank test on the other rows must break the ties as
    the selection passes do (lower id first)."""

    check_decode_forms(synthetic.MoEShape("ties", 128, ne, 64, top_k, 64, False, shared), ne, rows, 7, levels=levels)
