"""Benchmark configurations 1, 2 and 3 at their own sizes (128 experts; 512 experts + shared; a 4,096-token chunk with
Zipf(1.1) popularity) against the CPU oracle.  The expert tables are hundreds of megabytes, so they are drawn on the
GPU and only the experts that the checked rows use are copied back for the oracle; ids, sort permutation and items
are compared in full, bit for bit."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import native
from oracle import routing as orr
from tensorfold_amd import experts, moe, synthetic
from tests.helpers import bits16, f32, max_abs, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3          # relative L2 on bf16 outputs with fp32 accumulation, the benchmark's bound


def device_layer(shape, seed):
    """MLX tensors of every expert of ``shape`` (shared expert last) drawn on the GPU, and the packed layer."""

    gen = torch.Generator(device=DEV).manual_seed(seed)
    e = shape.experts + int(shape.shared)

    def table(n, k):
        words = torch.randint(-(2 ** 31), 2 ** 31, (e, n, k // 8), generator=gen, device=DEV,
                              dtype=torch.int64).to(torch.int32)
        scales = (torch.rand((e, n, k // shape.gs), generator=gen, device=DEV) * 0.018 + 0.002).bfloat16()
        return words, scales, (scales.float() * -8).bfloat16()

    up = [table(shape.width, shape.hidden) for _ in range(2 if shape.swiglu else 1)]
    down = table(shape.hidden, shape.width)
    return up, down, experts.make(up, down, shape.gs)


def oracle_rows(shape, up, down, x, picks, wts, prefill=False):
    """The CPU oracle's layer on the given rows, holding only the experts those rows use (ids renumbered)."""

    used = np.unique(picks)
    remap = np.full(shape.experts + 1, -1, dtype=np.int32)
    remap[used] = np.arange(len(used), dtype=np.int32)
    idx = torch.from_numpy(used.astype(np.int64)).to(DEV)
    cpu = lambda m: (m[0][idx].cpu().numpy().view(np.uint32), bits16(m[1][idx]), bits16(m[2][idx]))
    gate = cpu(up[0]) if shape.swiglu else None
    out = native.moe_layer(bits16(x), remap[picks], wts, gate, cpu(up[-1]), cpu(down), shape.gs, prefill=prefill)
    return ora.bf16_from_bits(out)


def cfg_of(shape):
    return type("cfg", (), dict(num_experts_per_tok=shape.top_k, num_experts=shape.experts,
                                moe_intermediate_size=shape.width, hidden_size=shape.hidden))


@pytest.mark.parametrize("tokens", [1, 4, 8])
def test_config1_at_full_size(tokens):
    """128 experts, D 2688, NI 1856, relu^2, top-6, g64 through ``moe.decode`` (two launches)."""

    shape = synthetic.C1
    up, down, ex = device_layer(shape, 11000)
    x = synthetic.activations(tokens, shape.hidden, 11001)
    l = synthetic.logits(tokens, shape.experts, 11002)
    buf = moe.MoEBuffers(tokens, cfg_of(shape), DEV, shared=False)
    out = moe.decode(x.to(DEV), l.to(DEV), ex, buf, shape.top_k, shape.experts)
    torch.cuda.synchronize()
    picks, wts = orr.topk_rows(l.numpy(), shape.experts, shape.top_k, shared=False)
    assert np.array_equal(buf.pick.cpu().numpy(), picks)
    items, members, distinct = orr.plan(picks, shape.experts, experts.TILE)
    assert np.array_equal(buf.plan.members.cpu().numpy(), members)
    assert buf.plan.counts.cpu().tolist() == [len(items), distinct, 0, 0]
    assert np.array_equal(buf.plan.items[:len(items)].cpu().numpy(), items)
    want = oracle_rows(shape, up, down, x, picks, buf.wts.cpu().numpy())
    err = rel_l2(f32(out), want)
    print(f"config 1 at full size, {tokens} tokens: rel-L2 {err:.2e}, max-abs {max_abs(f32(out), want):.3e}")
    assert err <= TOL
    # a row's bits do not depend on the rows beside it
    one = moe.MoEBuffers(1, cfg_of(shape), DEV, shared=False)
    for r in {0, tokens - 1}:
        alone = moe.decode(x[r:r + 1].to(DEV), l[r:r + 1].to(DEV), ex, one, shape.top_k, shape.experts)
        assert torch.equal(alone[0], out[r]), r


def test_config2_at_full_size():
    """512 experts + the shared one, D 2048, NI 512, SwiGLU, top-10, g32, 32 rows (8 lanes x 4 draft tokens)."""

    shape, rows = synthetic.C2, 32
    up, down, ex = device_layer(shape, 12000)
    x = synthetic.activations(rows, shape.hidden, 12001)
    l = synthetic.logits(rows, shape.experts + 1, 12002)
    buf = moe.MoEBuffers(rows, cfg_of(shape), DEV, shared=True)
    out = moe.decode(x.to(DEV), l.to(DEV), ex, buf, shape.top_k, shape.experts)
    torch.cuda.synchronize()
    picks, wts = orr.topk_rows(l.numpy(), shape.experts, shape.top_k, shared=True)
    assert np.array_equal(buf.pick.cpu().numpy(), picks)
    items, members, distinct = orr.plan(picks, shape.experts + 1, experts.TILE)
    assert np.array_equal(buf.plan.members.cpu().numpy(), members)
    assert buf.plan.counts.cpu().tolist() == [len(items), distinct, 0, 0]
    assert np.array_equal(buf.plan.items[:len(items)].cpu().numpy(), items)
    want = oracle_rows(shape, up, down, x, picks, buf.wts.cpu().numpy())
    err = rel_l2(f32(out), want)
    print(f"config 2 at full size: rel-L2 {err:.2e}, max-abs {max_abs(f32(out), want):.3e}, {distinct} experts")
    assert err <= TOL
    # the same window through the reference-shaped separate calls: the same bits
    ref = moe.MoEBuffers(rows, cfg_of(shape), DEV, shared=True)
    moe.select(l.to(DEV), ref, shape.top_k, shape.experts)
    experts.gate_up(x.to(DEV), ex, ref.plan, ref.act.view(-1, ex.width), rows)
    experts.down(ref.act.view(-1, ex.width), ex, ref.plan, ref.y.view(-1, ex.dims), rows)
    assert torch.equal(moe.combine(ref.y, ref.wts), out)


def chunk_inputs(shape, rows, seed):
    ids = synthetic.zipf_picks(rows, shape.experts, shape.top_k, seed)
    picks = torch.cat([ids, torch.full((rows, 1), shape.experts, dtype=torch.int32)], 1).contiguous()
    sel = synthetic.logits(rows, shape.top_k + 1, seed + 1)
    wts = torch.cat([torch.softmax(sel[:, :-1], 1).bfloat16().float(),
                     torch.sigmoid(sel[:, -1:].bfloat16().float()).bfloat16().float()], 1).contiguous()
    return picks, wts


def run_chunk(ex, x, picks, wts, tile, y_dtype=torch.float32):
    rows, slots = picks.shape
    plan = experts.Plan(rows, slots, ex.count, DEV, prefill=True)
    experts.route(picks, plan, tile)
    act = torch.empty((rows * slots, ex.width), dtype=torch.bfloat16, device=DEV)
    y = torch.empty((rows * slots, ex.dims), dtype=y_dtype, device=DEV)
    experts.gate_up(x, ex, plan, act, rows)
    experts.down(act, ex, plan, y, rows)
    return moe.combine(y.view(rows, slots, ex.dims), wts), plan


def test_config3_at_full_size():
    """A 4,096-token chunk, 10 distinct experts a token drawn Zipf(1.1) over 512 plus the shared expert (45,056
    pairs): tokens sorted by expert bit-exact, 96 sampled token rows within 2e-3 of the oracle's layer, and rows
    bit-equal to what a small chunk holding them gives (a row's bits do not depend on the chunk)."""

    shape, rows = synthetic.C2, 4096
    up, down, ex = device_layer(shape, 13000)
    x = synthetic.activations(rows, shape.hidden, 13001)
    picks, wts = chunk_inputs(shape, rows, 13002)
    xd, pd, wd = x.to(DEV), picks.to(DEV), wts.to(DEV)
    outs = {}
    for tile in (64, 128):
        outs[tile], plan = run_chunk(ex, xd, pd, wd, tile)
        torch.cuda.synchronize()
        items, members, distinct = orr.plan(picks.numpy(), shape.experts + 1, tile)
        assert np.array_equal(plan.members.cpu().numpy(), members), tile
        # items, distinct experts, and the prompt kernels' ticket word back at zero after the two launches
        assert plan.counts.cpu().tolist() == [len(items), distinct, 0, 0], tile
        assert np.array_equal(plan.items[:len(items)].cpu().numpy(), items), tile
    assert torch.equal(outs[64], outs[128])
    counts = np.bincount(picks.numpy().reshape(-1), minlength=shape.experts + 1)
    assert counts[shape.experts] == rows and counts[:shape.experts].max() > 2000          # the skew is there
    rng = np.random.default_rng(5)
    sample = np.sort(rng.choice(rows, 96, replace=False))
    want = oracle_rows(shape, up, down, x[sample], picks[sample].numpy(), wts[sample].numpy())
    got = f32(outs[128][torch.from_numpy(sample).to(DEV)])
    err = rel_l2(got, want)
    print(f"config 3 at full size: rel-L2 {err:.2e}, max-abs {max_abs(got, want):.3e} over {len(sample)} rows, "
          f"{len(items)} items of up to 128, {distinct} experts")
    assert err <= TOL
    idx = torch.from_numpy(sample[:40]).to(DEV)
    small, _ = run_chunk(ex, xd[idx].contiguous(), pd[idx].contiguous(), wd[idx].contiguous(), 64)
    assert torch.equal(small, outs[128][idx])
    # pair outputs kept in fp16 between the down projection and the combine, as moe.run keeps a prompt's
    half, _ = run_chunk(ex, xd, pd, wd, 128, torch.float16)
    got16 = f32(half[torch.from_numpy(sample).to(DEV)])
    err16 = rel_l2(got16, want)
    print(f"config 3 at full size, fp16 pair outputs: rel-L2 {err16:.2e}, max-abs {max_abs(got16, want):.3e}")
    assert err16 <= TOL
    small16, _ = run_chunk(ex, xd[idx].contiguous(), pd[idx].contiguous(), wd[idx].contiguous(), 64, torch.float16)
    assert torch.equal(small16, half[idx])
