"""Many launches of the kernels that hand partial results from workgroup to workgroup inside one launch (the decode
layer's combine, the dense matmul's K slices): each result against the bits of the kernels that pass nothing between
workgroups.  The hand-offs order "stores acknowledged, then the count" without a fence, so what a handful of launches
shows in the other tests is shown here on a couple of thousand, on changing inputs, replayed from graphs as a serving
loop replays them.  Bounded: a fixed number of launches, and the loop ends at the first difference."""

import pytest
import torch

from tensorfold_amd import _lib, experts, moe, qmm, synthetic
from tests.test_gpu_moe import layer_tables

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROUNDS = 2000


def test_decode_layer_two_thousand_replays():
    """Configuration 1's layer (8 tokens, hidden 2688, width 1856, top-6) over three tables of 24 experts: the
    captured ``decode`` replayed on new inputs and logits each time against the captured separate kernels (top-k,
    pair sort, up, down, combine)."""

    shape, ne, rows, tables = synthetic.C1, 24, 8, 3
    cfg = type("c", (), dict(num_experts_per_tok=shape.top_k, num_experts=ne, moe_intermediate_size=shape.width,
                             hidden_size=shape.hidden))
    x = torch.empty((rows, shape.hidden), dtype=torch.bfloat16, device=DEV)
    l = torch.empty((rows, ne), dtype=torch.float32, device=DEV)
    xs = torch.stack([synthetic.activations(rows, shape.hidden, 7000 + i) for i in range(16)]).to(DEV)
    ls = torch.stack([synthetic.logits(rows, ne, 7100 + i) for i in range(17)]).to(DEV)
    x.copy_(xs[0])
    l.copy_(ls[0])
    layers = []
    for t in range(tables):
        up, down = layer_tables(shape, 7200 + t, ne)
        ex = experts.make([tuple(v.to(DEV) for v in m) for m in up], tuple(v.to(DEV) for v in down), shape.gs)
        buf, ref = moe.MoEBuffers(rows, cfg, DEV, shared=False), moe.MoEBuffers(rows, cfg, DEV, shared=False)
        got = torch.empty((rows, shape.hidden), dtype=torch.bfloat16, device=DEV)
        want = torch.empty_like(got)

        def fused(ex=ex, buf=buf, got=got):
            moe.decode(x, l, ex, buf, shape.top_k, ne, got)

        def separate(ex=ex, ref=ref, want=want):
            moe.select(l, ref, shape.top_k, ne)
            experts.gate_up(x, ex, ref.plan, ref.act.view(-1, ex.width), rows)
            experts.down(ref.act.view(-1, ex.width), ex, ref.plan, ref.y.view(-1, ex.dims), rows)
            moe.combine(ref.y, ref.wts, want)

        graphs = []
        for fn in (fused, separate):
            fn()                                     # scratch is made outside the capture
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                fn()
            graphs.append(g)
        # the graphs hold addresses, not references: everything they read or write lives as long as they do (entering
        # a capture empties the allocator's cache, which would unmap a table freed before it)
        layers.append((graphs, buf, ref, got, want, ex))
    for i in range(ROUNDS):
        x.copy_(xs[i % 16])
        l.copy_(ls[i % 17])
        (g_fused, g_sep), buf, ref, got, want, _ = layers[i % tables]
        g_fused.replay()
        g_sep.replay()
        if not (torch.equal(got, want) and torch.equal(buf.y, ref.y) and torch.equal(buf.pick, ref.pick)):
            pytest.fail(f"replay {i}: the decode layer's bits differ from the separate kernels'")
    torch.cuda.synchronize()
    for _, buf, _, _, _, _ in layers:
        buf.check()
        assert not buf.fused(shape.gs)["counters"].any()          # every arrival counter is back at zero


def test_dense_matmul_two_thousand_arrivals():
    """``tf_qmm`` on 1 to 8 rows with the weight's arrival counters (the last workgroup of a column tile adds the K
    slices) against the same call without counters, whose forms pass nothing between workgroups, two weights in
    turn, new rows every call."""

    n, k, gs = 4096, 4096, 64
    qs = [qmm.pack(*(t.to(DEV) for t in synthetic.affine_general(n, k, gs, 7300 + i)), gs) for i in range(2)]
    sk = qmm.split_k(n, k, gs)
    assert sk > 1
    pool = synthetic.activations(64, k, 7310).to(DEV)
    sums = qmm.group_sums(pool, gs)
    part = torch.empty((sk, 8, n), device=DEV, dtype=torch.float32)
    for i in range(ROUNDS):
        m, at, q = 1 + i % 8, (5 * i) % 56, qs[i % 2]
        rows, xs = pool[at:at + m], sums[at:at + m].contiguous()
        got = qmm.matmul(rows, q, xs)
        want = torch.empty((m, n), device=DEV, dtype=torch.bfloat16)
        _lib.call("tf_qmm", _lib.ptr(rows), rows.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales),
                  _lib.ptr(q.biases), q.scales.stride(0), _lib.ptr(want), _lib.ptr(part), None, 0, m, n, k, sk, gs,
                  qmm.bucket(m), 0, 1)
        if not torch.equal(got, want):
            pytest.fail(f"call {i} ({m} rows): the arriving form's bits differ from the counter-less form's")
    assert not qs[0].counters.any() and not qs[1].counters.any()
