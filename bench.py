"""Benchmark of the hot path on one MI355X: the 4-bit decode MoE layer of benchmark configuration 1.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens T]

A step is one pass of the layer (top-k routing, pair sort, up projection with relu^2, down projection, weighted
combine; two launches) over one batch of T tokens, all inputs resident in HBM.  Steps cycle over several layers' expert tables
(each 718 MB, together far past the 256 MB Infinity Cache) and over a pool of router logits, so every step streams
its experts from HBM as a model's forward pass does.  The K timed steps are one hipGraph replay; the dominant
kernels are then timed by themselves with HIP events around back-to-back launches on the same stream.  Prints one
JSON line.  Synthetic data, random-init weights (there are no checkpoints here).
"""

from __future__ import annotations

import argparse
import json
import sys
import time

import numpy as np
import torch

from tensorfold_amd import _lib, experts, moe, synthetic

HBM_PEAK_GBS = 8000.0
SHAPE = synthetic.C1
LAYERS = 4          # 4 x 718 MB of expert tables
POOL = 64           # distinct routing draws
PLANS = 16          # pre-routed plans the kernel timing cycles through


def device_tables(shape, layers: int, dev: str):
    """Random MLX tensors drawn on the GPU and packed; the MLX copies of layer 0 are kept for the CPU baseline."""

    g = torch.Generator(device=dev).manual_seed(1100)
    out, keep = [], None
    for layer in range(layers):
        def table(n, k):
            words = torch.randint(-(2 ** 31), 2 ** 31, (shape.experts, n, k // 8), generator=g, device=dev,
                                  dtype=torch.int64).to(torch.int32)
            scales = (torch.rand((shape.experts, n, k // shape.gs), generator=g, device=dev) * 0.018 + 0.002).bfloat16()
            return words, scales, (scales.float() * -8).bfloat16()
        up, down = table(shape.width, shape.hidden), table(shape.hidden, shape.width)
        out.append(experts.make([up], down, shape.gs))
        if layer == 0:
            keep = (up, down)
        del up, down
    return out, keep


class Layer:
    """One batch size's buffers and the launch sequence of a step."""

    def __init__(self, tokens: int, tables, dev: str) -> None:
        s = SHAPE
        self.tokens, self.tables = tokens, tables
        cfg = type("cfg", (), dict(num_experts_per_tok=s.top_k, num_experts=s.experts,
                                   moe_intermediate_size=s.width, hidden_size=s.hidden))
        self.buf = moe.MoEBuffers(tokens, cfg, dev, shared=False)
        self.plans = [moe.MoEBuffers(tokens, cfg, dev, shared=False) for _ in range(PLANS)]   # pre-routed, for kernel timing
        self.x = [synthetic.activations(tokens, s.hidden, 1101 + i).to(dev) for i in range(4)]
        self.logits = [synthetic.logits(tokens, s.experts, 2000 + i).to(dev) for i in range(POOL)]
        self.out = torch.empty((tokens, s.hidden), dtype=torch.bfloat16, device=dev)

    def route(self, i: int) -> None:
        moe.select(self.logits[i % POOL], self.buf, SHAPE.top_k, SHAPE.experts)

    def up(self, i: int, buf=None) -> None:
        """The routing + up projection launch alone."""

        ex, buf = self.tables[i % len(self.tables)], buf or self.buf
        f, x, l = buf.fused(SHAPE.gs), self.x[i % 4], self.logits[getattr(buf, "draw", i % POOL)]
        items = experts.max_items(self.tokens * buf.slots, SHAPE.experts, moe.DESC_TILE)
        _lib.call("tf_moe_route_up", _lib.ptr(l), l.stride(0), self.tokens, SHAPE.experts, SHAPE.top_k, 0, ex.gs,
                  int(ex.swiglu), _lib.ptr(x), x.stride(0), _lib.ptr(ex.up), ex.dims, ex.width, _lib.ptr(buf.pick),
                  _lib.ptr(buf.wts), _lib.ptr(buf.plan.members), _lib.ptr(buf.plan.items), _lib.ptr(buf.plan.counts),
                  _lib.ptr(f["desc"]), _lib.ptr(buf.act), ex.limit, items, None, 0)

    def down(self, i: int, buf=None) -> None:
        """The down projection + combine launch alone (the unit that completes a cell leaves its arrival counter at
        zero, so launches can follow one another)."""

        ex, buf = self.tables[i % len(self.tables)], buf or self.buf
        f = buf.fused(SHAPE.gs)
        items = experts.max_items(self.tokens * buf.slots, SHAPE.experts, moe.DESC_TILE)
        ctr = f["counters"]
        _lib.call("tf_moe_down_combine", ex.gs, _lib.ptr(buf.act), self.tokens, buf.slots, _lib.ptr(ex.down), ex.dims,
                  ex.width, _lib.ptr(f["desc"]), _lib.ptr(buf.wts), _lib.ptr(buf.y),
                  _lib.ptr(self.out), ctr.data_ptr() + 4 * (1 + f["items"]), items)

    def route_plans(self) -> float:
        """Route every pre-built plan on its own logits; returns the mean number of distinct experts a plan holds."""

        for j, b in enumerate(self.plans):
            b.draw = (7 * j + 3) % POOL          # the routing draw this buffer keeps for the kernel timings
            moe.decode(self.x[j % 4], self.logits[b.draw], self.tables[j % len(self.tables)], b,
                       SHAPE.top_k, SHAPE.experts)      # routes the plan and fills its descriptors and activations
        torch.cuda.synchronize()
        return float(np.mean([int(b.plan.counts[1]) for b in self.plans]))

    def combine(self) -> None:
        moe.combine(self.buf.y, self.buf.wts, self.out)

    def step(self, i: int) -> None:
        """One layer pass the way ``moe.run`` issues it: the routing launch, then up, down and combine launches, or
        (with ``moe.FUSED_DECODE``) the one fused experts launch."""

        moe.decode(self.x[i % 4], self.logits[i % POOL], self.tables[i % len(self.tables)], self.buf, SHAPE.top_k,
                   SHAPE.experts, self.out)

    def fused_experts(self, i: int, buf) -> None:
        """The fused experts launch alone, on a pre-routed buffer, with the small fill that clears its counters (the
        figure includes the fill)."""

        ex, f = self.tables[i % len(self.tables)], buf.fused(SHAPE.gs)
        f["counters"].zero_()
        n = self.tokens
        items = experts.max_items(n * buf.slots, SHAPE.experts, moe.DESC_TILE)
        ctr = f["counters"]
        _lib.call("tf_moe_decode_experts", ex.gs, int(ex.swiglu), _lib.ptr(self.x[i % 4]), self.x[i % 4].stride(0), n,
                  buf.slots, _lib.ptr(ex.up), _lib.ptr(ex.down), ex.dims, ex.width, _lib.ptr(f["desc"]),
                  _lib.ptr(buf.plan.counts), _lib.ptr(buf.wts), _lib.ptr(buf.act),
                  _lib.ptr(buf.y), _lib.ptr(self.out), ctr.data_ptr() + 4,
                  ctr.data_ptr() + 4 * (1 + f["items"]), _lib.ptr(ctr), ex.limit, items)

    def unique_experts(self, i: int) -> int:
        self.route(i)
        torch.cuda.synchronize()
        return int(self.buf.plan.counts[1])


def bytes_per_expert(shape) -> int:
    """Codes plus scales and biases of one expert's up and down matrices (the algorithmic bytes of a routed expert)."""

    per_matrix = shape.width * shape.hidden // 2 + 2 * 2 * shape.width * shape.hidden // shape.gs
    return 2 * per_matrix


def run_batch(tokens: int, tables, steps: int, warmup: int, dev: str) -> dict:
    s = SHAPE
    layer = Layer(tokens, tables, dev)
    uniq = [layer.unique_experts(i) for i in range(steps)]

    def graph_us(step) -> float:
        for i in range(warmup):
            step(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(steps):
                step(i)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e6

    layer_us = graph_us(layer.step)

    def other_path(i: int) -> None:
        moe.FUSED_DECODE = not moe.FUSED_DECODE
        try:
            layer.step(i)
        finally:
            moe.FUSED_DECODE = not moe.FUSED_DECODE

    other_us = graph_us(other_path)
    fused_layer_us, split_layer_us = (layer_us, other_us) if moe.FUSED_DECODE else (other_us, layer_us)

    def sliced_path(i: int) -> None:
        saved = moe.SLICED_DECODE, moe.FUSED_DECODE
        moe.SLICED_DECODE, moe.FUSED_DECODE = True, False
        try:
            layer.step(i)
        finally:
            moe.SLICED_DECODE, moe.FUSED_DECODE = saved

    # the layer as ONE launch cut along the intermediate width (what moe.SLICED_DECODE selects)
    sliced_layer_us = layer_us if moe.SLICED_DECODE and not moe.FUSED_DECODE else graph_us(sliced_path)

    # the two expert kernels by themselves: HIP events around back-to-back launches on the launch stream
    def kernel_us(fn) -> float:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 4 * PLANS
        for i in range(4):
            fn(i, layer.plans[i % PLANS])
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(reps):
                fn(i, layer.plans[(i // LAYERS) % PLANS])
        g.replay()
        torch.cuda.synchronize()
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / reps

    u0 = layer.route_plans()
    up_us, down_us = kernel_us(layer.up), kernel_us(layer.down)
    fused_us = kernel_us(layer.fused_experts)
    layer.buf.check()
    half = bytes_per_expert(s) // 2
    act_bytes = tokens * s.top_k * (s.hidden + s.width) * 2
    mean_u = float(np.mean(uniq))
    algo = mean_u * bytes_per_expert(s) + tokens * s.hidden * 2 * 2 + tokens * s.top_k * 8
    return {
        "tokens": tokens, "layer_us": layer_us, "us_per_token": layer_us / tokens, "unique_experts": mean_u,
        "layer_bytes": algo, "layer_gbs": algo / layer_us * 1e-3, "layer_frac": algo / layer_us * 1e-3 / HBM_PEAK_GBS,
        "fused_layer_us": fused_layer_us, "split_layer_us": split_layer_us, "sliced_layer_us": sliced_layer_us, "up_kernel_us": up_us, "down_kernel_us": down_us, "fused_kernel_us": fused_us,
        "fused_gbs": (u0 * 2 * half + act_bytes) / fused_us * 1e-3,
        "up_gbs": (u0 * half + act_bytes / 2) / up_us * 1e-3, "down_gbs": (u0 * half + act_bytes / 2) / down_us * 1e-3,
        "kernel_unique_experts": u0, "kernel_bytes": u0 * half,
    }


def cpu_baseline(keep, tokens: int, dev: str) -> dict:
    """The C oracle (dequant-then-matmul per selected expert, OpenMP) on one layer pass of ``tokens`` tokens, and a
    parity check of the GPU result against it on the same inputs."""

    from oracle import affine as ora
    from oracle import native
    from oracle import routing as orr

    s = SHAPE
    up, down = keep
    x = synthetic.activations(tokens, s.hidden, 1101)
    l = synthetic.logits(tokens, s.experts, 2000)
    picks, wts = orr.topk_rows(l.numpy(), s.experts, s.top_k, shared=False)
    used = np.unique(picks)
    remap = np.zeros(s.experts, dtype=np.int32)
    remap[used] = np.arange(len(used), dtype=np.int32)
    idx = torch.from_numpy(used.astype(np.int64)).to(dev)
    b16 = lambda t: t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
    cpu = lambda m: (m[0][idx].cpu().numpy().view(np.uint32), b16(m[1][idx]), b16(m[2][idx]))
    upc, downc = cpu(up), cpu(down)
    native.moe_layer(b16(x), remap[picks], wts, None, upc, downc, s.gs)             # warm-up
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        out = native.moe_layer(b16(x), remap[picks], wts, None, upc, downc, s.gs)
        times.append(time.perf_counter() - t0)
    # the GPU on the same inputs (layer 0's table)
    ex = experts.make([up], down, s.gs)
    cfg = type("cfg", (), dict(num_experts_per_tok=s.top_k, num_experts=s.experts, moe_intermediate_size=s.width,
                               hidden_size=s.hidden))
    buf = moe.MoEBuffers(tokens, cfg, dev, shared=False)
    moe.select(l.to(dev), buf, s.top_k, s.experts)
    experts.gate_up(x.to(dev), ex, buf.plan, buf.act.view(-1, s.width), tokens)
    experts.down(buf.act.view(-1, s.width), ex, buf.plan, buf.y.view(-1, s.hidden), tokens)
    got = moe.combine(buf.y, buf.wts).float().cpu().numpy().astype(np.float64)
    want = ora.bf16_from_bits(out).astype(np.float64)
    rel = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    ids_ok = bool(np.array_equal(buf.pick.cpu().numpy(), picks))
    med = float(np.median(times))
    return {"value": med / tokens * 1e6, "unit": "us/token", "cores": native.threads(), "kind": "port",
            "sample": f"one layer pass, {tokens} tokens x top-{s.top_k} ({len(used)} experts), median of 5",
            "parity_rel_l2": rel, "parity_ids_exact": ids_ok}


def other_configs() -> dict:
    """Short legs of the benchmark's other configurations (bench_configs.py's functions): the dense projection (0),
    the verify window (2), the prompt chunk on the matrix cores (3: chunk time and TFLOP/s) and the EXL3 MLP (4)."""

    import bench_configs as bc

    def rnd(v):
        if isinstance(v, dict):
            return {k: rnd(u) for k, u in v.items()}
        return round(v, 4) if isinstance(v, float) else v

    out = {}
    r = bc.c0()
    out["c0"] = {"workload": r["config"],
                 "rows": {str(m): {k: rnd(v) for k, v in d.items()} for m, d in r["rows"].items()},
                 "prompt_form": {k: rnd(v) for k, v in r["prompt_form"].items()},
                 "prompt_form_fp8": rnd(r["prompt_form_fp8"])}
    torch.cuda.empty_cache()
    r = bc.c2()
    out["c2"] = {k: rnd(v) for k, v in r.items() if k != "config"} | {"workload": r["config"]}
    torch.cuda.empty_cache()
    # pair outputs in fp16 between the down projection and the combine, as moe.run keeps them for prompts
    # (`python bench_configs.py c3` also times fp32 and the reference's bf16)
    r = bc.c3(tiles=(("128_y_f16", torch.float16),))
    t = r["tiles"]["128_y_f16"]
    out["c3"] = {"workload": r["config"], "bound": "mfma", "pair_outputs": "fp16", "chunk_us": rnd(t["chunk_us"]),
                 "tokens_per_s": rnd(t["tokens_per_s"]), "tflops": rnd(t["tflops"]), "peak_tflops": bc.MFMA,
                 "frac": rnd(t["frac"]), "flop": t["flop"], "route_us": rnd(t["route_us"]), "up_us": rnd(t["up_us"]),
                 "down_us": rnd(t["down_us"]), "combine_us": rnd(t["combine_us"]), "items": t["items"]}
    torch.cuda.empty_cache()
    r = bc.c4()
    # two rooflines: the stream of trellis words against HBM, and the decode's vector instructions against the
    # vector units, which is the one that binds (`roofline_valu`, of the 1-row pass)
    out["c4"] = {"workload": r["config"], "bound": "hbm", "roofline_valu": rnd(r["rows"][1]["valu"]),
                 "rows": {str(m): {k: rnd(v) for k, v in d.items()} for m, d in r["rows"].items()}}
    torch.cuda.empty_cache()
    # what the vendor's tuned plain GEMM reaches on this box at the prompt kernels' sizes, same timing method: the
    # ceiling the two prompt fractions above can be read against beside the data sheet's peak
    r = bc.cal()
    out["calibration"] = {"workload": r["config"], "sizes": rnd(r["sizes"])}
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=8, help="batch of the headline value (1, 4 and 8 are all reported)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the short legs of configurations 0, 2, 3 and 4 (the `configs` key of the line)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB in / 256 MiB out elementwise kernel three times: the known-size "
                         "dispatch that FETCH_SIZE / WRITE_SIZE counter readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus above 1 is not supported (the path has no multi-GPU code)",
              file=sys.stderr)
        return 2
    dev = "cuda:0"
    torch.cuda.set_device(0)
    tables, keep = device_tables(SHAPE, LAYERS, dev)
    results = {t: run_batch(t, tables, args.steps, args.warmup, dev) for t in sorted({1, 4, 8, args.tokens})}
    head = results[args.tokens]
    # HBM bytes a launch are counter readings (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE) of this same command, not
    # something a timing run can see: the line carries null and the summary of those two runs is kept beside the
    # kernel trace (profiles/expert_kernel_c1_decode_traffic.txt).
    traffic = None
    if moe.FUSED_DECODE:
        dom_us, dom_bytes = head["fused_kernel_us"], 2 * head["kernel_bytes"]
        dom = "moe_fused_kernel (up + down + combine"
    else:
        which = "up" if head["up_kernel_us"] >= head["down_kernel_us"] else "down"
        dom_us, dom_bytes = head[f"{which}_kernel_us"], head["kernel_bytes"]
        dom = ("route_up_kernel (routing + up projection" if which == "up" else "down_combine_kernel (down projection + combine")
    achieved = dom_bytes / dom_us * 1e-3
    line = {
        "metric": "moe_decode_layer_us_per_token", "value": head["us_per_token"], "unit": "us/token", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["layer_us"] * 1e-3,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 x int4 -> fp32",
        "data": "synthetic",
        "config": {"workload": f"benchmark configuration 1: {SHAPE.name}; {args.tokens} tokens a step; {LAYERS} layers' tables "
                               f"cycled", "tokens": args.tokens, "hidden": SHAPE.hidden, "experts": SHAPE.experts,
                   "intermediate": SHAPE.width, "top_k": SHAPE.top_k, "group_size": SHAPE.gs},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "kernel": f"{dom}, {head['kernel_unique_experts']:.1f} experts a launch)",
                     "kernel_us": dom_us, "bytes_per_launch": dom_bytes},
        "layer_hbm": {"achieved": head["layer_gbs"], "frac": head["layer_frac"], "unit": "GB/s",
                      "bytes_per_step": head["layer_bytes"]},
        "batches": {str(t): {k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()}
                    for t, r in results.items()},
    }
    if args.copy_probe:
        a = torch.ones(64 << 20, dtype=torch.float32, device=dev)
        b = torch.empty_like(a)
        for _ in range(3):
            torch.mul(a, 2.0, out=b)
        torch.cuda.synchronize()
        del a, b
    del tables
    torch.cuda.empty_cache()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(keep, args.tokens, dev)
    del keep
    torch.cuda.empty_cache()
    if not args.no_configs:
        line["configs"] = other_configs()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
