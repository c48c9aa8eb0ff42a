"""Kernel timings of the benchmark configurations that are not bench.py's headline: 0 (dense 4-bit projection),
2 (verify-window MoE layer), 3 (prompt chunk, grouped MFMA) and 4 (EXL3 projections).

    python bench_configs.py [c0] [c2] [c3] [c3d] [c4] [c4p] [glue] [c4x] [cal] [timeline] [timeline_c0] [timeline_c2] [timeline_c3]

One JSON line a configuration: time of one pass (hipGraph of back-to-back passes cycling over enough weight copies to
miss the 256 MB Infinity Cache, HIP events around the replay), algorithmic bytes or flops, and the fraction of the
MI355X peak (8 TB/s HBM, 2.5 PFLOP/s dense 16-bit MFMA).  Synthetic data drawn on the GPU; parity is the tests' job.
"""

from __future__ import annotations

import json
import sys
import time

import torch

from tensorfold_amd import experts, moe, qmm, synthetic
from tensorfold_amd.exl3 import linear as exl3

DEV = "cuda:0"
HBM, MFMA = 8000.0, 2500.0          # GB/s, TFLOP/s
# Vector-unit peak in lane-operations a second: 256 CUs x 4 SIMDs x 16 lanes a cycle at the 2.4 GHz peak clock.
VALU = 256 * 4 * 16 * 2.4e9
# Vector instructions the EXL3 linear kernel spends on a weight: its loop over a pair of k tiles decodes 64 weights a
# lane (4,096 a wave) in 310 vector instructions beside 16 matrix ones (counted in the compiled loop of
# linear_kernel<6, 0, 8>; the 3INST hash alone is a bit-field extract, a multiply, an add and a bit operation).
EXL3_VALU_PER_WEIGHT = 310 / 64


def graph_us(step, reps: int, window_ms: float = 25.0) -> float:
    """Mean time of ``step(i)`` over a replayed graph of ``reps`` calls, at the clock the card settles at under that
    load: the graph is replayed back to back for ``window_ms`` untimed, then for ``window_ms`` between two events
    with no synchronization inside, three times over (the median counts).  The shader clock follows the load with a
    delay of some milliseconds: a 2 ms burst between two idle waits runs at 1.7-1.8 GHz where the same kernels back
    to back run at 2.2 GHz (cycles a launch the same), and a prompt pass or a decode loop is the latter."""

    for i in range(3):
        step(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(reps):
            step(i)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    g.replay()
    b.record()
    torch.cuda.synchronize()
    n = max(1, min(2000, int(window_ms / max(a.elapsed_time(b), 1e-3) + 0.5)))
    times = []
    for _ in range(3):
        for _ in range(n):
            g.replay()
        a.record()
        for _ in range(n):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) * 1e3 / (n * reps))
    return sorted(times)[1]


def burst_us(step, reps: int) -> float:
    """The same graph timed as one replay between two idle waits (the median of five): a burst of a millisecond or
    two, which the card runs at the clock of an idle card woken up.  Reported beside ``graph_us`` where the difference
    matters (the matrix-bound legs), so that both regimes can be read from one run."""

    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(reps):
            step(i)
    g.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        time.sleep(0.02)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) * 1e3 / reps)
    return sorted(times)[2]


def rand_affine(n: int, k: int, gs: int, gen, lead=()):
    words = torch.randint(-(2 ** 31), 2 ** 31, (*lead, n, k // 8), generator=gen, device=DEV,
                          dtype=torch.int64).to(torch.int32)
    scales = (torch.rand((*lead, n, k // gs), generator=gen, device=DEV) * 0.018 + 0.002).bfloat16()
    return words, scales, (scales.float() * -8).bfloat16()


def c0() -> dict:
    n = k = 4096
    gen = torch.Generator(device=DEV).manual_seed(1)
    copies = [qmm.pack(*rand_affine(n, k, 64, gen), 64) for _ in range(40)]       # 40 x 9.4 MB
    out = {}
    for m in (1, 8):
        x = synthetic.activations(m, k, 7).to(DEV)
        y = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
        xs = qmm.group_sums(x, 64)                  # the producer of x makes these in a model
        part = torch.empty((qmm.split_k(n, k, 64), m, n), dtype=torch.float32, device=DEV)
        us = graph_us(lambda i: qmm.matmul(x, copies[i % len(copies)], xs, out=y, part=part), 120)
        nbytes = n * k // 2 + 2 * 2 * n * k // 64 + m * (k + n) * 2
        out[m] = {"us": us, "bytes": nbytes, "gbs": nbytes / us * 1e-3, "frac": nbytes / us * 1e-3 / HBM}
    # the prompt form of the same weight: 4,096 rows on the matrix cores
    m = 4096
    x = synthetic.activations(m, k, 8).to(DEV)
    y = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    us = graph_us(lambda i: qmm.prefill_matmul(x, copies[i % len(copies)], out=y), 12)
    flop = 2.0 * m * n * k
    prompt = {"rows": m, "us": us, "tflops": flop / us * 1e-6, "frac_mfma": flop / us * 1e-6 / MFMA,
              "burst_us": burst_us(lambda i: qmm.prefill_matmul(x, copies[i % len(copies)], out=y), 12)}
    # the reference's own prompt arithmetic on the same kernel: w = bf16(fma(q, s, b)), bf16 matrix instruction
    us_b = graph_us(lambda i: qmm.prefill_matmul(x, copies[i % len(copies)], out=y, arith=1), 12)
    prompt["bf16_arithmetic"] = {"us": us_b, "tflops": flop / us_b * 1e-6, "frac_mfma": flop / us_b * 1e-6 / MFMA}
    # the FP8 prompt path on the same weight: the rows quantized to e4m3 (a launch of its own), then the matmul; and
    # at groups of 32, where the per-group fma weighs twice as much
    xq = qmm.quantize_rows(x, 64)
    q_us = graph_us(lambda i: qmm.quantize_rows(x, 64), 12)
    m_us = graph_us(lambda i: qmm.prefill_matmul8(xq, copies[i % len(copies)], out=y), 12)
    fp8 = {"rows": m, "quantize_us": q_us, "matmul_us": m_us, "tflops": flop / m_us * 1e-6,
           "tflops_with_quantize": flop / (m_us + q_us) * 1e-6}
    del copies
    torch.cuda.empty_cache()
    g32 = [qmm.pack(*rand_affine(n, k, 32, gen), 32) for _ in range(24)]
    xq32 = qmm.quantize_rows(x, 32)
    us16 = graph_us(lambda i: qmm.prefill_matmul(x, g32[i % len(g32)], out=y), 12)
    us8 = graph_us(lambda i: qmm.prefill_matmul8(xq32, g32[i % len(g32)], out=y), 12)
    fp8["g32"] = {"f16_tflops": flop / us16 * 1e-6, "fp8_tflops": flop / us8 * 1e-6}
    return {"config": "c0: dense 4-bit/g64 projection, N = K = 4096 (the K slices added up in the matmul's launch; group sums given)",
            "bound": "hbm", "rows": out, "prompt_form": prompt, "prompt_form_fp8": fp8}


def moe_tables(shape, layers: int, gen):
    e = shape.experts + int(shape.shared)
    tabs = []
    for _ in range(layers):
        up = [rand_affine(shape.width, shape.hidden, shape.gs, gen, (e,)) for _ in range(2 if shape.swiglu else 1)]
        down = rand_affine(shape.hidden, shape.width, shape.gs, gen, (e,))
        tabs.append(experts.make(up, down, shape.gs))
        del up, down
    return tabs


def cfg_of(shape):
    return type("cfg", (), dict(num_experts_per_tok=shape.top_k, num_experts=shape.experts,
                                moe_intermediate_size=shape.width, hidden_size=shape.hidden))


def c2() -> dict:
    s, rows = synthetic.C2, 32
    gen = torch.Generator(device=DEV).manual_seed(2)
    tabs = moe_tables(s, 2, gen)                                                  # 2 x 1.0 GB
    x = synthetic.activations(rows, s.hidden, 1201).to(DEV)
    logits = [synthetic.logits(rows, s.experts + 1, 3000 + i).to(DEV) for i in range(16)]
    buf = moe.MoEBuffers(rows, cfg_of(s), DEV, shared=True)
    out = torch.empty((rows, s.hidden), dtype=torch.bfloat16, device=DEV)
    per_expert = 3 * (s.width * s.hidden // 2 + 2 * 2 * s.width * s.hidden // s.gs)
    uniq = []
    for l in logits:
        moe.select(l, buf, s.top_k, s.experts)
        torch.cuda.synchronize()
        uniq.append(int(buf.plan.counts[1]))
    mean_u = sum(uniq) / len(uniq)

    def step(i):
        moe.decode(x, logits[i % 16], tabs[i % 2], buf, s.top_k, s.experts, out)

    def step_api(i):               # the same layer through the reference-shaped calls, one launch each
        ex = tabs[i % 2]
        moe.select(logits[i % 16], buf, s.top_k, s.experts)
        experts.gate_up(x, ex, buf.plan, buf.act.view(-1, ex.width), rows)
        experts.down(buf.act.view(-1, ex.width), ex, buf.plan, buf.y.view(-1, ex.dims), rows)
        moe.combine(buf.y, buf.wts, out)

    def up_only(i):
        ex = tabs[i % 2]
        experts.gate_up(x, ex, buf.plan, buf.act.view(-1, ex.width), rows)

    def down_only(i):
        ex = tabs[i % 2]
        experts.down(buf.act.view(-1, ex.width), ex, buf.plan, buf.y.view(-1, ex.dims), rows)

    us = graph_us(step, 32)
    api_us = graph_us(step_api, 32)
    moe.select(logits[0], buf, s.top_k, s.experts)
    up_us, down_us = graph_us(up_only, 32), graph_us(down_only, 32)
    nbytes = mean_u * per_expert + rows * s.hidden * 2 * 2
    return {"config": "c2: verify-window MoE layer, 512 experts + shared, SwiGLU, top-10, g32, 32 rows",
            "bound": "hbm", "layer_us": us, "layer_us_separate_calls": api_us, "us_per_token": us / rows, "distinct_experts": mean_u, "bytes": nbytes,
            "gbs": nbytes / us * 1e-3, "frac": nbytes / us * 1e-3 / HBM, "up_kernel_us": up_us,
            "down_kernel_us": down_us, "up_gbs": uniq[0] * per_expert * 2 / 3 / up_us * 1e-3,
            "down_gbs": uniq[0] * per_expert / 3 / down_us * 1e-3}


def c3(tiles=((64, torch.float32), (128, torch.float32), ("128_y_bf16", torch.bfloat16), ("128_y_f16", torch.float16),
             ("128_bf16_arithmetic", torch.bfloat16))) -> dict:
    s, rows = synthetic.C2, 4096
    gen = torch.Generator(device=DEV).manual_seed(3)
    ex_f16 = moe_tables(s, 1, gen)[0]
    import dataclasses
    # the same tables on the reference's prompt arithmetic (bf16 weights, bf16 pair outputs: cuda/moe.py:99)
    ex_bf16 = dataclasses.replace(ex_f16, arith=experts.ARITH_BF16)
    x = synthetic.activations(rows, s.hidden, 1301).to(DEV)
    ids = synthetic.zipf_picks(rows, s.experts, s.top_k, 1302)
    picks = torch.cat([ids, torch.full((rows, 1), s.experts, dtype=torch.int32)], 1).contiguous().to(DEV)
    sel = synthetic.logits(rows, s.top_k + 1, 1303)
    wts = torch.cat([torch.softmax(sel[:, :-1], 1), torch.sigmoid(sel[:, -1:])], 1).bfloat16().float().contiguous().to(DEV)
    slots = s.top_k + 1
    out = {}
    # items of 64 and of 128 with fp32 pair outputs (this build's default), then items of 128 with the reference's
    # bf16 pair outputs (cuda/moe.py:99), which halve the traffic between the down projection and the combine, and
    # with fp16 ones: the same bytes at an eighth of the rounding
    for tile, ydt in tiles:
        key, tile = tile, 128 if isinstance(tile, str) else tile
        ex = ex_bf16 if key == "128_bf16_arithmetic" else ex_f16
        plan = experts.Plan(rows, slots, s.experts + 1, DEV, prefill=True)
        act = torch.empty((rows * slots, s.width), dtype=torch.bfloat16, device=DEV)
        y = torch.empty((rows * slots, s.hidden), dtype=ydt, device=DEV)
        res = torch.empty((rows, s.hidden), dtype=torch.bfloat16, device=DEV)

        def step(i):
            experts.route(picks, plan, tile)
            experts.gate_up(x, ex, plan, act, rows)
            experts.down(act, ex, plan, y, rows)
            moe.combine(y.view(rows, slots, s.hidden), wts, res)

        us = graph_us(step, 8)
        experts.route(picks, plan, tile)
        up_us = graph_us(lambda i: experts.gate_up(x, ex, plan, act, rows), 8)
        down_us = graph_us(lambda i: experts.down(act, ex, plan, y, rows), 8)
        route_us = graph_us(lambda i: experts.route(picks, plan, tile), 8)
        flop = rows * slots * 3 * 2 * s.hidden * s.width
        combine_us = graph_us(lambda i: moe.combine(y.view(rows, slots, s.hidden), wts, res), 8)
        out[key] = {"chunk_us": us, "combine_us": combine_us, "tokens_per_s": rows / us * 1e6, "flop": flop, "tflops": flop / us * 1e-6,
                     "frac": flop / us * 1e-6 / MFMA, "route_us": route_us, "up_us": up_us, "down_us": down_us,
                     "up_tflops": flop * 2 / 3 / up_us * 1e-6, "down_tflops": flop / 3 / down_us * 1e-6,
                     "items": int(plan.counts[0])}
    return {"config": "c3: prompt chunk of 4,096 tokens, Zipf(1.1) over 512 experts + shared, SwiGLU, g32 "
                      "(flops count the shared expert's 4,096 pairs)", "bound": "mfma", "tiles": out}


def c3d() -> dict:
    """Configuration 3 with the default pair outputs only (items of 128, fp16): the leg counters are collected on."""

    return c3(tiles=(("128_y_f16", torch.float16),))


def c4() -> dict:
    gen = torch.Generator(device=DEV).manual_seed(4)

    def layer(k, n):
        trellis = torch.randint(-2 ** 15, 2 ** 15, (k // 16, n // 16, 48), generator=gen, device=DEV,
                                dtype=torch.int32).to(torch.int16)
        sc = lambda size: (torch.rand(size, generator=gen, device=DEV) * 1.5 + 0.5).half()
        return exl3.Exl3Linear.from_tensors(trellis, sc(k), sc(n), "3inst", device=DEV)

    mlps = [(layer(5120, 17408), layer(5120, 17408), layer(17408, 5120)) for _ in range(4)]     # 4 x 100 MB
    stacks = [exl3.Exl3Stack.of([g, u]) for g, u, _ in mlps]          # gate and up side by side: one launch for both
    out = {}
    for m in (1, 8):
        x = synthetic.activations(m, 5120, 4200 + m, dtype=torch.float16).to(DEV)
        h = synthetic.activations(m, 17408, 4300 + m, dtype=torch.float16).to(DEV)
        ys = [torch.empty((m, 17408), dtype=torch.float16, device=DEV) for _ in range(2)]
        yd = torch.empty((m, 5120), dtype=torch.float16, device=DEV)
        xh, hh = torch.empty_like(x), torch.empty_like(h)
        z = torch.empty((16 * m * 17408,), dtype=torch.float32, device=DEV)

        def step(i):
            g, u, d = mlps[i % len(mlps)]
            g(x, ys[0], xh=xh, z=z)
            u(x, ys[1], xh=xh, z=z)
            d(h, yd, xh=hh, z=z)

        separate_us = graph_us(step, 48)
        y2 = torch.empty((2, m, 17408), dtype=torch.float16, device=DEV)
        xh2 = torch.empty((2, m, 5120), dtype=torch.float16, device=DEV)
        z2 = torch.empty((2 * 16 * m * 17408,), dtype=torch.float32, device=DEV)

        def step_stacked(i):
            stacks[i % len(stacks)](x, y2, xh=xh2, z=z2)
            mlps[i % len(mlps)][2](h, yd, xh=hh, z=z)

        stacked_us = graph_us(step_stacked, 48)
        # the whole MLP, SwiGLU included: the gate and up launch's workgroups apply it and the down projection's rotation
        whole = [exl3.Exl3MLP(stacks[i], mlps[i][2]) for i in range(len(mlps))]
        scratch = whole[0].scratch(m)
        us = graph_us(lambda i: whole[i % len(whole)](x, yd, scratch=scratch), 48)
        gate_us = graph_us(lambda i: mlps[i % 4][0](x, ys[0], xh=xh, z=z), 48)
        down_us = graph_us(lambda i: mlps[i % 4][2](h, yd, xh=hh, z=z), 48)
        per = 5120 * 17408 * 3 // 8
        nbytes = 3 * per + 3 * 2 * (5120 + 17408) + m * (2 * 5120 + 17408 + 17408 * 2 + 5120) * 2
        ops = 3 * 5120 * 17408 * EXL3_VALU_PER_WEIGHT          # lane-operations of one MLP's decode
        out[m] = {"mlp_us": us, "mlp_linears_only_us": stacked_us, "mlp_separate_calls_us": separate_us, "bytes": nbytes, "gbs": nbytes / us * 1e-3, "frac": nbytes / us * 1e-3 / HBM,
                  "gate_us": gate_us, "gate_gbs": per / gate_us * 1e-3, "down_us": down_us,
                  "down_gbs": per / down_us * 1e-3,
                  "valu": {"bound": "valu", "achieved": ops / us * 1e-6, "peak": VALU * 1e-12, "unit": "Tlane-op/s",
                           "frac": ops / us * 1e6 / VALU, "ops_per_weight": EXL3_VALU_PER_WEIGHT,
                           "floor_us": ops / VALU * 1e6}}
    return {"config": "c4: EXL3 3.0 bpw MLP down(silu(gate(x)) * up(x)), 5120 -> 17408 -> 5120, three launches (rotation; gate "
                      "and up with the SwiGLU and down's rotation; down); mlp_linears_only_us: the stack and the down layer "
                      "as two calls on independent inputs, no SwiGLU; mlp_separate_calls_us: three separate layers, no SwiGLU",
            "bound": "hbm", "rows": out}


def c4p() -> dict:
    """Prompt form of configuration 4's gate projection: input rotation, W_q decoded once a chunk, MFMA GEMM."""

    from tensorfold_amd.exl3 import prefill

    gen = torch.Generator(device=DEV).manual_seed(5)
    k, n = 5120, 17408
    trellis = torch.randint(-2 ** 15, 2 ** 15, (k // 16, n // 16, 48), generator=gen, device=DEV,
                            dtype=torch.int32).to(torch.int16)
    sc = lambda size: (torch.rand(size, generator=gen, device=DEV) * 1.5 + 0.5).half()
    layer = exl3.Exl3Linear.from_tensors(trellis, sc(k), sc(n), "3inst", device=DEV)
    ws = prefill.Workspace()
    out = {}
    for m in (512, 4096):
        x = synthetic.activations(m, k, 4400 + m, dtype=torch.float16).to(DEV)
        y = torch.empty((m, n), dtype=torch.float16, device=DEV)
        prefill.matmul(layer, x, y, ws)
        wt = prefill.decode(layer, ws)
        whole = graph_us(lambda i: prefill.matmul(layer, x, y, ws), 8)
        gemm = graph_us(lambda i: prefill.matmul(layer, x, y, ws, wt=wt), 8)
        dec = graph_us(lambda i: prefill.decode(layer, ws), 8)
        flops = 2.0 * m * k * n
        out[m] = {"matmul_us": whole, "decode_us": dec, "rot_gemm_us": gemm, "tflops": flops / whole * 1e-6,
                  "frac": flops / whole * 1e-6 / MFMA, "gemm_tflops": flops / gemm * 1e-6,
                  "decode_gbs": (k * n * 3 // 8 + k * n * 2) / dec * 1e-3}
    return {"config": "c4p: EXL3 3.0 bpw gate projection 5120 -> 17408 on a prompt chunk (rotation + decode + MFMA GEMM)",
            "bound": "mfma", "rows": out}


def glue_() -> dict:
    """The fused producers either side of the MoE layer: pair outputs -> residual + RMSNorm + group sums."""

    from tensorfold_amd import glue

    gen = torch.Generator(device=DEV).manual_seed(6)
    out = {}
    for name, rows, d, slots, top_k, ydt in (("decode_8x7x2688_f32", 8, 2688, 7, 6, torch.float32),
                                             ("window_32x11x2048_f32", 32, 2048, 11, 10, torch.float32),
                                             ("prompt_4096x9x2048_bf16", 4096, 2048, 9, 8, torch.bfloat16),
                                             ("prompt_4096x7x2688_bf16", 4096, 2688, 7, 6, torch.bfloat16)):
        copies = 1 if rows <= 32 else 3
        h = [torch.randn((rows, d), generator=gen, device=DEV).bfloat16() for _ in range(copies)]
        y = [(torch.randn((rows * slots, d), generator=gen, device=DEV) * 0.5).to(ydt) for _ in range(copies)]
        wt = torch.rand((rows, slots), generator=gen, device=DEV)
        w = (torch.rand((d,), generator=gen, device=DEV) + 0.5).bfloat16()
        us = graph_us(lambda i: glue.add_moe_norm(h[i % copies], y[i % copies], wt, w, 1e-5, top_k), 24)
        nbytes = rows * d * (slots * y[0].element_size() + 3 * 2) + rows * (d // 64 + slots) * 4 + d * 2
        out[name] = {"us": us, "bytes": nbytes, "gbs": nbytes / us * 1e-3, "frac": nbytes / us * 1e-3 / HBM}
    return {"config": "glue: add_moe_norm (weighted pair outputs + residual + RMSNorm + group sums), one launch",
            "bound": "hbm", "rows": out}


def c4x() -> dict:
    """EXL3 routed experts at decode: GLM-shaped layer (288 experts, 4096 -> 2048 -> 4096, 4.0 bpw mcg, top-8)."""

    from tensorfold_amd.exl3 import experts as xexp

    gen = torch.Generator(device=DEV).manual_seed(7)
    n_exp, d, width, top_k = 288, 4096, 2048, 8

    def trellis(k, n):
        return torch.randint(-2 ** 15, 2 ** 15, (n_exp, k // 16, n // 16, 64), generator=gen, device=DEV,
                             dtype=torch.int32).to(torch.int16)

    sc = lambda n, m: (torch.randn((n_exp, n), generator=gen, device=DEV) * m).half()
    ex = xexp.prepare_stacked(trellis(d, width), trellis(d, width), trellis(width, d), sc(d, 0.02), sc(d, 0.02),
                              sc(width, 0.5), sc(width, 0.5), sc(width, 0.05), sc(d, 0.2), "mcg")
    out = {}
    for rows in (1, 8):
        scratch = xexp.Scratch(ex, rows, top_k + 1)
        x = synthetic.activations(rows, d, 4500 + rows).to(DEV)
        y = torch.empty((rows, d), dtype=torch.float32, device=DEV)
        sets = []
        for i in range(4):                                  # four draws of experts, cycled: no draw finds the last one's weights cached
            sel = torch.stack([torch.randperm(n_exp, generator=gen, device=DEV)[:top_k] for _ in range(rows)]).int()
            sel = torch.cat([sel, torch.full((rows, 1), n_exp, dtype=torch.int32, device=DEV)], 1).contiguous()
            w = torch.cat([torch.rand((rows, top_k), generator=gen, device=DEV) * 0.2 + 0.05,
                           torch.ones((rows, 1), device=DEV)], 1).contiguous()
            sets.append((sel, w, len(set(sel[:, :top_k].flatten().tolist()))))
        us = graph_us(lambda i: xexp.routed(x, sets[i % 4][0], sets[i % 4][1], ex, scratch, y, rows, limit=10.0,
                                            act_mode=xexp.ACT_BF16), 16)
        distinct = sum(s[2] for s in sets) / 4
        nbytes = distinct * (3 * d * width // 2 + 2 * (3 * d + 3 * width)) + rows * d * 6
        out[rows] = {"layer_us": us, "distinct_experts": distinct, "bytes": nbytes, "gbs": nbytes / us * 1e-3,
                     "frac": nbytes / us * 1e-3 / HBM}
    return {"config": "c4x: EXL3 routed experts at decode, 288 experts 4096 -> 2048 -> 4096, 4.0 bpw mcg, top-8 (grouping + "
                      "rotation, gate/up, SwiGLU epilogue, down, rotation + combine: five launches)",
            "bound": "hbm", "rows": out}


def cal() -> dict:
    """What a tuned library GEMM gets from this chip at this clock, by the same graph method as the other legs:
    ``torch.matmul`` (hipBLASLt / rocBLAS) on fp16 and bf16 operands already in HBM, fp32 accumulation, at the dense
    prompt form's size (4096 cubed) and at configuration 4's gate projection (4096 x 5120 -> 17408).  No
    dequantization, no epilogue: the ceiling the 4-bit and EXL3 prompt kernels are judged against beside the
    2.5 PFLOP/s of the data sheet."""

    out = {}
    for name, (m, k, n) in {"4096x4096x4096": (4096, 4096, 4096), "4096x5120x17408": (4096, 5120, 17408)}.items():
        row = {}
        for dtype in (torch.float16, torch.bfloat16):
            gen = torch.Generator(device=DEV).manual_seed(3)
            a = torch.randn((m, k), generator=gen, device=DEV).to(dtype)
            # weight copies cycled as in the other legs ([N, K] each, used transposed, as a linear layer holds them)
            ws = [(torch.randn((n, k), generator=gen, device=DEV) * 0.05).to(dtype) for _ in range(6)]
            y = torch.empty((m, n), dtype=dtype, device=DEV)
            us = graph_us(lambda i: torch.matmul(a, ws[i % len(ws)].t(), out=y), 12)
            flop = 2.0 * m * n * k
            row[str(dtype).split(".")[-1]] = {"us": us, "tflops": flop / us * 1e-6, "frac_mfma": flop / us * 1e-6 / MFMA,
                                              "burst_us": burst_us(lambda i: torch.matmul(a, ws[i % len(ws)].t(), out=y), 12)}
            del ws
            torch.cuda.empty_cache()
        out[name] = row
    return {"config": "cal: torch.matmul (the vendor's tuned GEMM) at the prompt kernels' sizes, same timing method",
            "bound": "mfma", "sizes": out}


def timeline() -> dict:
    """Where a decode launch of configuration 1 spends its time, workgroup by workgroup: the two launches of the
    layer (routing + up projection; down projection + combine) run through the timeline build of the library, whose
    kernels note when each workgroup passes six marks.  Ten launches back to back in a graph, cycling the layers'
    tables; the marks kept are the last launch's, in microseconds from its first workgroup's start."""

    import ctypes

    import numpy as np

    import bench as b
    from tensorfold_amd import _lib, build

    marks = ("entry", "item_known", "first_loads_out", "wave0_streamed", "all_waves_streamed", "unit_done")
    tables, keep = b.device_tables(b.SHAPE, b.LAYERS, DEV)
    del keep
    out = {"config": "timeline: per-workgroup marks of the decode layer's two launches (configuration 1)",
           "marks": list(marks), "unit": "us from the launch's first workgroup", "launches": {}}
    for tokens in (1, 4, 8):
        layer = b.Layer(tokens, tables, DEV)
        layer.route_plans()
        plan = layer.plans[2]
        with _lib.through(build.timeline_lib()) as tl:
            for name, fn in (("route_up", lambda i: layer.up(i, plan)), ("down_combine", lambda i: layer.down(i, plan))):
                fn(0)
                torch.cuda.synchronize()
                if tl.tf_timeline_clear_moe():
                    raise RuntimeError(tl.tf_last_error().decode())
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for i in range(10):
                        fn(i)
                g.replay()
                g.replay()
                torch.cuda.synchronize()
                h = np.zeros((len(marks) + 2, 16384), dtype=np.uint64)
                if tl.tf_timeline_read_moe(h.ctypes.data_as(ctypes.c_void_p), h.shape[0], h.shape[1]):
                    raise RuntimeError(tl.tf_last_error().decode())
                where = h[len(marks)]
                h = h[:len(marks)].astype(np.int64)
                started, live = h[0] > 0, h[3] > 0
                t0 = h[0][started].min()
                row = {"workgroups": int(started.sum()), "streaming": int(live.sum())}
                for k, mark in enumerate(marks):
                    sel = (started if k == 0 else live) & (h[k] > 0)
                    if not sel.any():
                        continue
                    v = (h[k][sel] - t0) / 100.0
                    row[mark] = {"min": float(v.min()), "median": float(np.median(v)),
                                 "p90": float(np.percentile(v, 90)), "max": float(v.max())}
                d = (h[3] - h[2])[live] / 100.0
                row["wave0_stream_us"] = {"min": float(d.min()), "median": float(np.median(d)), "max": float(d.max())}
                # the compute unit of a workgroup: (XCC, engine, shader array, unit); how many streaming workgroups
                # each unit ran, and when the last of them finished
                hw = where[live]
                cu = ((hw >> np.uint64(32)) << np.uint64(8)) | ((hw >> np.uint64(8)) & np.uint64(0xFF))
                ids, count = np.unique(cu, return_counts=True)
                end = (h[5][live] - t0) / 100.0
                last = {int(n): [float(np.max(end[cu == u])) for u in ids[count == n]] for n in np.unique(count)}
                row["units_used"] = int(len(ids))
                row["by_workgroups_a_unit"] = {str(n): {"units": len(v), "mean_last_done_us": float(np.mean(v))}
                                               for n, v in last.items()}
                out["launches"][f"{tokens}_tokens_{name}"] = row
    del tables
    torch.cuda.empty_cache()
    # the EXL3 linear kernel of configuration 4 at one row: marks 0 entry, 1 the wave's walk over its k-tile pairs
    # begins, 2 wave 0 has walked, 3 every wave has, 4 the K split's partial sums are out and acknowledged, 5 done
    # (the last workgroup of a column block has added the splits and stored the rows)
    gen = torch.Generator(device=DEV).manual_seed(4)
    names = ("entry", "walk_begins", "wave0_walked", "all_waves_walked", "partials_out", "done")
    for label, (k, n), stacked in (("gate_5120x17408", (5120, 17408), 1), ("gate_and_up_stacked_2x5120x17408", (5120, 17408), 2),
                                  ("down_17408x5120", (17408, 5120), 1)):
        layers = []
        for _ in range(4):
            made = []
            for _ in range(stacked):
                trellis = torch.randint(-2 ** 15, 2 ** 15, (k // 16, n // 16, 48), generator=gen, device=DEV,
                                        dtype=torch.int32).to(torch.int16)
                sc = lambda size: (torch.rand(size, generator=gen, device=DEV) * 1.5 + 0.5).half()
                made.append(exl3.Exl3Linear.from_tensors(trellis, sc(k), sc(n), "3inst", device=DEV))
            layers.append(made[0] if stacked == 1 else exl3.Exl3Stack.of(made))
        x = synthetic.activations(1, k, 4201, dtype=torch.float16).to(DEV)
        lead = () if stacked == 1 else (stacked,)
        y = torch.empty((*lead, 1, n), dtype=torch.float16, device=DEV)
        xh = torch.empty((*lead, 1, k), dtype=torch.float16, device=DEV)
        z = torch.empty((stacked * 16 * n,), dtype=torch.float32, device=DEV)
        with _lib.through(build.timeline_lib()) as tl:
            layers[0](x, y, xh=xh, z=z)
            torch.cuda.synchronize()
            if tl.tf_timeline_clear_exl3():
                raise RuntimeError(tl.tf_last_error().decode())
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for i in range(12):
                    layers[i % 4](x, y, xh=xh, z=z)
            g.replay()
            g.replay()
            torch.cuda.synchronize()
            h = np.zeros((len(names) + 2, 16384), dtype=np.uint64)
            if tl.tf_timeline_read_exl3(h.ctypes.data_as(ctypes.c_void_p), h.shape[0], h.shape[1]):
                raise RuntimeError(tl.tf_last_error().decode())
        where = h[len(names)]
        h = h[:len(names)].astype(np.int64)
        live = h[5] > 0
        t0 = h[0][live].min()
        row = {"workgroups": int(live.sum())}
        hw = where[live]
        cu = ((hw >> np.uint64(32)) << np.uint64(8)) | ((hw >> np.uint64(8)) & np.uint64(0xFF))
        ids, count = np.unique(cu, return_counts=True)
        end = (h[5][live] - t0) / 100.0
        row["units_used"] = int(len(ids))
        row["by_workgroups_a_unit"] = {
            str(int(c)): {"units": int((count == c).sum()),
                          "mean_last_done_us": float(np.mean([end[cu == u].max() for u in ids[count == c]]))}
            for c in np.unique(count)}
        for i, mark in enumerate(names):
            sel = live & (h[i] > 0)
            v = (h[i][sel] - t0) / 100.0
            row[mark] = {"min": float(v.min()), "median": float(np.median(v)), "p90": float(np.percentile(v, 90)),
                         "max": float(v.max())}
        out["launches"][f"exl3_linear_1_row_{label}"] = row
        del layers
        torch.cuda.empty_cache()
    return out


def timeline_c2() -> dict:
    """The same marks for the two expert launches of configuration 2's layer (32 rows, 513 experts: the top-k runs in
    a launch before them, so the up launch finds its items from the picks), with each launch's own time beside them:
    how long a workgroup lives, how many are alive at once, how many a compute unit ran."""

    import ctypes

    import numpy as np

    from tensorfold_amd import _lib, build

    s, rows = synthetic.C2, 32
    gen = torch.Generator(device=DEV).manual_seed(2)
    tabs = moe_tables(s, 2, gen)
    x = synthetic.activations(rows, s.hidden, 1201).to(DEV)
    logits = [synthetic.logits(rows, s.experts + 1, 3000 + i).to(DEV) for i in range(4)]
    bufs = [moe.MoEBuffers(rows, cfg_of(s), DEV, shared=True) for _ in range(4)]
    out = torch.empty((rows, s.hidden), dtype=torch.bfloat16, device=DEV)
    for j, b in enumerate(bufs):          # routes each buffer's plan and fills its descriptors and activations
        moe.decode(x, logits[j], tabs[j % 2], b, s.top_k, s.experts, out)
    torch.cuda.synchronize()
    items = experts.max_items(rows * bufs[0].slots, s.experts + 1, moe.DESC_TILE)

    def up(i):
        b, ex = bufs[i % 4], tabs[i % 2]
        f, plan = b.fused(ex.gs), b.plan
        _lib.call("tf_moe_route_up", None, logits[0].stride(0), rows, s.experts, s.top_k, 1, ex.gs, int(ex.swiglu),
                  _lib.ptr(x), x.stride(0), _lib.ptr(ex.up), ex.dims, ex.width, _lib.ptr(b.pick), _lib.ptr(b.wts),
                  _lib.ptr(plan.members), _lib.ptr(plan.items), _lib.ptr(plan.counts), _lib.ptr(f["desc"]),
                  _lib.ptr(b.act.view(-1, ex.width)), ex.limit, items, None, 0)

    def down(i):
        b, ex = bufs[i % 4], tabs[i % 2]
        f = b.fused(ex.gs)
        _lib.call("tf_moe_down_combine", ex.gs, _lib.ptr(b.act.view(-1, ex.width)), rows, b.slots, _lib.ptr(ex.down),
                  ex.dims, ex.width, _lib.ptr(f["desc"]), _lib.ptr(b.wts), _lib.ptr(b.y), _lib.ptr(out),
                  f["counters"].data_ptr() + 4 * (1 + f["items"]), items)

    res = {"config": "timeline_c2: the decode layer's launches on configuration 2 (32 rows), each alone",
           "items": [int(b.fused(s.gs)["desc"].view(-1)[0]) for b in bufs],
           "topk_us": graph_us(lambda i: moe.select_rows(logits[i % 4], bufs[i % 4], s.top_k, s.experts), 32),
           "up_us": graph_us(up, 32), "down_us": graph_us(down, 32), "launches": {}}
    marks = 6
    with _lib.through(build.timeline_lib()) as tl:
        for name, fn in (("up", up), ("down", down)):
            fn(0)
            torch.cuda.synchronize()
            if tl.tf_timeline_clear_moe():
                raise RuntimeError(tl.tf_last_error().decode())
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for i in range(10):
                    fn(i)
            g.replay()
            g.replay()
            torch.cuda.synchronize()
            h = np.zeros((marks + 2, 16384), dtype=np.uint64)
            if tl.tf_timeline_read_moe(h.ctypes.data_as(ctypes.c_void_p), h.shape[0], h.shape[1]):
                raise RuntimeError(tl.tf_last_error().decode())
            where, h = h[marks], h[:marks].astype(np.int64)
            # a launch's workgroups differ from draw to draw: keep the marks of the last launch alone
            end = h[5].max()
            live = (h[5] > 0) & (h[0] > end - int(115 * res[name + "_us"]))
            t0 = h[0][live].min()
            quart = lambda v: [round(float(q), 2) for q in (v.min(), np.median(v), np.percentile(v, 90), v.max())]
            row = {"workgroups": int(live.sum()), "launch_us": float((end - t0) / 100.0)}
            for k, mark in enumerate(("entry", "item_known", "first_loads_out", "wave0_streamed", "all_waves_streamed",
                                      "unit_done")):
                sel = live & (h[k] > 0)
                if sel.any():
                    row[mark] = quart((h[k][sel] - t0) / 100.0)
            row["life_us"] = quart((h[5] - h[0])[live] / 100.0)
            hw = where[live]
            cu = ((hw >> np.uint64(32)) << np.uint64(8)) | ((hw >> np.uint64(8)) & np.uint64(0xFF))
            count = np.unique(cu, return_counts=True)[1]
            row["a_compute_unit"] = [int(count.min()), round(float(count.mean()), 2), int(count.max())]
            begin, done = (h[0][live] - t0) / 100.0, (h[5][live] - t0) / 100.0
            row["alive_at_us"] = {str(t): int((begin <= t).sum() - (done <= t).sum()) for t in (5, 15, 25, 35, 45, 55)}
            res["launches"][name] = row
    return res


def timeline_c0() -> dict:
    """The clock the dense prompt kernel runs at, read inside it through the timeline build: every workgroup counts the
    shader cycles (s_memtime) of its loop over K between two of its 100 MHz marks, and cycles over time is the clock of
    its compute unit.  The same launch (4096 cubed, 64 steps of 64 inputs) in a short burst after an idle wait, after
    hundreds of launches back to back, and on activations of zeros: the cycles a step stay, the clock does not."""

    import ctypes

    import numpy as np

    from tensorfold_amd import _lib, build

    n = k = m = 4096
    gen = torch.Generator(device=DEV).manual_seed(1)
    q = qmm.pack(*rand_affine(n, k, 64, gen), 64)
    x = synthetic.activations(m, k, 8).to(DEV)
    y = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    cases = []
    with _lib.through(build.timeline_lib()) as tl:
        def run(what, xin, launches, idle_s):
            torch.cuda.synchronize()
            time.sleep(idle_s)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(launches):
                qmm.prefill_matmul(xin, q, out=y)
            b.record()
            torch.cuda.synchronize()
            h = np.zeros((8, 16384), dtype=np.uint64)
            if tl.tf_timeline_read_prefill(h.ctypes.data_as(ctypes.c_void_p), h.shape[0], h.shape[1]):
                raise RuntimeError(tl.tf_last_error().decode())
            t = h.astype(np.int64)
            live = (t[5] > 0) & (t[3] > t[2])
            ghz = t[7][live] / ((t[3][live] - t[2][live]) * 10.0)
            cases.append({"case": what, "launches": launches, "us_a_launch": a.elapsed_time(b) * 1e3 / launches,
                          "clock_ghz": [round(float(v), 3) for v in np.percentile(ghz, [0, 50, 100])],
                          "cycles_a_step": round(float(np.median(t[7][live])) / (k // 64), 1),
                          "loop_us": round(float(np.median(t[3][live] - t[2][live])) / 100.0, 1)})

        for _ in range(3):
            qmm.prefill_matmul(x, q, out=y)
        run("a burst after 50 ms of idling", x, 12, 0.05)
        run("back to back", x, 100, 0.0)
        run("back to back", x, 500, 0.0)
        run("back to back", x, 2000, 0.0)
        run("zero activations, back to back", torch.zeros_like(x), 500, 0.0)
        run("a burst after 50 ms of idling", x, 12, 0.05)
    return {"config": "timeline_c0: the dense prompt kernel's clock and cycles, read inside the kernel (marks of each "
                      "case's last launch; clock as min / median / max over its 256 workgroups)", "cases": cases}


def timeline_c3() -> dict:
    """Per-unit marks of configuration 3's two expert launches (the eight-wave prompt kernel, items of 128, fp16 pair
    outputs) through the timeline build; a unit is an item's 512 weight columns, taken one after another by the
    workgroup that stays on a compute unit ("workgroups" below counts units): 0 the unit begins, 1 its rows are known
    (at once: they were fetched under the unit before), 2 first operands staged (the loop begins), 3 the loop over K
    done, 4 results issued, 5 results written.  By the item's rows: how long a unit takes and where; by compute unit:
    the gap between one unit's end and the next one's start, and when each went idle for good (the launch's tail)."""

    import ctypes

    import numpy as np

    from tensorfold_amd import _lib, build

    s, rows = synthetic.C2, 4096
    gen = torch.Generator(device=DEV).manual_seed(3)
    ex = moe_tables(s, 1, gen)[0]
    x = synthetic.activations(rows, s.hidden, 1301).to(DEV)
    ids = synthetic.zipf_picks(rows, s.experts, s.top_k, 1302)
    picks = torch.cat([ids, torch.full((rows, 1), s.experts, dtype=torch.int32)], 1).contiguous().to(DEV)
    slots = s.top_k + 1
    plan = experts.Plan(rows, slots, s.experts + 1, DEV, prefill=True)
    act = torch.empty((rows * slots, s.width), dtype=torch.bfloat16, device=DEV)
    y = torch.empty((rows * slots, s.hidden), dtype=torch.float16, device=DEV)
    experts.route(picks, plan, 128)
    experts.gate_up(x, ex, plan, act, rows)
    torch.cuda.synchronize()
    n_items = int(plan.counts[0])
    counts = plan.items[:n_items, 2].cpu().numpy()
    res = {"config": "timeline_c3: the prompt chunk's two expert launches, workgroup by workgroup", "items": n_items,
           "marks": ["entry", "rows_known", "loop_begins", "loop_done", "results_issued", "results_written"],
           "unit": "us", "launches": {}}
    with _lib.through(build.timeline_lib()) as tl:
        for name, fn, per_item in (("up", lambda: experts.gate_up(x, ex, plan, act, rows), 2),
                                   ("down", lambda: experts.down(act, ex, plan, y, rows), 4)):
            fn()
            torch.cuda.synchronize()
            if tl.tf_timeline_clear_prefill():
                raise RuntimeError(tl.tf_last_error().decode())
            fn()
            torch.cuda.synchronize()
            h = np.zeros((8, 16384), dtype=np.uint64)
            if tl.tf_timeline_read_prefill(h.ctypes.data_as(ctypes.c_void_p), h.shape[0], h.shape[1]):
                raise RuntimeError(tl.tf_last_error().decode())
            hw, t = h[6], h[:6].astype(np.int64)
            live = t[5] > 0
            t0 = t[0][live].min()
            us = (t[:, live] - t0) / 100.0
            group = np.nonzero(live)[0]
            item_rows = counts[np.minimum(group // per_item, n_items - 1)]
            cu = ((hw[live] >> np.uint64(32)) << np.uint64(8)) | ((hw[live] >> np.uint64(8)) & np.uint64(0xFF))
            row = {"workgroups": int(live.sum()), "span_us": float(us[5].max())}
            med = lambda v: round(float(np.median(v)), 2)
            by_rows = {}
            for lo, hi in ((1, 16), (17, 32), (33, 64), (65, 127), (128, 128)):
                m = (item_rows >= lo) & (item_rows <= hi)
                if m.any():
                    by_rows[f"{lo}-{hi}"] = {"workgroups": int(m.sum()), "life": med(us[5][m] - us[0][m]),
                                             "head": med(us[2][m] - us[0][m]), "loop": med(us[3][m] - us[2][m]),
                                             "issue_results": med(us[4][m] - us[3][m]),
                                             "results_acknowledged": med(us[5][m] - us[4][m])}
            row["by_item_rows"] = by_rows
            gaps, idle_from, per_cu = [], [], []
            for u in np.unique(cu):
                m = cu == u
                order = np.argsort(us[0][m])
                begin, end = us[0][m][order], us[5][m][order]
                gaps += list(begin[1:] - end[:-1])
                idle_from.append(end.max())
                per_cu.append(int(m.sum()))
            row["gap_between_workgroups_on_a_unit"] = {"median": med(gaps), "p90": round(float(np.percentile(gaps, 90)), 2)}
            idle = np.array(idle_from)
            row["units"] = len(idle_from)
            row["workgroups_a_unit"] = [min(per_cu), round(float(np.mean(per_cu)), 2), max(per_cu)]
            row["unit_idle_before_the_end_us"] = {"mean": round(float((idle.max() - idle).mean()), 2),
                                                   "p90": round(float(np.percentile(idle.max() - idle, 90)), 2)}
            res["launches"][name] = row
    return res


def main() -> int:
    torch.cuda.set_device(0)
    which = sys.argv[1:] or ["c0", "c2", "c3", "c4"]
    for name in which:
        res = {"c0": c0, "c2": c2, "c3": c3, "c3d": c3d, "c4": c4, "c4p": c4p, "glue": glue_, "c4x": c4x, "cal": cal, "timeline": timeline, "timeline_c2": timeline_c2, "timeline_c0": timeline_c0, "timeline_c3": timeline_c3}[name]()
        torch.cuda.empty_cache()
        print(json.dumps(res, default=lambda v: round(v, 4)), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
