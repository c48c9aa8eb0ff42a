"""From files to the kernels' inputs on the GPU: the reader's uploads, a projection, a Qwen-MoE layer and a
Nemotron-H block's experts built from safetensors files by name, EXL3 layers from a scanned folder, and row blocks of
a packed weight.  What is built from a file must equal, bit for bit, what the same tensors give when handed over in
memory (that path is checked against the oracle elsewhere), and each also runs once against the oracle."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import exl3 as ore
from oracle import native
from oracle import routing as orr
from tensorfold_amd import direct_read as dr
from tensorfold_amd import experts, moe, qmm, synthetic, weights
from tensorfold_amd.exl3 import checkpoint as ck
from tensorfold_amd.exl3 import linear
from tests.helpers import bits16, f32, rel_l2, u32, write_safetensors

pytestmark = pytest.mark.gpu
DEV = "cuda"


def on_gpu(files: dr.SafeTensors):
    return lambda name: files.get(name, DEV)


def test_uploads_equal_the_files_bytes(tmp_path, monkeypatch):
    """Ranges that start and end anywhere, longer than the staging ring, one after another through the same ring."""

    monkeypatch.setattr(dr, "PIECE", 4 * dr.ALIGN)
    rng = np.random.default_rng(1)
    blob = rng.integers(0, 256, 300_001, dtype=np.uint8)
    path = tmp_path / "blob.bin"
    path.write_bytes(blob.tobytes())
    reader = dr.Reader()
    for first, n in ((0, 300_001), (13, 70_000), (4096, 4096), (299_990, 11), (5, 1), (100, 0)):
        got = reader.read(path, first, n, DEV)
        assert got.device.type == "cuda" and got.dtype == torch.uint8
        assert np.array_equal(got.cpu().numpy(), blob[first:first + n]), (first, n)
    assert len(reader.ring) in (0, dr.RING)                       # 0 where this file system refuses O_DIRECT
    reader.close()
    assert not reader.ring
    with pytest.raises(IOError, match="short read"):
        reader.read(path, 299_990, 100, DEV)


def test_reading_ahead_onto_the_gpu(tmp_path):
    tensors = {f"t{i}": torch.from_numpy(np.random.default_rng(i).integers(0, 2 ** 31, (50 + i, 33), dtype=np.int32))
               for i in range(6)}
    path = tmp_path / "model.safetensors"
    write_safetensors(path, tensors)
    files = dr.SafeTensors([path])
    ahead = dr.ReadAhead(files.reader, threads=2, run=16 << 10, gap=0)
    ahead.queue([(name, p, a, a + n, (dt, shape)) for name, (p, a, n, dt, shape) in files.where.items()], DEV,
                cut=lambda raw, meta: raw.clone().view(dr.DTYPES[meta[0]]).reshape(meta[1]))
    for name, want in tensors.items():
        got = ahead.take(name)
        assert got.device.type == "cuda" and torch.equal(got.cpu(), want), name
    ahead.close()
    files.close()


def test_a_projection_from_a_file(tmp_path):
    w, s, b = synthetic.affine_general(192, 512, 64, 21)
    write_safetensors(tmp_path / "m.safetensors", {"lm_head.weight": w.view(torch.uint32), "lm_head.scales": s,
                                                   "lm_head.biases": b}, shift=40)
    files = dr.SafeTensors([tmp_path / "m.safetensors"])
    q = weights.linear(on_gpu(files), "lm_head")
    want = qmm.pack(w.to(DEV), s.to(DEV), b.to(DEV), 64)
    assert (q.n, q.k, q.gs, q.arith) == (192, 512, 64, want.arith)
    assert torch.equal(q.weight, want.weight) and torch.equal(q.scales, want.scales) and torch.equal(q.biases, want.biases)
    x = synthetic.activations(3, 512, 22)
    ref = native.affine_linear(bits16(x), u32(w), bits16(s), bits16(b), 64)
    assert rel_l2(f32(qmm.matmul(x.to(DEV), q)), ref) <= 2e-3
    with pytest.raises(ValueError, match="groups of 32"):
        weights.linear(on_gpu(files), "lm_head", gs=32)


def test_pack_takes_tensors_that_need_a_copy_first():
    """Scales and biases in another float type, or laid out with strides, are converted on the way in; each copy must
    outlive the launch's other arguments (two temporaries of one size would otherwise share one block of memory)."""

    w, s, b = (t.to(DEV) for t in synthetic.affine_general(128, 256, 64, 23))
    want = qmm.pack(w, s, b, 64)
    wide = lambda t: torch.stack([t.float(), t.float()], dim=-1)[..., 0]            # fp32, every other element
    got = qmm.pack(w, wide(s), wide(b), 64)
    assert not wide(s).is_contiguous()
    assert torch.equal(got.weight, want.weight) and torch.equal(got.scales, want.scales) and torch.equal(got.biases, want.biases)
    ws, ss, bs = (t.to(DEV) for t in synthetic.affine_general(64, 128, 64, 24, (3,)))
    table = experts.pack(ws, ss, bs, 64)
    assert torch.equal(experts.pack(ws, wide(ss), wide(bs), 64), table)
    assert torch.equal(experts.pack(ws, ss.half(), bs.half(), 64), experts.pack(ws, ss.half().bfloat16(), bs.half().bfloat16(), 64))


def qwen_layer(tmp_path, ne=12, d=512, ni=128, gs=64):
    """A layer under the names of an MLX Qwen-MoE checkpoint, in two files; the router rows stored at 8 bits."""

    rng = np.random.default_rng(5)
    t = {}
    for i, proj in enumerate(("gate_proj", "up_proj", "down_proj")):
        n, k = (d, ni) if proj == "down_proj" else (ni, d)
        for part, many, one in zip(("weight", "scales", "biases"), synthetic.affine(n, k, gs, 30 + i, (ne,)),
                                   synthetic.affine(n, k, gs, 40 + i)):
            t[f"model.layers.3.mlp.switch_mlp.{proj}.{part}"] = many
            t[f"model.layers.3.mlp.shared_expert.{proj}.{part}"] = one
    for name, rows in (("gate", ne), ("shared_expert_gate", 1)):
        t[f"model.layers.3.mlp.{name}.weight"] = torch.from_numpy(rng.integers(0, 2 ** 32, (rows, d // 4), dtype=np.uint32))
        t[f"model.layers.3.mlp.{name}.scales"] = torch.from_numpy(rng.uniform(2e-4, 6e-4, (rows, d // gs)).astype(np.float32)).bfloat16()
        t[f"model.layers.3.mlp.{name}.biases"] = (t[f"model.layers.3.mlp.{name}.scales"].float() * -128).bfloat16()
    names = sorted(t)
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", {n: t[n] for n in names[::2]})
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", {n: t[n] for n in names[1::2]}, shift=24)
    return t


def test_a_qwen_moe_layer_from_files(tmp_path):
    t = qwen_layer(tmp_path)
    ne, d, gs, top_k, p = 12, 512, 64, 4, "model.layers.3.mlp."
    files = dr.SafeTensors(sorted(tmp_path.glob("*.safetensors")))
    layer = weights.routed(p, on_gpu(files), top_k)
    files.close()
    assert layer.count == ne and layer.top_k == top_k and layer.experts.count == ne + 1 and layer.experts.swiglu

    tri = lambda name: tuple(t[f"{p}{name}.{part}"] for part in ("weight", "scales", "biases"))
    both = lambda proj: tuple(torch.cat([a, b[None]]) for a, b in zip(tri(f"switch_mlp.{proj}"), tri(f"shared_expert.{proj}")))
    up, down = [both("gate_proj"), both("up_proj")], both("down_proj")
    want = experts.make([tuple(v.to(DEV) for v in m) for m in up], tuple(v.to(DEV) for v in down), gs)
    assert torch.equal(layer.experts.up, want.up) and torch.equal(layer.experts.down, want.down)
    rows = torch.cat([weights.dequantize(*tri("gate")), weights.dequantize(*tri("shared_expert_gate"))]).bfloat16()
    assert layer.router.dtype == torch.bfloat16 and torch.equal(layer.router.cpu(), rows)

    # the whole layer against the oracle, on the logits the GPU router gives (so a near-tie cannot split the ids)
    x = synthetic.activations(5, d, 50)
    out = moe.run(x.to(DEV), layer)
    logits = moe.router(x.to(DEV), layer.router).cpu()
    picks, wts = orr.topk_rows(logits.numpy(), ne, top_k, shared=True)
    tables = [(u32(m[0].view(torch.int32)), bits16(m[1]), bits16(m[2])) for m in (*up, down)]
    ref = ora.bf16_from_bits(native.moe_layer(bits16(x), picks, wts, *tables, gs))
    assert rel_l2(f32(out), ref) <= 2e-3


def test_a_nemotron_blocks_experts_from_a_file(tmp_path):
    ne, w, d, gs, p = 6, 128, 256, 64, "backbone.layers.1.mixer."
    t = {}
    for name, (n, k, lead) in {"switch_mlp.fc1": (w, d, (ne,)), "switch_mlp.fc2": (d, w, (ne,)),
                               "shared_experts.up_proj": (2 * w, d, ()), "shared_experts.down_proj": (d, 2 * w, ())}.items():
        for part, v in zip(("weight", "scales", "biases"), synthetic.affine(n, k, gs, len(t) + 60, lead)):
            t[p + name + "." + part] = v
    write_safetensors(tmp_path / "model.safetensors", t)
    files = dr.SafeTensors([tmp_path / "model.safetensors"])
    ex = weights.folded(p, on_gpu(files), w)
    assert (ex.count, ex.swiglu, ex.width, ex.dims) == (ne + 2, False, w, d)

    tri = lambda name: tuple(t[f"{p}{name}.{part}"] for part in ("weight", "scales", "biases"))
    fc1, fc2 = weights.fold_shared(tri("switch_mlp.fc1"), tri("switch_mlp.fc2"), tri("shared_experts.up_proj"),
                                   tri("shared_experts.down_proj"), w)
    # a token's slots: two routed experts, then the shared expert's halves (ids E and E + 1), as the family routes
    picks = torch.tensor([[4, 1, ne, ne + 1], [0, 5, ne, ne + 1], [2, 4, ne, ne + 1]], dtype=torch.int32)
    x = synthetic.activations(3, d, 70)
    plan = experts.Plan(3, 4, ne + 2, DEV)
    experts.route(picks.to(DEV), plan, experts.TILE)
    act = torch.empty((12, w), dtype=torch.bfloat16, device=DEV)
    y = torch.empty((12, d), dtype=torch.float32, device=DEV)
    experts.gate_up(x.to(DEV), ex, plan, act, 3)
    experts.down(act, ex, plan, y, 3)
    as_np = lambda m: (u32(m[0]), f32(m[1]), f32(m[2]))
    want_act, want_y = ora.expert_pairs(f32(x), picks.numpy(), [as_np(fc1)], as_np(fc2), gs)
    assert rel_l2(f32(act), want_act) <= 2e-3 and rel_l2(f32(y), want_y) <= 2e-3


def exl3_folder(tmp_path):
    """Four layers: unmarked 3inst at 3 bits, marked mcg at 4 and mul1 at 2.5, and an older one with sign words and
    a bias; plus a plain tensor and a config."""

    rng = np.random.default_rng(9)
    made, t = {}, {}
    for prefix, cb, bits, k, n in (("model.layers.0.mlp.up_proj", "3inst", 3, 256, 128),
                                   ("model.layers.0.mlp.down_proj", "mcg", 4, 128, 256),
                                   ("model.layers.0.mlp.gate_proj", "mul1", 2.5, 256, 128),
                                   ("model.layers.0.attn.o_proj", "3inst", 4, 128, 128)):
        trellis, suh, svh = synthetic.exl3_layer(k, n, bits, int(10 * bits) + k)
        made[prefix] = dict(trellis=trellis, suh=suh, svh=svh, codebook=cb, bits=bits, bias=None)
        t[prefix + ".trellis"] = trellis
        if cb != "3inst":
            t[f"{prefix}.{cb}"] = torch.tensor(ck.MARKERS[cb] - (1 << 32), dtype=torch.int32)
        if prefix.endswith("o_proj"):
            signs = lambda v: torch.from_numpy(np.packbits((v.numpy() < 0).reshape(-1, 16), axis=1, bitorder="little")
                                               .view(np.int16).reshape(-1).copy())
            bias = torch.from_numpy((rng.standard_normal(n) * 0.1).astype(np.float16))
            t.update({prefix + ".su": signs(suh), prefix + ".sv": signs(svh), prefix + ".bias": bias})
            made[prefix].update(suh=torch.where(suh < 0, -1.0, 1.0).half(), svh=torch.where(svh < 0, -1.0, 1.0).half(), bias=bias)
        else:
            t.update({prefix + ".suh": suh, prefix + ".svh": svh})
    t["model.norm.weight"] = torch.ones(128, dtype=torch.bfloat16)
    write_safetensors(tmp_path / "model.safetensors", t, shift=8)
    return made, t


def test_exl3_layers_from_a_scanned_folder(tmp_path):
    made, t = exl3_folder(tmp_path)
    found = ck.scan(tmp_path)
    assert set(found.groups) == set(made) and not found.bad and set(found.plain) == {"model.norm.weight"}
    files = dr.SafeTensors(sorted(tmp_path.glob("*.safetensors")))
    layers = ck.load_groups(files, found.groups, DEV, plans={(4.0, 128, 256): (2, 2)})
    assert layers["model.layers.0.mlp.down_proj"].split == (2, 2)
    assert layers["model.layers.0.mlp.up_proj"].split == linear.plan(256, 128)
    for prefix, m in made.items():
        layer = layers[prefix]
        assert (layer.bits, layer.codebook) == (m["bits"], m["codebook"]) and (layer.bias is not None) == (m["bias"] is not None)
        want = ore.unpack(m["trellis"].numpy(), m["bits"], m["codebook"])
        assert np.array_equal(layer.unpack().cpu().numpy().view(np.uint16), want.view(np.uint16)), prefix
        assert torch.equal(layer.suh.cpu(), m["suh"]) and torch.equal(layer.svh.cpu(), m["svh"])
        x = synthetic.activations(4, layer.k, 80, dtype=torch.float16)
        ref = ore.forward(x.numpy(), m["trellis"].numpy(), m["suh"].numpy(), m["svh"].numpy(), m["bits"], m["codebook"],
                          None if m["bias"] is None else m["bias"].numpy(), half_input=True)
        assert rel_l2(f32(layer(x.to(DEV), out_dtype=torch.float32)), ref) <= 2e-3, prefix

    # a marker that holds another codebook's value is refused before anything is uploaded
    t["model.layers.0.mlp.down_proj.mcg"] = torch.tensor(ck.MARKERS["mul1"] - (1 << 32), dtype=torch.int32)
    other = tmp_path / "other"
    other.mkdir()
    write_safetensors(other / "model.safetensors", t)
    with pytest.raises(ValueError, match="mcg"):
        ck.load_groups(dr.SafeTensors([other / "model.safetensors"]), ck.scan(other).groups, DEV)


def test_row_blocks_of_a_packed_weight():
    w, s, b = synthetic.affine_general(448, 512, 64, 90)
    q = qmm.pack(w.to(DEV), s.to(DEV), b.to(DEV), 64)
    x = synthetic.activations(5, 512, 91).to(DEV)
    sk = qmm.split_k(q.n, q.k, q.gs)
    whole = qmm.matmul(x, q)
    view = qmm.rows(q, 64, 320)                                    # from a tile edge, two blocks of 128: a view
    assert view.weight.data_ptr() == q.weight[1].data_ptr() and view.scales.data_ptr() == q.scales[:, 64:].data_ptr()
    assert torch.equal(qmm.matmul(x, view, sk=sk), whole[:, 64:320])
    for a, e in ((100, 229), (0, 448), (321, 448), (63, 65)):       # anything else: the rows packed again
        part = qmm.rows(q, a, e)
        assert part.n == e - a and torch.equal(qmm.matmul(x, part, sk=sk), whole[:, a:e]), (a, e)
        got = qmm.unpack(part)
        assert torch.equal(got[0].cpu(), w[a:e]) and torch.equal(got[1].cpu(), s[a:e]) and torch.equal(got[2].cpu(), b[a:e])
    assert torch.equal(qmm.matmul_rows(x, [qmm.rows(q, 0, 128), qmm.rows(q, 128, 301), qmm.rows(q, 301, 448)]), whole)
    assert torch.equal(qmm.prefill_matmul(x, view), qmm.prefill_matmul(x, q)[:, 64:320])
    with pytest.raises(ValueError):
        qmm.rows(q, 300, 449)
