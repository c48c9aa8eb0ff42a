"""EXL3 checkpoints read from their headers: which groups are layers and why another is not, a mixed folder sorted
into layers, plain tensors and broken groups, and what config.json may say.  (The cases of the reference's
tests/test_exl3_format.py:137-233.)"""

import json
import struct

import pytest

from tensorfold_amd.exl3 import checkpoint as ck
from tensorfold_amd.exl3 import format as fmt


def entry(dtype: str, shape: list[int]) -> dict:
    return {"dtype": dtype, "shape": shape}


GOOD = {"trellis": entry("I16", [256, 768, 32]), "suh": entry("F16", [4096]), "svh": entry("F16", [12288]),
        "mul1": entry("I32", [])}


def test_a_group_with_fp16_scales_and_a_marker():
    g = ck.parse_group("model.layers.0.self_attn.q_proj", GOOD, ["b.safetensors", "a.safetensors", "a.safetensors"])
    assert (g.bits, g.codebook, g.k, g.n, g.in_scales, g.out_scales, g.bias) == (2, "mul1", 4096, 12288, "suh", "svh", False)
    assert g.trellis_bytes == 4096 * 12288 * 2 // 8 and g.files == ("a.safetensors", "b.safetensors")
    assert g.describe() == "model.layers.0.self_attn.q_proj: EXL3 2-bit mul1, K=4096 N=12288"


def test_half_bits_sign_words_and_a_bias():
    assert ck.parse_group("p", {**GOOD, "trellis": entry("I16", [256, 768, 40])}).bits == 2.5
    g = ck.parse_group("p", {"trellis": entry("I16", [8, 8, 64]), "su": entry("I16", [8]), "sv": entry("I16", [8]),
                             "bias": entry("F16", [128])})
    assert (g.bits, g.codebook, g.in_scales, g.out_scales, g.bias) == (4, "3inst", "su", "sv", True)
    mcg = {**{k: v for k, v in GOOD.items() if k != "mul1"}, "mcg": entry("I32", [])}
    assert ck.parse_group("p", mcg).codebook == "mcg"


@pytest.mark.parametrize("parts,why", [
    ({**GOOD, "mcg": entry("I32", [])}, "both"),
    ({k: v for k, v in GOOD.items() if k != "suh"}, "input scales"),
    ({k: v for k, v in GOOD.items() if k != "svh"}, "output scales"),
    ({**GOOD, "svh": entry("F16", [100])}, "svh"),
    ({**GOOD, "suh": entry("BF16", [4096])}, "suh"),
    ({**GOOD, "trellis": entry("I16", [256, 768, 72])}, "bits"),
    ({**GOOD, "trellis": entry("I32", [256, 768, 32])}, "int16"),
    ({k: v for k, v in {**GOOD, "trellis": entry("I16", [256, 768, 40])}.items() if k != "mul1"}, "mul1"),
    ({**GOOD, "trellis": entry("I16", [4, 768, 32]), "suh": entry("F16", [64])}, "multiples"),
    ({k: v for k, v in GOOD.items() if k != "trellis"}, "trellis"),
])
def test_groups_that_are_refused_say_why(parts, why):
    with pytest.raises(ValueError, match=why) as refused:
        ck.parse_group("some.prefix", parts)
    assert str(refused.value).startswith("some.prefix: ")


def write_safetensors(path, tensors: dict[str, tuple[str, list[int], bytes]]) -> None:
    header, blob = {"__metadata__": {"format": "pt"}}, b""
    for name, (dtype, shape, data) in tensors.items():
        header[name] = {"dtype": dtype, "shape": shape, "data_offsets": [len(blob), len(blob) + len(data)]}
        blob += data
    text = json.dumps(header).encode()
    path.write_bytes(struct.pack("<Q", len(text)) + text + blob)


def layer(prefix: str, k: int, n: int, bits: float, marker: str | None = "mul1", value: int | None = None) -> dict:
    words = fmt.tile_words(bits)
    out = {f"{prefix}.trellis": ("I16", [k // 16, n // 16, words], bytes(2 * (k // 16) * (n // 16) * words)),
           f"{prefix}.suh": ("F16", [k], bytes(2 * k)), f"{prefix}.svh": ("F16", [n], bytes(2 * n))}
    if marker:
        out[f"{prefix}.{marker}"] = ("I32", [], struct.pack("<I", ck.MARKERS[marker] if value is None else value))
    return out


def test_a_mixed_folder(tmp_path):
    """Three widths in one MoE layer, two marked codebooks and an unmarked one, layers spread over two files, plain
    tensors (one of them a plain layer's .bias), and a trellis without scales."""

    first, second = {}, {}
    first.update(layer("model.layers.0.mlp.experts.0.gate_proj", 256, 128, 2))
    first.update(layer("model.layers.0.mlp.experts.1.gate_proj", 256, 128, 3.5))
    first.update(layer("model.layers.1.mlp.experts.0.gate_proj", 256, 128, 5))
    first.update(layer("model.layers.0.self_attn.q_proj", 128, 256, 4, "mcg"))
    second.update(layer("model.layers.0.self_attn.k_proj", 128, 128, 3, None))
    head = layer("lm_head", 128, 512, 6)
    second["lm_head.trellis"] = head.pop("lm_head.trellis")              # a group's parts may sit in different files
    first.update(head)
    first["model.embed_tokens.weight"] = ("BF16", [512, 128], bytes(2 * 512 * 128))
    first["model.layers.0.input_layernorm.weight"] = ("BF16", [128], bytes(256))
    first["model.layers.0.conv.bias"] = ("BF16", [128], bytes(256))
    second["model.layers.1.self_attn.o_proj.trellis"] = ("I16", [8, 8, 32], bytes(2 * 8 * 8 * 32))
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", first)
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", second)
    (tmp_path / "config.json").write_text(json.dumps({"model_type": "fake", "quantization_config": {
        "quant_method": "exl3", "version": "1.5.0", "bits": 3.1, "head_bits": 6, "codebook": "mul1"}}))

    found = ck.scan(tmp_path)
    assert len(found.groups) == 6
    assert found.bad == {"model.layers.1.self_attn.o_proj": "no input scales (.suh or .su)"}
    assert found.groups["model.layers.0.mlp.experts.1.gate_proj"].bits == 3.5
    assert found.groups["model.layers.0.self_attn.k_proj"].codebook == "3inst"
    assert found.groups["lm_head"].files == ("model-00001-of-00002.safetensors", "model-00002-of-00002.safetensors")
    assert found.markers == {"model.layers.0.mlp.experts.0.gate_proj.mul1": ck.MARKERS["mul1"],
                             "model.layers.0.mlp.experts.1.gate_proj.mul1": ck.MARKERS["mul1"],
                             "model.layers.1.mlp.experts.0.gate_proj.mul1": ck.MARKERS["mul1"],
                             "model.layers.0.self_attn.q_proj.mcg": ck.MARKERS["mcg"],
                             "lm_head.mul1": ck.MARKERS["mul1"]}
    assert set(found.plain) == {"model.embed_tokens.weight", "model.layers.0.input_layernorm.weight",
                                "model.layers.0.conv.bias"}
    assert found.plain["model.embed_tokens.weight"] == ("BF16", (512, 128))
    assert found.config["quantization_config"]["version"] == "1.5.0"
    assert ck.scan(tmp_path, read_markers=False).markers == {}
    assert ck.is_exl3(tmp_path)


def test_the_format_is_named_by_config_or_a_side_file(tmp_path):
    assert not ck.is_exl3(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps({"quantization": {"group_size": 64, "bits": 4}}))
    assert not ck.is_exl3(tmp_path)
    (tmp_path / "quantization_config.json").write_text(json.dumps({"quant_method": "EXL3"}))
    assert ck.is_exl3(tmp_path)


QWEN = {"quantization_config": {"quant_method": "exl3", "version": "1.4.2", "bits": 4.0, "head_bits": 6,
                                "codebook": "mul1", "mtp_bits": 4}}


def test_where_the_block_may_sit():
    assert ck.config_fields(QWEN)["codebook"] == "mul1"
    assert ck.config_fields({"text_config": QWEN})["version"] == "1.4.2"
    assert ck.config_fields({"quantization": {"quant_method": "exl3", "bits": 3}})["bits"] == 3
    assert ck.config_fields({"quantization_config": {"quant_method": "mlx", "bits": 4}}) == {}
    assert ck.config_fields({}) == {}
    assert ck.describe_config(ck.config_fields(QWEN)) == "exl3, 1.4.2, mul1, average 4.0 bits, head 6, MTP head 4"
    assert ck.describe_config({}) == "exl3"


@pytest.mark.parametrize("block", [
    QWEN["quantization_config"],
    {"quant_method": "exl3", "version": "1.5.1", "bits": 2.5078, "head_bits": 6, "codebook": "mul1"},
    {"quant_method": "exl3", "codebook": "3inst", "bits": 2.5},
    {"quant_method": "exl3"},
    {"quant_method": "exl3", "bits": 4.15, "head_bits": "8"},
])
def test_configs_that_are_read(block):
    assert ck.require_config({"quantization_config": block}, where="a model", tested="owner/tested") == block


@pytest.mark.parametrize("block,what", [
    ({"codebook": "mcg2"}, "codebook 'mcg2'"),
    ({"head_bits": 2.5}, "head_bits 2.5"),               # a head is one layer: whole bits
    ({"head_bits": 0}, "head_bits 0"),
    ({"mtp_bits": "six"}, "mtp_bits 'six'"),
    ({"bits": 9}, "average bits 9"),
])
def test_configs_that_are_refused(block, what):
    with pytest.raises(ValueError) as refused:
        ck.require_config({"quantization_config": {"quant_method": "exl3", **block}}, where="Fake Model on MI355X",
                          tested="owner/tested", help="See the runbook.")
    said = str(refused.value)
    assert "Fake Model on MI355X does not read" in said and what in said
    assert "owner/tested" in said and said.endswith("See the runbook.")
