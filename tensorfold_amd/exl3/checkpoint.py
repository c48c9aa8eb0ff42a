"""EXL3 checkpoints on disk: which tensors of a folder form trellis layers, what config.json says of them, and the
layers themselves on the GPU.

The names follow the reference's header-only metadata (src/tensorfold/cuda/exl3/format.py:186-386: ``Exl3Tensor``,
``read_header``, ``read_scalar``, ``parse_group``, ``Checkpoint``, ``config_fields``, ``require_config``,
``describe_config``, ``scan``, ``is_exl3``) and its group reader (src/tensorfold/families/qwen3_5/cuda/exl3_load.py:73-89).
A layer is a group of tensors sharing a prefix: ``.trellis`` int16 [K/16, N/16, 16 bits], input scales ``.suh`` fp16
[K] (or ``.su``: one sign bit an input, int16 [K/16]), output scales ``.svh`` fp16 [N] (or ``.sv``), at most one
codebook marker (``.mcg`` or ``.mul1``, a scalar int32; none means 3inst) and an optional ``.bias``.  Everything but
``load_groups`` reads safetensors headers only.
"""

from __future__ import annotations

import dataclasses
import json
import pathlib
import struct
from typing import Any, Iterable

from . import format as fmt

MARKERS = {"mcg": 0xCBAC1FED, "mul1": 0x83DCD12D}       # what a marker tensor holds (its int32's bit pattern)
PARTS = ("trellis", "suh", "su", "svh", "sv", "mcg", "mul1", "bias")
SIDECAR = "quantization_config.json"
_BLOCK_KEYS = ("quantization_config", "quantization")
# side -> the two ways its scales are stored: (part, safetensors dtype, elements a stored value covers)
_SCALES = {"input": (("suh", "F16", 1), ("su", "I16", 16)), "output": (("svh", "F16", 1), ("sv", "I16", 16))}


@dataclasses.dataclass(frozen=True)
class Exl3Tensor:
    """One layer as its headers describe it."""

    prefix: str               # "model.layers.0.self_attn.q_proj"
    bits: float
    codebook: str
    k: int
    n: int
    in_scales: str            # the part that holds them: "suh" or "su"
    out_scales: str           # "svh" or "sv"
    bias: bool
    files: tuple[str, ...]    # names of the files its parts sit in

    @property
    def trellis_bytes(self) -> int:
        return self.k * self.n * int(2 * self.bits) // 16

    def describe(self) -> str:
        return f"{self.prefix}: EXL3 {self.bits:g}-bit {self.codebook}, K={self.k} N={self.n}"


@dataclasses.dataclass
class Checkpoint:
    """A folder's tensors sorted three ways."""

    groups: dict[str, Exl3Tensor]                      # readable layers by prefix
    plain: dict[str, tuple[str, tuple[int, ...]]]      # every other tensor: name -> (dtype, shape)
    bad: dict[str, str]                                # prefix of a group with a trellis that does not parse -> why
    config: dict[str, Any]                             # config.json, {} without one
    markers: dict[str, int]                            # marker tensor -> the value read from it


def read_header(path) -> dict[str, dict]:
    """name -> {"dtype", "shape", "data_offsets"} of a safetensors file, without its ``__metadata__``."""

    with open(path, "rb") as f:
        (length,) = struct.unpack("<Q", f.read(8))
        entries = json.loads(f.read(length))
    return {name: e for name, e in entries.items() if name != "__metadata__"}


def read_scalar(path, entry: dict) -> int:
    """The unsigned 32-bit value of a scalar tensor, given its header entry."""

    with open(path, "rb") as f:
        (length,) = struct.unpack("<Q", f.read(8))
        f.seek(8 + length + int(entry["data_offsets"][0]))
        return struct.unpack("<I", f.read(4))[0]


def parse_group(prefix: str, parts: dict[str, dict], files: Iterable[str] = ()) -> Exl3Tensor:
    """The layer a group's header entries describe.  ValueError ("<prefix>: <why>") for a group that is not one."""

    def check(ok: bool, why: str) -> None:
        if not ok:
            raise ValueError(f"{prefix}: {why}")

    check("trellis" in parts, "no .trellis")
    dtype, shape = parts["trellis"]["dtype"], [int(v) for v in parts["trellis"]["shape"]]
    check(dtype == "I16" and len(shape) == 3, f"trellis must be int16 [K/16, N/16, 16 * bits], got {dtype} {shape}")
    try:
        bits = fmt.bits_of(shape)
    except ValueError as e:
        raise ValueError(f"{prefix}: {e}") from None
    marked = [name for name in MARKERS if name in parts]
    check(len(marked) < 2, "both mcg and mul1 markers")
    codebook = marked[0] if marked else "3inst"
    check(float(bits).is_integer() or codebook == "mul1", f"{bits}-bit tiles need the mul1 codebook, found {codebook}")
    sizes = {"input": 16 * shape[0], "output": 16 * shape[1]}
    chosen = {}
    for side, ways in _SCALES.items():
        found = [way for way in ways if way[0] in parts]
        check(bool(found), f"no {side} scales (.{ways[0][0]} or .{ways[1][0]})")
        part, want_dtype, covers = found[0]
        want = [sizes[side] // covers]
        got = (parts[part]["dtype"], [int(v) for v in parts[part]["shape"]])
        check(got == (want_dtype, want), f".{part} must be {want_dtype} {want}, got {got[0]} {got[1]}")
        chosen[side] = part
    k, n = sizes["input"], sizes["output"]
    check(k % fmt.HAD == 0 and n % fmt.HAD == 0, f"K={k} and N={n} must be multiples of {fmt.HAD} (the Hadamard blocks)")
    return Exl3Tensor(prefix, bits, codebook, k, n, chosen["input"], chosen["output"], "bias" in parts,
                      tuple(sorted(set(files))))


def config_fields(config: dict[str, Any]) -> dict[str, Any]:
    """The EXL3 block of a config.json (``quantization_config`` or ``quantization``, at the top or under
    ``text_config``): version, average bits, head_bits, codebook ...; {} when there is none."""

    for holder in (config, config.get("text_config") or {}):
        for key in _BLOCK_KEYS:
            block = holder.get(key)
            if isinstance(block, dict) and str(block.get("quant_method", "")).lower() == "exl3":
                return dict(block)
    return {}


def describe_config(fields: dict[str, Any]) -> str:
    """The fields that are there, for a message: ``exl3, 1.4.2, mul1, average 4.0 bits, head 6``."""

    said = ["exl3"] + [str(fields[key]) for key in ("version", "codebook") if fields.get(key)]
    for key, label in (("bits", "average {} bits"), ("head_bits", "head {}"), ("mtp_bits", "MTP head {}")):
        if fields.get(key) is not None:
            said.append(label.format(fields[key]))
    return ", ".join(said)


def require_config(config: dict[str, Any], *, where: str = "", tested: str = "", help: str = "") -> dict[str, Any]:
    """Refuse, from config.json alone, a codebook or width the kernels do not read; the fields read otherwise."""

    fields = config_fields(config)

    def number(key: str) -> float | None:
        if fields.get(key) is None:
            return None
        try:
            return float(fields[key])
        except (TypeError, ValueError):
            return float("nan")

    reasons = []
    codebook = fields.get("codebook")
    if codebook is not None and str(codebook).lower() not in fmt.CODEBOOKS:
        reasons.append(f"codebook {codebook!r}")
    for key in ("head_bits", "mtp_bits"):              # one layer's width: whole bits only
        value = number(key)
        if value is not None and not (value in fmt.BITS and value.is_integer()):
            reasons.append(f"{key} {fields[key]!r}")
    average = number("bits")                           # the model's average: any fraction between 1 and 8
    if average is not None and not 1 <= average <= 8:
        reasons.append(f"average bits {fields['bits']!r}")
    if reasons:
        tail = f" Tested checkpoints: {tested}." if tested else ""
        tail += f" {help}" if help else ""
        raise ValueError(f"the EXL3 module of {where or 'this engine'} does not read this checkpoint's weights "
                         f"({reasons[0]}; {describe_config(fields)}). It reads the {', '.join(fmt.CODEBOOKS)} "
                         f"codebooks at {', '.join(str(v) for v in fmt.BITS)} bits a weight (half bits with "
                         f"mul1 only).{tail}")
    return fields


def scan(model_dir, read_markers: bool = True) -> Checkpoint:
    """The headers of every ``*.safetensors`` in ``model_dir`` as a ``Checkpoint``; no weight is read."""

    root = pathlib.Path(model_dir)
    entry_of: dict[str, tuple[str, dict]] = {}
    for path in sorted(root.glob("*.safetensors")):
        for name, entry in read_header(path).items():
            entry_of[name] = (path.name, entry)
    gathered: dict[str, dict[str, str]] = {}           # prefix -> part -> tensor name
    for name in entry_of:
        prefix, _, part = name.rpartition(".")
        if part in PARTS:
            gathered.setdefault(prefix, {})[part] = name
    ck = Checkpoint({}, {}, {}, {}, {})
    grouped = set()
    for prefix, names in gathered.items():
        if "trellis" not in names:
            continue                                   # a plain layer's .bias and the like
        grouped.update(names.values())
        try:
            layer = parse_group(prefix, {part: entry_of[name][1] for part, name in names.items()},
                                [entry_of[name][0] for name in names.values()])
        except ValueError as e:
            ck.bad[prefix] = str(e)[len(prefix) + 2:]
            continue
        ck.groups[prefix] = layer
        if read_markers and layer.codebook in MARKERS:
            file, entry = entry_of[names[layer.codebook]]
            ck.markers[names[layer.codebook]] = read_scalar(root / file, entry)
    ck.plain = {name: (entry["dtype"], tuple(entry["shape"])) for name, (_, entry) in entry_of.items()
                if name not in grouped}
    if (root / "config.json").is_file():
        ck.config = json.loads((root / "config.json").read_text())
    return ck


def is_exl3(model_dir) -> bool:
    """Whether config.json, or the side file some packs carry instead, names the format."""

    root = pathlib.Path(model_dir)
    if (root / "config.json").is_file() and config_fields(json.loads((root / "config.json").read_text())):
        return True
    side = root / SIDECAR
    return side.is_file() and str(json.loads(side.read_text()).get("quant_method", "")).lower() == "exl3"


def load_groups(files, groups: dict[str, Exl3Tensor], device="cuda", plans: dict | None = None) -> dict:
    """``Exl3Linear`` layers on ``device`` for ``groups``, their parts read through ``files`` (a
    ``direct_read.SafeTensors`` over the folder).  ``plans`` maps (bits, K, N) to a (K splits, waves) pair for shapes
    that should not take ``linear.plan``'s choice.  A marker whose value is not its codebook's is refused."""

    import torch

    from .linear import Exl3Linear

    layers = {}
    for prefix in sorted(groups):
        meta = groups[prefix]
        if meta.codebook in MARKERS:
            path, first = files.where[f"{prefix}.{meta.codebook}"][:2]
            value = int(files.reader.read(path, first, 4).view(torch.int32)[0]) & 0xFFFFFFFF
            if value != MARKERS[meta.codebook]:
                raise ValueError(f"{prefix}.{meta.codebook} holds {value:#x}, not the {meta.codebook} codebook's "
                                 f"{MARKERS[meta.codebook]:#x}")
        part = lambda name: files.get(f"{prefix}.{name}", device)
        layer = Exl3Linear.from_tensors(part("trellis"), part(meta.in_scales), part(meta.out_scales), meta.codebook,
                                        part("bias") if meta.bias else None, device=device)
        if plans and (layer.bits, layer.k, layer.n) in plans:
            layer.split = plans[(layer.bits, layer.k, layer.n)]
        layers[prefix] = layer
    return layers
