"""From an MLX 4-bit checkpoint's tensors to what the kernels take: ``Q4`` projections, packed ``Experts``, a ``Routed``
layer.

These are the steps of the reference's weight loaders that end in ``pack`` / ``make`` — the tensor names, which
expert goes where, what is dequantized once at load time — restated over a ``get(name) -> tensor`` callable, so they
work over ``direct_read.SafeTensors.get`` and over a dict alike:
  ``linear``       src/tensorfold/families/nemotron_h/cuda/weights.py:172-178 with ``tile``,
                   src/tensorfold/families/qwen3_5/cuda/qmm_fast.py:13-17
  ``routed``       src/tensorfold/families/qwen3_5_moe/cuda/weights.py:34-49 (shared expert last, router rows in bf16)
  ``fold_shared``, ``folded``  src/tensorfold/families/nemotron_h/cuda/weights.py:151-196 (the shared expert, twice as
                   wide as a routed one, becomes experts E and E + 1)
  ``dequantize``   src/tensorfold/families/qwen3_5_moe/cuda/weights.py:21-31
The model files around them (configs, attention, state-space blocks, the layer loop) belong to the families and are
not here.
"""

from __future__ import annotations

from typing import Callable

import torch

from . import experts as grouped
from . import qmm
from .moe import Routed

Get = Callable[[str], torch.Tensor]
Triple = tuple[torch.Tensor, torch.Tensor, torch.Tensor]


def triple(get: Get, name: str) -> Triple:
    """A quantized tensor's (words as int32, scales, biases), stored as ``name.weight / .scales / .biases``."""

    words = get(name + ".weight")
    if words.dtype not in (torch.int32, torch.uint32):
        raise ValueError(f"{name}.weight holds {words.dtype}, not packed 32-bit words")
    scales, biases = get(name + ".scales"), get(name + ".biases")
    if not (scales.is_floating_point() and biases.is_floating_point()) or scales.shape != biases.shape:
        raise ValueError(f"{name}: scales and biases must be floating point and of one shape")
    return (words if words.dtype == torch.int32 else words.view(torch.int32)), scales, biases


def dequantize(words: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, gs: int = 64) -> torch.Tensor:
    """Affine words [..., K * bits / 32] with scales and biases [..., K / gs] -> fp32 [..., K]: ``s q + b``, element
    i of a word in bits [bits i, bits (i + 1)).  The width follows from the shapes (2, 4 or 8 bits)."""

    k = int(scales.shape[-1]) * gs
    bits, rest = divmod(32 * int(words.shape[-1]), k)
    if rest or bits not in (2, 4, 8):
        raise ValueError(f"words {tuple(words.shape)} with scales {tuple(scales.shape)} at groups of {gs} hold no whole width")
    w = words.view(torch.int32).to(torch.int64).bitwise_and(0xFFFFFFFF).unsqueeze(-1)
    at = torch.arange(0, 32, bits, device=words.device)
    q = w.bitwise_right_shift(at).bitwise_and((1 << bits) - 1).flatten(-2).to(torch.float32)
    spread = lambda t: t.to(torch.float32).repeat_interleave(gs, dim=-1)
    return q * spread(scales) + spread(biases)


def linear(get: Get, name: str, gs: int = 64) -> qmm.Q4:
    """The projection ``name`` packed for ``qmm.matmul`` / ``qmm.prefill_matmul`` (4-bit, groups of 32 or 64)."""

    words, scales, biases = triple(get, name)
    if 8 * words.shape[-1] != gs * scales.shape[-1]:
        raise ValueError(f"{name} is not 4-bit with groups of {gs}: words {tuple(words.shape)}, scales {tuple(scales.shape)}")
    return qmm.pack(words.contiguous(), scales.contiguous(), biases.contiguous(), gs)


def _with_last(table: Triple, extra: Triple) -> Triple:
    """Per-expert tables [E, ...] with one more expert appended."""

    return tuple(torch.cat([t, x.unsqueeze(0)]).contiguous() for t, x in zip(table, extra))


def routed(prefix: str, get: Get, top_k: int, gs: int = 64) -> Routed:
    """A Qwen-MoE layer (``prefix`` ends in "mlp."): experts ``switch_mlp.{gate,up,down}_proj`` [E, ...] with
    ``shared_expert.*`` appended as expert E; router rows ``gate`` [E, D] and ``shared_expert_gate`` [1, D]
    dequantized once and kept in bf16, the shared expert's row last."""

    rows = torch.cat([dequantize(*triple(get, prefix + "gate"), gs),
                      dequantize(*triple(get, prefix + "shared_expert_gate"), gs)])
    table = lambda proj: _with_last(triple(get, f"{prefix}switch_mlp.{proj}"), triple(get, f"{prefix}shared_expert.{proj}"))
    ex = grouped.make([table("gate_proj"), table("up_proj")], table("down_proj"), gs)
    return Routed(rows.to(torch.bfloat16).contiguous(), ex, int(top_k))


def fold_shared(fc1: Triple, fc2: Triple, up: Triple, down: Triple, width: int, gs: int = 64) -> tuple[Triple, Triple]:
    """Routed tables fc1 [E, W, D/8...] and fc2 [E, D, W/8...] with a shared expert of width 2 W (``up`` [2 W, ...],
    ``down`` [D, 2 W / 8 ...]) appended as two experts: rows [0, W) and [W, 2 W) of ``up``, and the matching halves
    of ``down``'s inputs.  Their outputs add up to the shared expert's, since relu^2 acts on each row alone."""

    if int(up[0].shape[0]) != 2 * width:
        raise ValueError(f"a shared expert of {int(up[0].shape[0])} rows does not fold into two experts of {width}")
    first = tuple(torch.cat([t, u[:width].unsqueeze(0), u[width:].unsqueeze(0)]) for t, u in zip(fc1, up))
    cut = (width // 8, width // gs, width // gs)                # where W inputs end in words, scales, biases
    second = tuple(torch.cat([t, d[:, :c].unsqueeze(0), d[:, c:].unsqueeze(0)]) for t, d, c in zip(fc2, down, cut))
    return first, second


def folded(prefix: str, get: Get, width: int, gs: int = 64) -> grouped.Experts:
    """A Nemotron-H MoE block's experts (``prefix`` ends in "mixer."): ``switch_mlp.fc1 / fc2`` and
    ``shared_experts.up_proj / down_proj`` as E + 2 relu^2 experts."""

    fc1, fc2 = fold_shared(triple(get, prefix + "switch_mlp.fc1"), triple(get, prefix + "switch_mlp.fc2"),
                           triple(get, prefix + "shared_experts.up_proj"), triple(get, prefix + "shared_experts.down_proj"),
                           width, gs)
    return grouped.make([fc1], fc2, gs)
