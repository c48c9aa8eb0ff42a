"""Routed-expert matmuls over 4-bit affine tables (MI355X).

Host side of ``tf_experts_*`` in ``include/tfmi.h``.  The function names, argument order and error behaviour follow
the operator interface the reference's engines call (reference: src/tensorfold/cuda/experts.py:28-150), so an
engine can swap the import; everything below the signatures is this package's own.

Contract kept from the reference: the bits computed for a (row, slot) pair are a function of that row and that
expert only - not of the other rows in the call, of the item the pair lands in, or of the row count.
"""

from __future__ import annotations

import dataclasses

import torch

from . import _lib

COLS = 32             # columns of one weight block
TILE = 16             # largest decode item, in pairs
PREFILL_TILE = 128    # default prompt item; the MFMA kernels also take 16 and 64
SMALL = 1024          # a plan up to this many pairs is sorted by one workgroup
_GROUPS = (32, 64)
ARITH_F16, ARITH_BF16 = 0, 1      # TF_ARITH_* of the C header: the prompt form's operand arithmetic
F16_TABLE_LIMIT = 255.9           # the fp16 form holds 256 w, so |w| below this stays finite in fp16


def fits_f16(*tensors: torch.Tensor) -> bool:
    """Whether the tables given as (scales, biases, scales, biases, ...) fit the prompt form's fp16 arithmetic, which
    holds fp16(fma(q, 256 s, 256 b)) for every code q of 0..15: every scale finite and below the limit, and both ends
    of every group's range of weights, b and 15 s + b, below it too (a few reductions and a host read: for load
    time)."""

    if len(tensors) % 2:
        raise ValueError("fits_f16 takes scales and biases in pairs")
    for s, b in zip(tensors[::2], tensors[1::2]):
        if not s.numel():
            continue
        s, b = s.float(), b.float()
        top = 15.0 * s + b
        if not bool(torch.isfinite(top).all()):
            return False
        if max(float(s.abs().max()), float(b.abs().max()), float(top.abs().max())) >= F16_TABLE_LIMIT:
            return False
    return True


def block_words(gs: int) -> int:
    """Size in int32 of the block covering 32 columns and one group: gs/8 code words a column plus one
    (scale | bias << 16) word a column."""

    return COLS * gs // 8 + COLS


def _group_ok(gs: int) -> None:
    if gs not in _GROUPS:
        raise ValueError(f"groups of 32 or 64 inputs, not {gs}")


def pack(words: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, gs: int) -> torch.Tensor:
    """Stored MLX tensors of E experts -> kernel blocks.

    words int32/uint32 [E, N, K/8]; scales, biases bf16 [E, N, K/gs]  ->  int32 [E, N/32, K/gs, block_words(gs)].
    ``unpack`` is the exact inverse."""

    _group_ok(gs)
    e, n, k8 = words.shape
    k = 8 * k8
    want = (e, n, k // gs)
    if n % COLS or k % gs or tuple(scales.shape) != want or tuple(biases.shape) != want:
        raise ValueError(f"experts: shape {tuple(words.shape)} with scales {tuple(scales.shape)} does not pack")
    _lib.on_gpu(words, scales, biases)
    blocks = words.new_empty((e, n // COLS, k // gs, block_words(gs)), dtype=torch.int32)
    # converted or re-laid copies are held by name until the launch is queued: a temporary freed between two
    # arguments would hand its memory to the next one
    words, scales, biases = words.contiguous(), scales.to(torch.bfloat16).contiguous(), biases.to(torch.bfloat16).contiguous()
    _lib.call("tf_experts_pack", _lib.ptr(words), _lib.ptr(scales), _lib.ptr(biases), e, n, k, gs, _lib.ptr(blocks))
    return blocks


def unpack(blocks: torch.Tensor, gs: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Kernel blocks [E, N/32, K/gs, block] -> (words [E, N, K/8], scales, biases [E, N, K/gs]).

    ``blocks`` may be a view selecting one matrix of a stacked table (``table[:, :, :, m]``); it is copied only if
    its strides are not those of such a view."""

    _group_ok(gs)
    e, nb, kg, bw = blocks.shape
    if bw != block_words(gs):
        raise ValueError(f"experts: blocks of {bw} words are not groups of {gs}")
    s0, s1, s2, s3 = blocks.stride()
    if not (s3 == 1 and s1 == kg * s2 and s0 == nb * s1):
        blocks = blocks.contiguous()
        s2 = blocks.stride(2)
    n, k = nb * COLS, kg * gs
    words = blocks.new_empty((e, n, k // 8), dtype=torch.int32)
    scales = blocks.new_empty((e, n, kg), dtype=torch.bfloat16)
    biases = torch.empty_like(scales)
    _lib.call("tf_experts_unpack", _lib.ptr(blocks), s2, e, n, k, gs, _lib.ptr(words), _lib.ptr(scales),
              _lib.ptr(biases))
    return words, scales, biases


@dataclasses.dataclass
class Experts:
    """The packed experts of one layer.

    up   int32 [E, NI/32, D/gs, M, block]  M = 2: gate then up (SwiGLU); M = 1: up alone (relu^2)
    down int32 [E, D/32, NI/gs, 1, block]
    """

    up: torch.Tensor
    down: torch.Tensor
    gs: int
    width: int           # NI
    dims: int            # D
    limit: float = 0.0   # SwiGLU clip, 0 for none
    arith: int = ARITH_F16   # the prompt form's arithmetic: ARITH_BF16 when a scale or bias does not fit the fp16 form

    @property
    def count(self) -> int:
        return int(self.up.shape[0])

    @property
    def swiglu(self) -> bool:
        return int(self.up.shape[3]) == 2

    def bytes_per_expert(self) -> int:
        return 4 * (self.up[0].numel() + self.down[0].numel())


def make(up: list[tuple], down: tuple, gs: int, *, limit: float = 0.0, arith: int | None = None) -> Experts:
    """Pack a layer.  ``up`` = [(words, scales, biases)] for relu^2 or [gate, up] for SwiGLU; ``down`` one triple.

    ``arith`` fixes the prompt form's arithmetic.  Left None, a gated (SwiGLU) layer takes the fp16 form unless a
    group of one of its tables holds a weight too large for it (``fits_f16``); then, and for every relu^2 layer, it
    is the reference's bf16 form.  The fp16 form clamps activations (and ``moe.run`` a prompt's pair outputs) beyond
    +-65504, and a relu^2 activation passes that as soon as an up output passes 256, which no look at the tables
    rules out; a caller who knows the activations of such a layer stay below may ask for ``arith=ARITH_F16``."""

    if len(up) not in (1, 2):
        raise ValueError("experts take a gate and an up projection, or an up projection alone")
    ni, d = int(up[0][0].shape[1]), 8 * int(up[0][0].shape[2])
    table_up = torch.stack([pack(w, s, b, gs) for (w, s, b) in up], dim=3)
    table_down = pack(*down, gs).unsqueeze(3)
    if arith is None:
        small = len(up) == 2 and fits_f16(*[t for m in (*up, down) for t in m[1:]])
        arith = ARITH_F16 if small else ARITH_BF16
    return Experts(table_up, table_down, gs, ni, d, float(limit), int(arith))


def max_items(pairs: int, experts: int, tile: int = TILE) -> int:
    """Upper bound on the items of any plan over ``pairs`` pairs: each used expert opens one item and every full
    ``tile`` pairs can open one more, and no item is empty.  Grids are sized with it (a launch's surplus workgroups
    still route before they find they have no item); the live count stays on the device."""

    return min(pairs, min(pairs, experts) + pairs // tile)


class Plan:
    """Device scratch of the pair sort: ``members`` (pairs ordered by expert), ``items`` rows of
    (expert, first member, count) and ``counts`` = (items, distinct experts, the prompt kernels' ticket word, spare).
    The ticket word hands an item's units to the prompt kernels' workgroups; it is zero whenever no prompt launch on
    this plan is running, so launches that share a plan must not overlap.  Sized once for ``rows`` x ``slots``."""

    def __init__(self, rows: int, slots: int, experts: int, device: torch.device | str, *,
                 prefill: bool = False) -> None:
        self.rows, self.slots, self.experts, self.prefill = rows, slots, experts, prefill
        self.tile = PREFILL_TILE if prefill else TILE
        pairs = rows * slots

        def ints(*shape: int) -> torch.Tensor:
            return torch.zeros(shape, dtype=torch.int32, device=device)

        self.members = ints(pairs)
        self.items = ints(max_items(pairs, experts, TILE), 3)     # sized for the narrowest item any consumer takes
        self.counts = ints(4)
        blocks = -(-pairs // SMALL)
        self.rank = ints(pairs if pairs > SMALL else 1)            # the multi-workgroup sort's scratch
        self.hist = ints(blocks * experts if pairs > SMALL else 1)


def route(picks: torch.Tensor, plan: Plan, tile: int = PREFILL_TILE) -> None:
    """Sort the pairs of ``picks`` (int32 [R, slots], contiguous) into ``plan``.  ``tile`` is honoured by prompt
    plans only; decode plans always use items of 16."""

    rows, slots = picks.shape
    if slots != plan.slots or rows > plan.rows:
        raise ValueError(f"picks {tuple(picks.shape)} do not fit a plan of {plan.rows} x {plan.slots}")
    if picks.dtype != torch.int32 or not picks.is_contiguous():
        raise ValueError("picks: contiguous int32, one id a pair")
    _lib.on_gpu(picks)
    plan.tile = tile if plan.prefill else TILE
    _lib.call("tf_experts_plan", _lib.ptr(picks), rows * slots, plan.experts, plan.tile, _lib.ptr(plan.members),
              _lib.ptr(plan.items), _lib.ptr(plan.counts), _lib.ptr(plan.rank), _lib.ptr(plan.hist))


def _check(x: torch.Tensor, k: int, out: torch.Tensor, n: int, epi: int) -> None:
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.stride(1) != 1 or x.stride(0) % 8 or x.shape[1] != k:
        raise RuntimeError("x: rows of K = groups * group size inputs, 16-byte aligned")
    if not out.is_contiguous() or out.dim() != 2 or out.shape[1] != n:
        raise RuntimeError("out: contiguous rows of n columns")
    if out.dtype != {0: torch.float32, 4: torch.float16}.get(epi, torch.bfloat16):
        raise RuntimeError("out has the wrong dtype")
    _lib.on_gpu(x, out)


def _fits(plan: Plan, rows: int, x_rows: int | None, pair_rows: int) -> None:
    """The kernels index token rows below ``rows`` and pair rows below ``rows * slots``: the buffers must hold them."""

    if not 1 <= rows <= plan.rows:
        raise ValueError(f"rows = {rows} does not fit a plan made for {plan.rows}")
    if (x_rows is not None and x_rows < rows) or pair_rows < rows * plan.slots:
        raise ValueError(f"buffers too small for {rows} rows x {plan.slots} slots")


def _launch(x: torch.Tensor, slots: int, table: torch.Tensor, gs: int, k: int, n: int, epi: int, plan: Plan,
            out: torch.Tensor, limit: float, rows: int, arith: int = ARITH_F16) -> None:
    bound = max_items(rows * plan.slots, plan.experts, plan.tile)
    common = (gs, epi, _lib.ptr(x), x.stride(0), slots, _lib.ptr(table), k // gs, n // COLS, _lib.ptr(plan.items),
              _lib.ptr(plan.counts), _lib.ptr(plan.members), _lib.ptr(out), n, limit)
    if plan.prefill:
        _lib.call("tf_experts_prefill", *common, bound, plan.tile, arith)
    else:
        _lib.call("tf_experts_run", *common, bound * (n // COLS))


def gate_up(x: torch.Tensor, ex: Experts, plan: Plan, out: torch.Tensor, rows: int) -> None:
    """Token rows x bf16 [R, D] -> the activation of every pair, out bf16 [R * slots, NI]."""

    epi = 2 if ex.swiglu else 1
    _check(x, ex.dims, out, ex.width, epi)
    _fits(plan, rows, x.shape[0], out.shape[0])
    _launch(x, plan.slots, ex.up, ex.gs, ex.dims, ex.width, epi, plan, out, ex.limit, rows, ex.arith)


def down(act: torch.Tensor, ex: Experts, plan: Plan, out: torch.Tensor, rows: int) -> None:
    """Pair activations bf16 [R * slots, NI] -> every pair's output [R * slots, D]: fp32; a prompt plan also takes a
    bf16 ``out`` (the reference's choice, cuda/moe.py:99: half the bytes, a rounding of 2^-9) or an fp16 one (half the
    bytes, a rounding of 2^-12; a value beyond +-65504 is stored as +-65504)."""

    epi = 0
    if plan.prefill and out.dtype in (torch.bfloat16, torch.float16):
        epi = 3 if out.dtype == torch.bfloat16 else 4
    _check(act, ex.width, out, ex.dims, epi)
    _fits(plan, rows, None, min(act.shape[0], out.shape[0]))
    _launch(act, 0, ex.down, ex.gs, ex.width, ex.dims, epi, plan, out, 0.0, rows, ex.arith)
