"""Routed EXL3 experts of any codebook, a width per expert, one grouped launch a projection; rows never depend on the
window.

Host side of ``tf_exl3x_*``; names and argument meaning follow the reference's operator module
(src/tensorfold/cuda/exl3/experts.py:33-213): ``prepare`` / ``prepare_stacked`` build a layer from per-expert
(trellis, suh, svh) triples referenced in place, ``Scratch`` holds the buffers of up to ``rows`` x ``slots`` pairs,
``routed`` runs group -> input rotation -> gate/up -> SwiGLU epilogue -> down -> output rotation (+ weighted
combine) without a host sync.  Picks outside [0, E) (a shared expert's slot) are skipped; their ``y`` rows are the
caller's.  The grouping is the 4-bit experts' pair sort (items of at most 16 pairs of one expert).
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Sequence

import torch

from .. import _lib
from .. import experts as grouped
from . import format as fmt
from .linear import CODEBOOK_IDS, _DTYPES

CB_3INST, CB_MCG, CB_MUL1 = 0, 1, 2
ACT_BF16, ACT_F32 = 0, 1          # SwiGLU with bf16 roundings after each step / in fp32
# Half-bits a value the kernels decode: every count from 2 to 16 (1 to 8 bits in half-bit steps) with every codebook,
# as the reference's module accepts them (cuda/exl3/experts.py:15-16); an odd count gives the odd stream positions
# the extra bit.
K2_SUPPORTED = {cb: tuple(range(2, 17)) for cb in (CB_3INST, CB_MCG, CB_MUL1)}
WAVES = 4                         # waves a workgroup of the grouped kernel (each takes a share of a K split)
GATE, UP, DOWN = 0, 1, 2          # rows of the per-layer address and width tables
MAX_EXPERTS = 1024                # the pair sort's table


def codebook_id(name: str) -> int:
    """'3inst' / 'mcg' / 'mul1' -> 0 / 1 / 2."""

    if name not in CODEBOOK_IDS:
        raise ValueError(f"unknown EXL3 codebook {name!r}")
    return CODEBOOK_IDS[name]


def k2_of(trellis: torch.Tensor) -> int:
    """Half-bits a value of a trellis int16 [K/16, N/16, 16 * bits]."""

    w = int(trellis.shape[-1])
    if w % 8:
        raise ValueError(f"trellis last dim {w} is not a multiple of 8")
    return w // 8


@dataclass
class Exl3RoutedExperts:
    """One layer's routed experts as the kernels read them: a table of trellis addresses and one of widths (rows
    ``GATE``, ``UP``, ``DOWN``; a column an expert) and the experts' sign-scale vectors stacked per projection."""

    ptr: torch.Tensor             # int64 [3, E] on the GPU: where each expert's gate / up / down trellis starts
    k2: torch.Tensor              # int32 [3, E] on the GPU: its half-bits a value
    suh: tuple                    # fp16 input scales: gate [E, D], up [E, D], down [E, I]
    svh: tuple                    # fp16 output scales: gate [E, I], up [E, I], down [E, D]
    count: int                    # E
    dims: int                     # D
    width: int                    # I
    cb: int
    trellis_bytes: torch.Tensor   # int64 [E] on the host: bytes of an expert's three trellises
    keep: list = field(default_factory=list, repr=False)     # whatever owns the memory ``ptr`` points into

    def nbytes_read(self, ids: Sequence[int]) -> int:
        return int(self.trellis_bytes[list(ids)].sum())


def _codebook(codebook: int | str) -> int:
    cb = codebook_id(codebook) if isinstance(codebook, str) else int(codebook)
    if cb not in K2_SUPPORTED:
        raise ValueError(f"unknown EXL3 codebook id {cb}")
    return cb


def _trellis_ok(t: torch.Tensor, k: int, n: int, cb: int) -> int:
    """Checks one expert's trellis against the layer's K x N and returns its half-bits a value."""

    if t.dtype != torch.int16 or not t.is_contiguous() or not t.is_cuda:
        raise ValueError("trellis must be a contiguous GPU int16 tensor")
    if t.dim() != 3 or 16 * t.shape[0] != k or 16 * t.shape[1] != n:
        raise ValueError(f"expert shape {tuple(t.shape)} does not match [{k // 16}, {n // 16}, *]")
    if t.data_ptr() % 4:
        raise ValueError("trellis must start on a 4-byte boundary")
    k2 = k2_of(t)
    if k2 not in K2_SUPPORTED[cb]:
        raise ValueError(f"unsupported EXL3 bit width {k2 / 2} for codebook {cb}")
    return k2


def _layer(ptr, k2, suh, svh, d: int, width: int, cb: int, keep: list, device) -> Exl3RoutedExperts:
    """The layer from host-side [3][E] lists (or tensors) of addresses and widths and the stacked scale vectors."""

    n_exp = len(ptr[0])
    if d % fmt.HAD or width % fmt.HAD:
        raise ValueError(f"D={d} and I={width} must be multiples of 128")
    if n_exp > MAX_EXPERTS:
        raise ValueError("at most 1024 experts a layer (the pair sort's table)")
    widths = torch.as_tensor(k2, dtype=torch.int32).reshape(3, n_exp)
    tile_bytes = 16 * widths.to(torch.int64).sum(0)                  # a 16 x 16 tile at k2 half-bits is 16 k2 bytes
    for name, vs, sizes in (("suh", suh, (d, d, width)), ("svh", svh, (width, width, d))):
        for v, size in zip(vs, sizes):
            if tuple(v.shape) != (n_exp, size) or v.dtype != torch.float16 or not v.is_contiguous() or not v.is_cuda:
                raise ValueError(f"{name}: contiguous GPU fp16 [{n_exp}, {size}] expected, got {tuple(v.shape)} {v.dtype}")
    return Exl3RoutedExperts(torch.as_tensor(ptr, dtype=torch.int64).reshape(3, n_exp).to(device),
                             widths.to(device), tuple(suh), tuple(svh), n_exp, d, width, cb,
                             tile_bytes * (d * width // 256), keep)


def prepare(gate: Sequence[tuple], up: Sequence[tuple], down: Sequence[tuple], codebook: int | str,
            device: str | torch.device = "cuda") -> Exl3RoutedExperts:
    """A layer from per-expert (trellis, suh, svh) triples, trellises referenced in place, each at its own width."""

    cb = _codebook(codebook)
    projections = (gate, up, down)
    n_exp = len(gate)
    if n_exp == 0 or any(len(p) != n_exp for p in projections):
        raise ValueError("gate, up and down need the same, non-zero number of experts")
    d, width = 16 * int(gate[0][0].shape[0]), 16 * int(gate[0][0].shape[1])
    shapes = ((d, width), (d, width), (width, d))
    k2 = [[_trellis_ok(m[0], k, n, cb) for m in mats] for mats, (k, n) in zip(projections, shapes)]
    ptr = [[m[0].data_ptr() for m in mats] for mats in projections]

    def rows(mats, which: int) -> torch.Tensor:
        return torch.stack([m[which].reshape(-1) for m in mats]).to(device=device, dtype=torch.float16).contiguous()

    return _layer(ptr, k2, [rows(m, 1) for m in projections], [rows(m, 2) for m in projections], d, width, cb,
                  [m[0] for mats in projections for m in mats], device)


def prepare_stacked(gt: torch.Tensor, ut: torch.Tensor, dt: torch.Tensor, suh_g, suh_u, svh_g, svh_u, suh_d, svh_d,
                    codebook: int | str) -> Exl3RoutedExperts:
    """A uniform-width layer stacked per projection: trellis [E, K/16, N/16, 16 * bits] (int16, or the same bytes as
    int32 words), suh/svh [E, n].  Nothing is copied: expert e's trellis is the stack's base plus e strides."""

    cb = _codebook(codebook)
    stacks = [t.view(torch.int16) if t.dtype == torch.int32 else t for t in (gt, ut, dt)]
    n_exp = int(stacks[0].shape[0])
    if n_exp == 0 or any(t.dim() != 4 or t.shape[0] != n_exp for t in stacks):
        raise ValueError("gate, up and down need the same, non-zero number of experts")
    d, width = 16 * int(stacks[0].shape[1]), 16 * int(stacks[0].shape[2])
    ptr, k2 = [], []
    for t, (k, n) in zip(stacks, ((d, width), (d, width), (width, d))):
        k2.append([_trellis_ok(t[0], k, n, cb)] * n_exp)
        if not t.is_contiguous() or (t[0].numel() * 2) % 4:
            raise ValueError("stacked trellises must be contiguous, every expert on a 4-byte boundary")
        ptr.append((t.data_ptr() + torch.arange(n_exp, dtype=torch.int64) * (t[0].numel() * 2)).tolist())
    half = lambda v: v.to(device=gt.device, dtype=torch.float16).contiguous()
    return _layer(ptr, k2, [half(suh_g), half(suh_u), half(suh_d)], [half(svh_g), half(svh_u), half(svh_d)], d, width,
                  cb, stacks, gt.device)


def default_config(k: int, n: int, gateup: bool = True) -> int:
    """K splits of a K -> N projection: the shape's alone, so a row's sums run in one order at every row count.
    As many as keep four tile pairs a wave and at most 128 (column block, split) workgroups an item."""

    pairs, nb = k // 32, n // 128
    for sk in (8, 4, 2):
        if pairs // (WAVES * sk) >= 4 and nb * sk <= 128:
            return sk
    if pairs < WAVES:
        raise ValueError(f"K={k} is too short for {WAVES} waves")
    return 1


class Scratch:
    """Device buffers of ``routed`` for up to ``rows`` rows of ``slots`` slots: the rotated inputs of the three
    projections (``xg``, ``xu``, ``xd``, fp16 a pair), the K splits' fp32 partial sums ``z``, the pair outputs ``y``
    and the pair sort's plan.  Pairs whose pick is not a routed expert touch none of them (their ``y`` rows stay as
    the caller left them)."""

    def __init__(self, ex: Exl3RoutedExperts, rows: int, slots: int, sk_gu: int | None = None, sk_d: int | None = None,
                 device: str | torch.device = "cuda") -> None:
        self.rows, self.slots, self.count_experts = rows, slots, ex.count
        self.sk_gu = sk_gu or default_config(ex.dims, ex.width, True)
        self.sk_d = sk_d or default_config(ex.width, ex.dims, False)
        pairs = rows * slots

        def buffer(columns: int, dtype: torch.dtype) -> torch.Tensor:
            return torch.zeros((pairs, columns), dtype=dtype, device=device)

        self.xg, self.xu = buffer(ex.dims, torch.float16), buffer(ex.dims, torch.float16)
        self.xd = buffer(ex.width, torch.float16)
        self.y = buffer(ex.dims, torch.float32)
        # one buffer serves both grouped launches: [2 matrices][sk_gu][pairs][I] first, [sk_d][pairs][D] after
        self.z = torch.zeros((pairs * max(2 * self.sk_gu * ex.width, self.sk_d * ex.dims),), dtype=torch.float32,
                             device=device)
        self.plan = grouped.Plan(rows, slots, ex.count, device)          # ids outside [0, E) join no item


def routed(x: torch.Tensor, pick: torch.Tensor, wts: torch.Tensor | None, ex: Exl3RoutedExperts, s: Scratch,
           out: torch.Tensor | None, R: int, limit: float = math.inf, act_mode: int = ACT_F32,
           group: bool = True) -> torch.Tensor:
    """Routed experts of R rows (picks outside [0, E) skipped): Y fp32 per pair, or ``out`` fp32 [R, D] = the
    wts-weighted sum over the slots when ``wts`` is given; no host sync.  ``group=False`` reuses the grouping of the
    last call on the same picks.  Five launches up to 1,024 pairs (the grouping shares the rotation's), else six."""

    d, width, n_exp, slots = ex.dims, ex.width, ex.count, s.slots
    p = R * slots
    if R < 1 or R > s.rows:
        raise ValueError(f"{R} rows but the scratch holds {s.rows}")
    if x.dim() != 2 or x.shape[0] < R or x.shape[1] != d or x.dtype not in _DTYPES or x.stride(1) != 1:
        raise ValueError(f"x must be [>= {R}, {d}] fp16, bf16 or fp32 with unit column stride")
    if x.stride(0) % 2 or x.data_ptr() % 8:
        raise ValueError("x rows must be an even stride apart and 8-byte aligned")
    if pick.dtype != torch.int32 or tuple(pick.shape) != (R, slots) or not pick.is_contiguous():
        raise ValueError(f"pick must be a contiguous int32 [{R}, {slots}]")
    if wts is not None and (wts.dtype != torch.float32 or tuple(wts.shape) != (R, slots) or not wts.is_contiguous()):
        raise ValueError(f"wts must be a contiguous fp32 [{R}, {slots}]")
    if act_mode not in (ACT_BF16, ACT_F32):
        raise ValueError("act_mode is ACT_BF16 or ACT_F32")
    _lib.on_gpu(x, pick, wts)
    plan = s.plan
    items = grouped.max_items(p, n_exp, grouped.TILE)
    plan_args = (_lib.ptr(plan.items), _lib.ptr(plan.counts), _lib.ptr(plan.members))
    rot_args = (_lib.ptr(x), _DTYPES[x.dtype], x.stride(0), _lib.ptr(pick), _lib.ptr(ex.suh[GATE]), _lib.ptr(ex.suh[UP]),
                _lib.ptr(s.xg), _lib.ptr(s.xu), R, slots, d, n_exp)
    if group and p <= grouped.SMALL:
        # one launch for the pair sort (it drops ids outside [0, E)) and the rotation: neither needs the other
        plan.tile = grouped.TILE
        _lib.call("tf_exl3x_plan_rot_in", *rot_args, grouped.TILE, _lib.ptr(plan.members), _lib.ptr(plan.items),
                  _lib.ptr(plan.counts))
    else:
        if group:
            grouped.route(pick, plan)
        _lib.call("tf_exl3x_rot_in", *rot_args)
    _lib.call("tf_exl3x_grouped", _lib.ptr(s.xg), _lib.ptr(s.xu), _lib.ptr(ex.ptr[GATE]), _lib.ptr(ex.ptr[UP]),
              _lib.ptr(ex.k2[GATE]), _lib.ptr(ex.k2[UP]), *plan_args, _lib.ptr(s.z), 2, d, width, p, s.sk_gu, ex.cb,
              n_exp, items)
    _lib.call("tf_exl3x_gateup_epilogue", _lib.ptr(s.z), _lib.ptr(pick), _lib.ptr(ex.svh[GATE]), _lib.ptr(ex.svh[UP]),
              _lib.ptr(ex.suh[DOWN]), _lib.ptr(s.xd), p, width, s.sk_gu, n_exp,
              float(min(limit, 3.0e38)), act_mode)
    _lib.call("tf_exl3x_grouped", _lib.ptr(s.xd), None, _lib.ptr(ex.ptr[DOWN]), None, _lib.ptr(ex.k2[DOWN]), None,
              *plan_args, _lib.ptr(s.z), 1, width, d, p, s.sk_d, ex.cb, n_exp, items)
    if wts is None:
        _lib.call("tf_exl3x_down_combine", _lib.ptr(s.z), _lib.ptr(pick), _lib.ptr(ex.svh[DOWN]), _lib.ptr(s.y), None, None,
                  R, slots, d, s.sk_d, n_exp)
        return s.y[:p]
    if out is None:
        out = torch.empty((R, d), dtype=torch.float32, device=x.device)
    elif out.dtype != torch.float32 or tuple(out.shape) != (R, d) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous fp32 [{R}, {d}]")
    _lib.call("tf_exl3x_down_combine", _lib.ptr(s.z), _lib.ptr(pick), _lib.ptr(ex.svh[DOWN]), _lib.ptr(s.y), _lib.ptr(wts),
              _lib.ptr(out), R, slots, d, s.sk_d, n_exp)
    return out


def dequant(trellis: torch.Tensor, codebook: int | str) -> torch.Tensor:
    """W_q [K, N] fp16 of one matrix through the kernels' own lane decode; for tests."""

    cb = codebook_id(codebook) if isinstance(codebook, str) else int(codebook)
    k2 = k2_of(trellis)
    if k2 not in K2_SUPPORTED.get(cb, ()):
        raise ValueError(f"unsupported EXL3 bit width {k2 / 2} for codebook {cb}")
    k, n = int(trellis.shape[0]) * 16, int(trellis.shape[1]) * 16
    words = trellis.contiguous().view(torch.int32)
    out = torch.empty((k, n), dtype=torch.float16, device=trellis.device)
    tile = 4 * k2
    _lib.call("tf_exl3_unpack", _lib.ptr(words), _lib.ptr(out), k, n, (n // 16) * tile, 8 * tile, k2, cb)
    return out
