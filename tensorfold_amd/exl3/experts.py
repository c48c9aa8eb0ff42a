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
# Half-bits a value the kernels decode: 1..8 bits with every codebook, 1.5, 2.5, 3.5 with mul1
K2_SUPPORTED = {CB_3INST: (2, 4, 6, 8, 10, 12, 14, 16), CB_MCG: (2, 4, 6, 8, 10, 12, 14, 16),
                CB_MUL1: (2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16)}
WAVES = 4                         # waves a workgroup of the grouped kernel (each takes a share of a K split)


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
    """One layer's routed experts: trellis addresses and widths per projection, stacked suh/svh, and the tensors that
    keep the trellises alive."""

    gate_ptr: torch.Tensor    # int64 [E]
    up_ptr: torch.Tensor
    down_ptr: torch.Tensor
    gate_k2: torch.Tensor     # int32 [E], half-bits a value
    up_k2: torch.Tensor
    down_k2: torch.Tensor
    suh_g: torch.Tensor       # fp16 [E, D]
    suh_u: torch.Tensor
    svh_g: torch.Tensor       # fp16 [E, I]
    svh_u: torch.Tensor
    suh_d: torch.Tensor       # fp16 [E, I]
    svh_d: torch.Tensor       # fp16 [E, D]
    count: int                # E
    dims: int                 # D
    width: int                # I
    cb: int
    trellis_bytes: torch.Tensor   # int64 [E] (host): gate + up + down trellis bytes of each expert
    keep: list = field(default_factory=list, repr=False)

    def nbytes_read(self, ids: Sequence[int]) -> int:
        return int(self.trellis_bytes[list(ids)].sum())


def prepare(gate: Sequence[tuple], up: Sequence[tuple], down: Sequence[tuple], codebook: int | str,
            device: str | torch.device = "cuda") -> Exl3RoutedExperts:
    """A layer from per-expert (trellis, suh, svh) triples, trellises referenced in place, each at its own width."""

    cb = codebook_id(codebook) if isinstance(codebook, str) else int(codebook)
    if cb not in K2_SUPPORTED:
        raise ValueError(f"unknown EXL3 codebook id {cb}")
    n_exp = len(gate)
    if not (len(up) == len(down) == n_exp) or n_exp == 0:
        raise ValueError("gate, up and down need the same, non-zero number of experts")
    d, width = int(gate[0][0].shape[0]) * 16, int(gate[0][0].shape[1]) * 16
    if d % fmt.HAD or width % fmt.HAD:
        raise ValueError(f"D={d} and I={width} must be multiples of 128")
    if n_exp > 1024:
        raise ValueError("at most 1024 experts a layer (the pair sort's table)")
    keep: list = []

    def table(mats, k, n):
        ptrs, k2s = [], []
        for t, _, _ in mats:
            if t.dtype != torch.int16 or not t.is_contiguous() or not t.is_cuda:
                raise ValueError("trellis must be a contiguous GPU int16 tensor")
            if t.shape[0] * 16 != k or t.shape[1] * 16 != n:
                raise ValueError(f"expert shape {tuple(t.shape)} does not match [{k // 16}, {n // 16}, *]")
            k2 = k2_of(t)
            if k2 not in K2_SUPPORTED[cb]:
                raise ValueError(f"unsupported EXL3 bit width {k2 / 2} for codebook {cb}")
            if t.data_ptr() % 4:
                raise ValueError("trellis must start on a 4-byte boundary")
            k2s.append(k2)
            ptrs.append(t.data_ptr())
            keep.append(t)
        return (torch.tensor(ptrs, dtype=torch.int64, device=device),
                torch.tensor(k2s, dtype=torch.int32, device=device), k2s)

    gp, gk, gks = table(gate, d, width)
    upp, uk, uks = table(up, d, width)
    dp, dk, dks = table(down, width, d)

    def stack(mats, j, n):
        out = torch.empty((n_exp, n), dtype=torch.float16, device=device)
        for e, m in enumerate(mats):
            out[e].copy_(m[j].reshape(-1))
        return out

    tb = torch.tensor([(d * width // 256) * (gks[e] + uks[e] + dks[e]) * 16 for e in range(n_exp)], dtype=torch.int64)
    return Exl3RoutedExperts(gp, upp, dp, gk, uk, dk, stack(gate, 1, d), stack(up, 1, d), stack(gate, 2, width),
                             stack(up, 2, width), stack(down, 1, width), stack(down, 2, d), n_exp, d, width, cb, tb,
                             keep)


def prepare_stacked(gt: torch.Tensor, ut: torch.Tensor, dt: torch.Tensor, suh_g, suh_u, svh_g, svh_u, suh_d, svh_d,
                    codebook: int | str) -> Exl3RoutedExperts:
    """A uniform-width layer stacked per projection: trellis [E, K/16, N/16, 16 * bits] (int16, or the same bytes as
    int32 words), suh/svh [E, n]."""

    def as16(t):
        return t.view(torch.int16) if t.dtype == torch.int32 else t

    gt, ut, dt = as16(gt), as16(ut), as16(dt)
    n_exp = gt.shape[0]
    return prepare([(gt[e], suh_g[e], svh_g[e]) for e in range(n_exp)],
                   [(ut[e], suh_u[e], svh_u[e]) for e in range(n_exp)],
                   [(dt[e], suh_d[e], svh_d[e]) for e in range(n_exp)], codebook, device=gt.device)


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
    """Buffers for up to ``rows`` rows of ``slots`` slots; slots whose pick is not a routed expert are left to the
    caller (``y`` keeps what the caller wrote there)."""

    def __init__(self, ex: Exl3RoutedExperts, rows: int, slots: int, sk_gu: int | None = None, sk_d: int | None = None,
                 device: str | torch.device = "cuda") -> None:
        d, width = ex.dims, ex.width
        self.sk_gu = sk_gu or default_config(d, width, True)
        self.sk_d = sk_d or default_config(width, d, False)
        p = rows * slots
        self.xg = torch.zeros((p, d), dtype=torch.float16, device=device)
        self.xu = torch.zeros((p, d), dtype=torch.float16, device=device)
        self.xd = torch.zeros((p, width), dtype=torch.float16, device=device)
        # gate and up write 2 * splits * P * I partials, down splits * P * D
        self.z = torch.zeros((max(2 * self.sk_gu * width, self.sk_d * d) * p,), dtype=torch.float32, device=device)
        self.y = torch.zeros((p, d), dtype=torch.float32, device=device)
        self.plan = grouped.Plan(rows, slots, ex.count, device)          # ids outside [0, E) join no item
        self.rows, self.slots, self.count_experts = rows, slots, ex.count


def routed(x: torch.Tensor, pick: torch.Tensor, wts: torch.Tensor | None, ex: Exl3RoutedExperts, s: Scratch,
           out: torch.Tensor | None, R: int, limit: float = math.inf, act_mode: int = ACT_F32,
           group: bool = True) -> torch.Tensor:
    """Routed experts of R rows (picks outside [0, E) skipped): Y fp32 per pair, or ``out`` fp32 [R, D] = the
    wts-weighted sum over the slots when ``wts`` is given; no host sync.  ``group=False`` reuses the grouping of the
    last call on the same picks."""

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
    if group:
        grouped.route(pick, plan)                         # the pair sort drops ids outside [0, E)
    items = grouped.max_items(p, n_exp, grouped.TILE)
    plan_args = (_lib.ptr(plan.items), _lib.ptr(plan.counts), _lib.ptr(plan.members))
    _lib.call("tf_exl3x_rot_in", _lib.ptr(x), _DTYPES[x.dtype], x.stride(0), _lib.ptr(pick), _lib.ptr(ex.suh_g),
              _lib.ptr(ex.suh_u), _lib.ptr(s.xg), _lib.ptr(s.xu), R, slots, d, n_exp)
    _lib.call("tf_exl3x_grouped", _lib.ptr(s.xg), _lib.ptr(s.xu), _lib.ptr(ex.gate_ptr), _lib.ptr(ex.up_ptr),
              _lib.ptr(ex.gate_k2), _lib.ptr(ex.up_k2), *plan_args, _lib.ptr(s.z), 2, d, width, p, s.sk_gu, ex.cb,
              n_exp, items)
    _lib.call("tf_exl3x_gateup_epilogue", _lib.ptr(s.z), _lib.ptr(pick), _lib.ptr(ex.svh_g), _lib.ptr(ex.svh_u),
              _lib.ptr(ex.suh_d), _lib.ptr(s.xd), p, width, s.sk_gu, n_exp,
              float(min(limit, 3.0e38)), act_mode)
    _lib.call("tf_exl3x_grouped", _lib.ptr(s.xd), None, _lib.ptr(ex.down_ptr), None, _lib.ptr(ex.down_k2), None,
              *plan_args, _lib.ptr(s.z), 1, width, d, p, s.sk_d, ex.cb, n_exp, items)
    if wts is None:
        _lib.call("tf_exl3x_down_combine", _lib.ptr(s.z), _lib.ptr(pick), _lib.ptr(ex.svh_d), _lib.ptr(s.y), None, None,
                  R, slots, d, s.sk_d, n_exp)
        return s.y[:p]
    if out is None:
        out = torch.empty((R, d), dtype=torch.float32, device=x.device)
    elif out.dtype != torch.float32 or tuple(out.shape) != (R, d) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous fp32 [{R}, {d}]")
    _lib.call("tf_exl3x_down_combine", _lib.ptr(s.z), _lib.ptr(pick), _lib.ptr(ex.svh_d), _lib.ptr(s.y), _lib.ptr(wts),
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
