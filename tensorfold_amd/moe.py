"""MoE layer glue (MI355X): router logits, per-row top-k with softmax-over-selected weights, the expert calls and the
weighted combine.

Host side of ``tf_moe_*``.  Names and signatures follow the reference's operator module
(src/tensorfold/cuda/moe.py:41-186), whose Triton kernels the HIP ones replace.  Rules kept: fp32 logits, ties go
to the lower expert id, weights are bf16-rounded values held in fp32, each row is routed and run independently, and
the optional shared expert rides in the last slot with a sigmoid gate.
"""

from __future__ import annotations

import dataclasses

import torch

from . import _lib
from . import experts as grouped

# ``run`` issues a decode-sized layer as routing + up + down + combine launches; with this set it issues the routing
# launch and the one fused experts launch (``decode``) instead.  Same bits either way.
FUSED_DECODE = False
# Up to this many router logits (rows x experts) a call, the up projection's workgroups each repeat the top-k
# instead of waiting for a launch; past it the top-k runs once, a launch before, and they rebuild only the plan.
ROUTE_UP_LOGITS = 2048
# With this set ``decode`` makes the whole routing (top-k, plan, group sums, descriptors) in launches of its own and
# runs the up projection from its descriptors: one launch more, for callers that want the plan before the experts.
ROUTING_LAUNCH = False
# With this set ``decode`` runs the layer as ONE launch cut along the intermediate width (``tf_moe_decode_sliced``) when
# the call has at most SLICED_ROWS rows (its scratch holds a term for every pair, input group and column); same bits.
SLICED_DECODE = False
SLICED_ROWS = 16
# Item descriptors the routing launches leave for the decode expert kernels: rows of DESC_INTS int32, row 0 the
# count; items of at most DESC_TILE pairs (TF_DESC_INTS / TF_DESC_TILE of the C header).
DESC_INTS, DESC_TILE = 8, 2
ARRIVE_STRIDE = 16   # ints between the arrival counters of two (token, 64 columns) cells with at most 64 rows, else 1


def arrive_stride(rows: int) -> int:
    return ARRIVE_STRIDE if rows <= 64 else 1
DONE_STRIDE = 64     # ints between the arrival counters of two descriptors (the one-launch form): one a 256-byte block


def router(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 logits [R, rows.shape[0]] = x [R, D] @ rows.T, both bf16.  ``rows`` holds the router's rows followed, when
    the layer has a shared expert, by that expert's gate row."""

    _lib.on_gpu(x, rows)
    if x.dtype != torch.bfloat16 or rows.dtype != torch.bfloat16 or x.stride(1) != 1 or not rows.is_contiguous():
        raise ValueError("router: x and rows must be bf16 with unit-stride rows")
    r, d = x.shape
    ne = int(rows.shape[0])
    if out is None:
        out = x.new_empty((r, ne), dtype=torch.float32)
    elif not out.is_contiguous() or tuple(out.shape) != (r, ne) or out.dtype != torch.float32:
        raise ValueError("router: out must be contiguous [R, E + 1] fp32")
    _lib.call("tf_moe_router", _lib.ptr(x), x.stride(0), _lib.ptr(rows), _lib.ptr(out), r, d, ne)
    return out


class MoEBuffers:
    """Preallocated scratch of a layer for at most ``rows`` rows, so that a captured graph can replay it.

    ``prefill`` selects the prompt arithmetic of the experts; ``shared=False`` is for layers
    without a shared expert: no extra logit column, no extra slot.  ``y_dtype``: what the pair outputs are kept as
    between the down projection and the combine: fp32, or with ``prefill`` fp16 or bf16 (half the bytes)."""

    def __init__(self, rows: int, cfg, device: torch.device | str, *, prefill: bool = False,
                 shared: bool = True, y_dtype: torch.dtype = torch.float32) -> None:
        if y_dtype != torch.float32 and not (prefill and y_dtype in (torch.float16, torch.bfloat16)):
            raise ValueError("pair outputs are fp32; a prompt plan also takes fp16 or bf16")
        extra = int(shared)
        self.rows, self.shared = rows, shared
        self.slots = cfg.num_experts_per_tok + extra
        f32 = dict(dtype=torch.float32, device=device)
        self.logits = torch.empty((rows, cfg.num_experts + extra), **f32)
        self.pick = torch.empty((rows, self.slots), dtype=torch.int32, device=device)
        self.wts = torch.empty((rows, self.slots), **f32)
        self.plan = grouped.Plan(rows, self.slots, cfg.num_experts + extra, device, prefill=prefill)
        self.act = torch.empty((rows, self.slots, cfg.moe_intermediate_size), dtype=torch.bfloat16, device=device)
        # Pair outputs are fp32 unless told.  (The reference keeps bf16 pair outputs in its prompt form,
        # cuda/moe.py:99; that rounding alone puts the layer 2.7e-3 relative L2 from the dequant-then-matmul result,
        # past a 2e-3 bound.  fp16 takes the same bytes and leaves it at 9e-4: ``run`` uses it for prompts.)
        self.y = torch.empty((rows, self.slots, cfg.hidden_size), device=device, dtype=y_dtype)
        self.cfg, self.device, self._fused = cfg, device, {}

    def fused(self, gs: int) -> dict:
        """Scratch of ``decode`` for tables of group size ``gs``, made on first use: item descriptors, the counters of the one-launch
        form (status, then an arrival count a descriptor, then one a (token, 64 columns) cell) and the output."""

        if gs not in self._fused:
            cfg, dev, pairs = self.cfg, self.device, self.rows * self.slots
            items = grouped.max_items(pairs, cfg.num_experts + int(self.shared), DESC_TILE)
            cells = max(min(self.rows, 64) * ARRIVE_STRIDE, self.rows) * (cfg.hidden_size // 64)
            self._fused[gs] = dict(
                items=items * DONE_STRIDE,          # ints the descriptors' arrival counters take
                desc=torch.zeros((1 + items, DESC_INTS), dtype=torch.int32, device=dev),
                counters=torch.zeros((1 + items * DONE_STRIDE + cells,), dtype=torch.int32, device=dev),
                out=torch.empty((self.rows, cfg.hidden_size), dtype=torch.bfloat16, device=dev))
        return self._fused[gs]

    def sliced(self, gs: int) -> dict:
        """Scratch of the one-launch form cut along the intermediate width, made on first use, for up to SLICED_ROWS
        rows: a term for every (pair, 64 columns, input group, column) and the two levels of arrival counters."""

        key = ("sliced", gs)
        if key not in self._fused:
            cfg, rows, blocks = self.cfg, min(self.rows, SLICED_ROWS), self.cfg.hidden_size // 64
            self._fused[key] = dict(
                part=torch.empty((rows * self.slots, blocks, cfg.moe_intermediate_size // gs, 64), dtype=torch.float32,
                                 device=self.device),
                arrive=torch.zeros(((rows * self.slots + rows) * blocks * ARRIVE_STRIDE,), dtype=torch.int32,
                                   device=self.device))
        return self._fused[key]

    def check(self) -> None:
        """Host-side look at the fused layer's status flag (synchronises): raises if a bounded wait ran out."""

        if any(int(f["counters"][0]) for f in self._fused.values() if "counters" in f):
            raise RuntimeError("tensorfold-amd: the fused decode layer timed out waiting for its activations")


def select_rows(logits: torch.Tensor, buf: MoEBuffers, top_k: int, experts: int) -> None:
    """Fill ``buf.pick`` / ``buf.wts`` for the rows of ``logits`` (one wave a row)."""

    _lib.on_gpu(logits)
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise ValueError("select: logits must be fp32 with unit-stride rows")
    _lib.call("tf_moe_topk", _lib.ptr(logits), logits.stride(0), int(logits.shape[0]), experts, top_k,
              int(buf.shared), _lib.ptr(buf.pick), _lib.ptr(buf.wts))


def select(logits: torch.Tensor, buf: MoEBuffers, top_k: int, experts: int,
           tile: int = grouped.PREFILL_TILE) -> None:
    """``select_rows`` followed by the pair sort into ``buf.plan`` (``tile``: a prompt plan's item size)."""

    select_rows(logits, buf, top_k, experts)
    grouped.route(buf.pick[:logits.shape[0]], buf.plan, tile)


def moe(x: torch.Tensor, router_rows: torch.Tensor, ex: grouped.Experts, buf: MoEBuffers, top_k: int,
        experts: int) -> MoEBuffers:
    """Router, selection and both expert matmuls for x [R, D]; the pair outputs are left in ``buf.y`` [R, slots, D]
    (fp32; the caller combines them, often fused with its residual add)."""

    n = int(x.shape[0])
    router(x, router_rows, buf.logits[:n])
    select(buf.logits[:n], buf, top_k, experts)
    act = buf.act.view(-1, ex.width)
    grouped.gate_up(x, ex, buf.plan, act, n)
    grouped.down(act, ex, buf.plan, buf.y.view(-1, ex.dims), n)
    return buf


def fusable(x: torch.Tensor, ex: grouped.Experts, buf: MoEBuffers) -> bool:
    """Whether ``decode`` takes this call: decode arithmetic, at most 1,024 pairs, sizes in whole 64-column units."""

    return (not buf.plan.prefill and x.shape[0] * buf.slots <= grouped.SMALL and ex.dims % 64 == 0
            and ex.width % 64 == 0)


def decode(x: torch.Tensor, logits: torch.Tensor, ex: grouped.Experts, buf: MoEBuffers, top_k: int, experts: int,
           out: torch.Tensor | None = None) -> torch.Tensor:
    """The decode layer in two launches (routing + up projection; down projection + combine), three when there are
    many router logits (top-k; plan + up; down + combine) or with ``ROUTING_LAUNCH``, or, with ``FUSED_DECODE``, routing
    and one launch for the rest.  Same bits as
    ``select`` + ``gate_up`` + ``down`` + ``combine``; bf16 [R, D] out.  ``buf.pick``, ``buf.wts`` and ``buf.plan``
    are filled as by ``select``."""

    _lib.on_gpu(x, logits)
    n = int(x.shape[0])
    if not fusable(x, ex, buf) or n > buf.rows:
        raise ValueError("decode: this call does not fit the fused decode layer (see fusable)")
    if x.dtype != torch.bfloat16 or x.stride(1) != 1 or x.stride(0) % 8 or x.shape[1] != ex.dims:
        raise RuntimeError("x: rows of K = groups * group size inputs, 16-byte aligned")
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise ValueError("select: logits must be fp32 with unit-stride rows")
    f = buf.fused(ex.gs)
    if out is None:
        out = f["out"][:n]
    plan = buf.plan
    plan.tile = grouped.TILE
    items = grouped.max_items(n * buf.slots, experts + int(buf.shared), DESC_TILE)
    cells = n * (ex.dims // 64) * arrive_stride(n)
    ctr = f["counters"]
    if FUSED_DECODE:
        _lib.call("tf_moe_route_decode", _lib.ptr(logits), logits.stride(0), n, experts, top_k, int(buf.shared),
                  _lib.ptr(buf.pick), _lib.ptr(buf.wts), _lib.ptr(plan.members), _lib.ptr(plan.items),
                  _lib.ptr(plan.counts), _lib.ptr(f["desc"]), _lib.ptr(ctr), 1 + f["items"] + cells)
        _lib.call("tf_moe_decode_experts", ex.gs, int(ex.swiglu), _lib.ptr(x), x.stride(0), n, buf.slots,
                  _lib.ptr(ex.up), _lib.ptr(ex.down), ex.dims, ex.width, _lib.ptr(f["desc"]), _lib.ptr(plan.counts),
                  _lib.ptr(buf.wts), _lib.ptr(buf.act), _lib.ptr(buf.y),
                  _lib.ptr(out), ctr.data_ptr() + 4, ctr.data_ptr() + 4 * (1 + f["items"]), _lib.ptr(ctr), ex.limit,
                  items)
        return out
    act = buf.act.view(-1, ex.width)
    if SLICED_DECODE and n <= min(SLICED_ROWS, buf.rows):
        sl = buf.sliced(ex.gs)
        given = n * (experts + int(buf.shared)) > ROUTE_UP_LOGITS
        if given:
            select_rows(logits, buf, top_k, experts)
        _lib.call("tf_moe_decode_sliced", None if given else _lib.ptr(logits), logits.stride(0), n, experts, top_k,
                  int(buf.shared), ex.gs, int(ex.swiglu), _lib.ptr(x), x.stride(0), _lib.ptr(ex.up), _lib.ptr(ex.down),
                  ex.dims, ex.width, _lib.ptr(buf.pick), _lib.ptr(buf.wts), _lib.ptr(plan.members), _lib.ptr(plan.items),
                  _lib.ptr(plan.counts), _lib.ptr(f["desc"]), _lib.ptr(act), _lib.ptr(buf.y), _lib.ptr(out),
                  _lib.ptr(sl["part"]), _lib.ptr(sl["arrive"]), ex.limit, items)
        return out
    arrive = ctr.data_ptr() + 4 * (1 + f["items"])        # one arrival counter a (token, 64 columns) cell
    if ROUTING_LAUNCH:
        # the routing in a launch of its own, then up, down and combine from its item descriptors
        _lib.call("tf_moe_route_decode", _lib.ptr(logits), logits.stride(0), n, experts, top_k, int(buf.shared),
                  _lib.ptr(buf.pick), _lib.ptr(buf.wts), _lib.ptr(plan.members), _lib.ptr(plan.items),
                  _lib.ptr(plan.counts), _lib.ptr(f["desc"]), arrive, cells)
        _lib.call("tf_experts_run_desc", ex.gs, 2 if ex.swiglu else 1, _lib.ptr(x), x.stride(0), buf.slots,
                  _lib.ptr(ex.up), ex.dims // ex.gs, ex.width // grouped.COLS, _lib.ptr(f["desc"]),
                  _lib.ptr(plan.counts), _lib.ptr(act), ex.width, ex.limit, items)
    else:
        # few logits: every workgroup of the up projection routes for itself; many: the top-k runs once, in a launch
        # before, and the workgroups only rebuild the plan from its picks
        given = n * (experts + int(buf.shared)) > ROUTE_UP_LOGITS
        if given:
            select_rows(logits, buf, top_k, experts)
        _lib.call("tf_moe_route_up", None if given else _lib.ptr(logits), logits.stride(0), n, experts, top_k,
                  int(buf.shared), ex.gs,
                  int(ex.swiglu), _lib.ptr(x), x.stride(0), _lib.ptr(ex.up), ex.dims, ex.width, _lib.ptr(buf.pick),
                  _lib.ptr(buf.wts), _lib.ptr(plan.members), _lib.ptr(plan.items), _lib.ptr(plan.counts),
                  _lib.ptr(f["desc"]), _lib.ptr(act), ex.limit, items, arrive, cells)
    # the down projection; the workgroup that completes a (token, 64 columns) cell writes the combined output
    _lib.call("tf_moe_down_combine", ex.gs, _lib.ptr(act), n, buf.slots, _lib.ptr(ex.down), ex.dims, ex.width,
              _lib.ptr(f["desc"]), _lib.ptr(buf.wts), _lib.ptr(buf.y), _lib.ptr(out), arrive, items)
    return out


def combine(y: torch.Tensor, wts: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """bf16 [R, D] = sum over slots, in slot order and in fp32, of wts[r, k] * y[r, k]; y is fp32, bf16 or fp16
    [R, S, D]."""

    _lib.on_gpu(y, wts)
    if not y.is_contiguous() or not wts.is_contiguous() or wts.dtype != torch.float32:
        raise ValueError("combine: y and wts must be contiguous, wts fp32")
    r, s, d = y.shape
    if out is None:
        out = y.new_empty((r, d), dtype=torch.bfloat16)
    kind = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}.get(y.dtype)
    if kind is None:
        raise ValueError("combine: y must be fp32, bf16 or fp16")
    _lib.call("tf_moe_combine", _lib.ptr(y), kind, _lib.ptr(wts), _lib.ptr(out), r, s, d)
    return out


@dataclasses.dataclass
class Routed:
    """What ``run`` needs of a layer: router rows bf16 [E + 1, D] (gate row of the shared expert last), the packed
    E + 1 experts, and k."""

    router: torch.Tensor
    experts: grouped.Experts
    top_k: int

    @property
    def count(self) -> int:
        return int(self.router.shape[0]) - 1


class _Dims:
    """The four sizes MoEBuffers reads, taken from a ``Routed``."""

    def __init__(self, m: Routed) -> None:
        self.num_experts, self.num_experts_per_tok = m.count, m.top_k
        self.hidden_size, self.moe_intermediate_size = m.experts.dims, m.experts.width


_pool: dict[tuple, MoEBuffers] = {}


def run(x: torch.Tensor, m: Routed, *, prefill: bool = False) -> torch.Tensor:
    """The whole layer: bf16 [R, D] in, bf16 [R, D] out.  Scratch is pooled by the row count rounded up to a power
    of two (16 at least), so every layer of a model shares it.  A prompt's pair outputs are kept in fp16 between the
    down projection and the combine (half the traffic of fp32; a pair output beyond +-65504 is stored as +-65504)
    when the layer runs the fp16 prompt arithmetic, which makes the same assumption of its activations; a layer
    made with ``ARITH_BF16`` keeps them in fp32."""

    n = int(x.shape[0])
    cap = max(16, 1 << (n - 1).bit_length())
    y_dtype = torch.float16 if prefill and m.experts.arith == grouped.ARITH_F16 else torch.float32
    key = (cap, m.count, m.top_k, m.experts.width, m.experts.dims, m.experts.gs, prefill, y_dtype, x.device)
    if key not in _pool:
        _pool[key] = MoEBuffers(cap, _Dims(m), x.device, prefill=prefill, y_dtype=y_dtype)
    buf, x = _pool[key], x.contiguous()
    if fusable(x, m.experts, buf):
        router(x, m.router, buf.logits[:n])
        return decode(x, buf.logits[:n], m.experts, buf, m.top_k, m.count).clone()
    moe(x, m.router, m.experts, buf, m.top_k, m.count)
    return combine(buf.y[:n], buf.wts[:n])
