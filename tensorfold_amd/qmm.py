"""Dense 4-bit affine matmul ("lane matmul") on MI355X.

Host side of ``tf_qmm*`` / ``tf_group_sums``.  The public names and signatures are the operator interface of the
reference (src/tensorfold/cuda/kernels/qmm.py:41-219); the packed layout, the K split and the kernels are this
package's.  Invariant kept: groups and K slices are walked identically at every row count, so a row's output bits
do not depend on its neighbours.
"""

from __future__ import annotations

import dataclasses

import torch

from . import _lib


COUNTER_STRIDE = 16          # TF_QMM_COUNTER_STRIDE of include/tfmi.h


@dataclasses.dataclass
class Q4:
    """A packed (n, k) weight.

    weight int32 [npad/64, k/gs, gs/32, 64, 4]  (64-column tiles; chunks of 32 inputs; 4 words a column a chunk)
    scales, biases bf16 [k/gs, npad]            (npad = n rounded up to 128; padding is zero)
    """

    weight: torch.Tensor
    scales: torch.Tensor
    biases: torch.Tensor
    n: int
    k: int
    gs: int
    arith: int = 0       # the prompt form's arithmetic (TF_ARITH_*): 1 when a scale or bias does not fit the fp16 form
    _counters: torch.Tensor | None = dataclasses.field(default=None, init=False, repr=False, compare=False)

    def __post_init__(self) -> None:
        # made with the weight, never inside a matmul call (which may run under graph capture)
        if self.weight.is_cuda:
            self._counters = torch.zeros((-(-self.n // 64) * COUNTER_STRIDE,), dtype=torch.int32,
                                         device=self.weight.device)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.weight, self.scales, self.biases))

    @property
    def counters(self) -> torch.Tensor:
        """Arrival counters of the K slices, one a column tile of 64, each alone in 64 bytes; zero between calls.
        With them ``matmul`` on up to eight rows adds the slices up in its own launch.  Calls on one weight that
        overlap in time (two streams), or one weight given twice to ``matmul_group``, need a ``Q4`` of their own each
        (``dataclasses.replace`` shares the packed tensors and starts with fresh counters)."""

        if self._counters is None:
            self._counters = torch.zeros((-(-self.n // 64) * COUNTER_STRIDE,), dtype=torch.int32, device=self.weight.device)
        return self._counters


def pack(weight: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor, gs: int) -> Q4:
    """MLX layout (words [n, k/8] int32 or uint32, scales and biases [n, k/gs]) -> ``Q4``, in one kernel."""

    if gs not in (32, 64):
        raise ValueError(f"groups of 32 or 64 inputs, not {gs}")
    words = weight if weight.dtype == torch.int32 else weight.view(torch.int32)
    n, k8 = words.shape
    k = 8 * k8
    if k % gs or tuple(scales.shape) != (n, k // gs) or tuple(biases.shape) != (n, k // gs):
        raise ValueError(f"qmm: shape {tuple(words.shape)} with scales {tuple(scales.shape)} does not pack")
    _lib.on_gpu(words, scales, biases)
    kg, npad = k // gs, 128 * -(-n // 128)
    q = Q4(words.new_empty((npad // 64, kg, gs // 32, 64, 4)),
           words.new_empty((kg, npad), dtype=torch.bfloat16), words.new_empty((kg, npad), dtype=torch.bfloat16),
           n, k, gs)
    # converted or re-laid copies are held by name until the launch is queued: a temporary freed between two
    # arguments would hand its memory to the next one
    words, s16, b16 = words.contiguous(), scales.to(torch.bfloat16).contiguous(), biases.to(torch.bfloat16).contiguous()
    _lib.call("tf_qmm_pack", _lib.ptr(words), _lib.ptr(s16), _lib.ptr(b16), n, k, gs, _lib.ptr(q.weight),
              _lib.ptr(q.scales), _lib.ptr(q.biases))
    from .experts import ARITH_BF16, ARITH_F16, fits_f16

    q.arith = ARITH_F16 if fits_f16(scales, biases) else ARITH_BF16
    return q


def unpack(q: Q4) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``pack`` inverted: (words [n, k/8], scales [n, k/gs], biases [n, k/gs])."""

    kg = q.k // q.gs
    words = q.weight.new_empty((q.n, q.k // 8))
    scales = q.scales.new_empty((q.n, kg))
    biases = q.scales.new_empty((q.n, kg))
    weight, s16, b16 = q.weight.contiguous(), q.scales.contiguous(), q.biases.contiguous()      # views of ``rows``
    _lib.call("tf_qmm_unpack", _lib.ptr(weight), _lib.ptr(s16), _lib.ptr(b16), q.n, q.k, q.gs, _lib.ptr(words),
              _lib.ptr(scales), _lib.ptr(biases))
    return words, scales, biases


def rows(q: Q4, a: int, b: int) -> Q4:
    """Output rows [a, b) of a packed weight (families/qwen3_5/cuda/qmm_fast.py:28-38).  From a 64-row tile edge and in
    whole blocks of 128 rows it is a view of ``q``; any other range unpacks the tiles it touches and packs the rows
    again (a small copy).  ``matmul`` on the part gives the whole weight's bits when it is told the whole weight's
    ``sk`` (``matmul_rows`` does)."""

    if not 0 <= a < b <= q.n:
        raise ValueError(f"rows [{a}, {b}) of a weight of {q.n}")
    if a % 64 == 0 and (b - a) % 128 == 0:
        return Q4(q.weight[a // 64:b // 64], q.scales[:, a:b], q.biases[:, a:b], b - a, q.k, q.gs, q.arith)
    t0, t1 = a // 64, -(-b // 64)
    span = 128 * -(-(t1 - t0) // 2)                 # tiles come in pairs: a packed weight's rows are padded to 128
    first = min(t0, q.weight.shape[0] - span // 64)
    tiles = Q4(q.weight[first:first + span // 64], q.scales[:, 64 * first:64 * first + span],
               q.biases[:, 64 * first:64 * first + span], span, q.k, q.gs, q.arith)
    words, scales, biases = unpack(tiles)
    lo, hi = a - 64 * first, b - 64 * first
    part = pack(words[lo:hi].contiguous(), scales[lo:hi].contiguous(), biases[lo:hi].contiguous(), q.gs)
    part.arith = q.arith
    return part


def matmul_rows(x: torch.Tensor, parts: list[Q4]) -> torch.Tensor:
    """x against row blocks of one weight, side by side, with the bits of the stacked weight's ``matmul``: the K
    split is the stacked weight's (families/qwen3_5/cuda/qmm_fast.py:41-46)."""

    sk = split_k(sum(p.n for p in parts), parts[0].k, parts[0].gs)
    xs = group_sums(x, parts[0].gs)
    return torch.cat([matmul(x, p, xs, sk=sk) for p in parts], dim=1)


def split_k(n: int, k: int, gs: int = 64, target: int = 768) -> int:
    """Number of K slices of an (n, k) weight - from the shape alone, never the row count.

    Doubles while that keeps the workgroups (64-column tiles x slices) within ``target`` (an MI355X has 256 CUs and
    the launch is fastest with two or three four-wave workgroups on each: 4096 x 4096 at one row takes 6.0 us with 8
    slices, 6.1 with 16; 6144 x 5120 7.1 against 9.1; 5120 x 17408 12.3 against 15.4), the groups still divide evenly
    and a slice keeps at least 4 groups."""

    tiles, groups = -(-n // 64), k // gs
    sk = 1
    while sk < 16 and 2 * tiles * sk <= target and groups % (2 * sk) == 0 and groups // (2 * sk) >= 4:
        sk *= 2
    return sk


def bucket(m: int) -> int:
    """Rows a workgroup walks: 16, 32 or 64.  Purely a scheduling choice; bits do not change with it."""

    if m < 1:
        raise ValueError("the lane matmul takes at least one row")
    return 16 if m <= 16 else (32 if m <= 32 else 64)


def _aligned_rows(x: torch.Tensor) -> torch.Tensor:
    """The kernels read rows in 16-byte pieces: copy x when its rows are not laid out for that."""

    bad = x.stride(1) != 1 or x.data_ptr() % 16 or (x.shape[0] > 1 and x.stride(0) % 8)
    return x.clone(memory_format=torch.contiguous_format) if bad else x


def group_sums(x: torch.Tensor, gs: int = 64) -> torch.Tensor:
    """fp32 [M, K/gs]: the sum of every group of ``gs`` inputs of x (bf16 [M, K], rows may be strided)."""

    _lib.on_gpu(x)
    x = _aligned_rows(x)
    m, k = x.shape
    xs = x.new_empty((m, k // gs), dtype=torch.float32)
    _lib.call("tf_group_sums", _lib.ptr(x), x.stride(0), m, k, gs, _lib.ptr(xs))
    return xs


def _check_x(x: torch.Tensor, q: Q4, who: str) -> torch.Tensor:
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != q.k:
        raise ValueError(f"{who}: x must be (M, {q.k}) bf16")
    _lib.on_gpu(x)
    return _aligned_rows(x)


def matmul(x: torch.Tensor, q: Q4, xs: torch.Tensor | None = None, *, sk: int | None = None, f32: bool = False,
           out: torch.Tensor | None = None, part: torch.Tensor | None = None, reduce: bool = True) -> torch.Tensor:
    """Decode-form x @ W.T -> (M, n) bf16, or fp32 without the final rounding when ``f32``.

    With ``reduce=False`` the fp32 K slices come back unadded as (sk, M, n); adding them in order and rounding once
    reproduces the reduced result bit for bit."""

    x = _check_x(x, q, "matmul")
    m = int(x.shape[0])
    xs = group_sums(x, q.gs) if xs is None else xs
    sk = split_k(q.n, q.k, q.gs) if not sk else sk
    if out is None:
        out = x.new_empty((m, q.n), dtype=torch.float32 if f32 else torch.bfloat16)
    elif tuple(out.shape) != (m, q.n) or out.dtype != (torch.float32 if f32 else torch.bfloat16) \
            or not out.is_contiguous() or out.device != x.device:
        raise ValueError(f"matmul: out must be contiguous ({m}, {q.n}) {'fp32' if f32 else 'bf16'} on x's device")
    if sk > 1 and part is None:
        part = x.new_empty((sk, m, q.n), dtype=torch.float32)
    elif sk > 1 and (part.dtype != torch.float32 or part.numel() < sk * m * q.n or not part.is_contiguous()
                     or part.device != x.device):
        raise ValueError(f"matmul: part must hold {sk} x {m} x {q.n} fp32 values (split_k gives the slice count)")
    if xs.dtype != torch.float32 or tuple(xs.shape) != (m, q.k // q.gs) or not xs.is_contiguous() \
            or xs.device != x.device:
        raise ValueError(f"matmul: xs must be contiguous fp32 ({m}, {q.k // q.gs}), the group sums of x")
    counters = q.counters if reduce and sk > 1 and m <= 8 else None
    _lib.call("tf_qmm", _lib.ptr(x), x.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales),
              _lib.ptr(q.biases), q.scales.stride(0), _lib.ptr(out), _lib.ptr(part), _lib.ptr(counters),
              0 if counters is None else counters.numel() // COUNTER_STRIDE, m, q.n, q.k, sk, q.gs, bucket(m),
              int(f32), int(reduce))
    if reduce or sk == 1:
        return out
    return part.reshape(-1)[:sk * m * q.n].view(sk, m, q.n)


STATIC_FLOATS = 4 << 20          # TF_QMM_STATIC_FLOATS of include/tfmi.h


def matmul_static(x: torch.Tensor, q: Q4, xs: torch.Tensor, out: torch.Tensor, *, sk: int | None = None,
                  f32: bool = False) -> torch.Tensor:
    """``matmul`` into the caller's ``out`` with nothing allocated on the way: the K slices go to an array built into
    the library (one a GPU, 16 MiB), so ``sk * M * n`` may not exceed ``STATIC_FLOATS``.  x must already have
    16-byte aligned rows and ``xs`` its group sums.  Same bits as ``matmul``; calls that overlap on one GPU share
    that array and race.  No counterpart in the reference (for callers that cannot allocate)."""

    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != q.k:
        raise ValueError(f"matmul_static: x must be (M, {q.k}) bf16")
    _lib.on_gpu(x, xs, out)
    m = int(x.shape[0])
    if x.stride(1) != 1 or x.data_ptr() % 16 or (m > 1 and x.stride(0) % 8):
        raise ValueError("matmul_static: x rows must be contiguous and start on 16-byte boundaries (nothing is copied)")
    sk = split_k(q.n, q.k, q.gs) if not sk else sk
    if sk > 1 and sk * m * q.n > STATIC_FLOATS:
        raise ValueError(f"matmul_static: {sk} x {m} x {q.n} partial sums exceed the built-in {STATIC_FLOATS}; "
                         "use matmul with a part buffer")
    if tuple(out.shape) != (m, q.n) or out.dtype != (torch.float32 if f32 else torch.bfloat16) \
            or not out.is_contiguous() or out.device != x.device:
        raise ValueError(f"matmul_static: out must be contiguous ({m}, {q.n}) {'fp32' if f32 else 'bf16'} on x's device")
    if xs.dtype != torch.float32 or tuple(xs.shape) != (m, q.k // q.gs) or not xs.is_contiguous() \
            or xs.device != x.device:
        raise ValueError(f"matmul_static: xs must be contiguous fp32 ({m}, {q.k // q.gs}), the group sums of x")
    _lib.call("tf_qmm_static", _lib.ptr(x), x.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales),
              _lib.ptr(q.biases), q.scales.stride(0), _lib.ptr(out), m, q.n, q.k, sk, q.gs, bucket(m), int(f32))
    return out


def matmul_group(x: torch.Tensor, qs: list[Q4], xs: torch.Tensor | None = None, *, f32: bool = False,
                 sks: list[int] | None = None, outs: list[torch.Tensor] | None = None,
                 parts: list[torch.Tensor | None] | None = None) -> list[torch.Tensor]:
    """``[matmul(x, q) for q in qs]`` for one to four weights of the same K and group size in one launch (plus one
    reduce launch), same bits.  ``outs`` and ``parts`` may bring preallocated buffers (a part where sks[i] > 1)."""

    import ctypes

    if not 1 <= len(qs) <= 4:
        raise ValueError("matmul_group: one to four weights")
    if x.dtype != torch.bfloat16 or x.dim() != 2 or any(x.shape[1] != q.k for q in qs):
        raise ValueError("matmul_group: x must be (M, K) bf16 with every weight's K")
    if any(q.gs != qs[0].gs for q in qs):
        raise ValueError("matmul_group: the weights must share a group size")
    if len({id(q.counters) for q in qs}) != len(qs):
        raise ValueError("matmul_group: a weight given twice would share its arrival counters with itself; "
                         "give the second one as dataclasses.replace(q)")
    x = _check_x(x, qs[0], "matmul_group")
    m, gs, k = int(x.shape[0]), qs[0].gs, qs[0].k
    xs = group_sums(x, gs) if xs is None else xs
    if xs.dtype != torch.float32 or tuple(xs.shape) != (m, k // gs) or not xs.is_contiguous() or xs.device != x.device:
        raise ValueError(f"matmul_group: xs must be contiguous fp32 ({m}, {k // gs}), the group sums of x")
    sks = list(sks) if sks else [split_k(q.n, q.k, q.gs) for q in qs]
    dtype = torch.float32 if f32 else torch.bfloat16
    if outs is None:
        outs = [x.new_empty((m, q.n), dtype=dtype) for q in qs]
    parts = list(parts) if parts else [None] * len(qs)
    if len(sks) != len(qs) or len(outs) != len(qs) or len(parts) != len(qs):
        raise ValueError("matmul_group: one slice count, output and part a weight")
    for i, (q, sk, out) in enumerate(zip(qs, sks, outs)):
        if tuple(out.shape) != (m, q.n) or out.dtype != dtype or not out.is_contiguous() or out.device != x.device:
            raise ValueError(f"matmul_group: outs[{i}] must be contiguous ({m}, {q.n}) {'fp32' if f32 else 'bf16'}")
        if sk > 1 and parts[i] is None:
            parts[i] = x.new_empty((sk, m, q.n), dtype=torch.float32)
        elif sk > 1 and (parts[i].dtype != torch.float32 or parts[i].numel() < sk * m * q.n
                         or not parts[i].is_contiguous() or parts[i].device != x.device):
            raise ValueError(f"matmul_group: parts[{i}] must hold {sk} x {m} x {q.n} fp32 values")
    n = len(qs)
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[None if t is None else t.data_ptr() for t in ts])
    counters = [q.counters if sk > 1 and m <= 8 else None for q, sk in zip(qs, sks)]
    _lib.call("tf_qmm_group", _lib.ptr(x), x.stride(0), _lib.ptr(xs), n, ptrs([q.weight for q in qs]),
              ptrs([q.scales for q in qs]), ptrs([q.biases for q in qs]),
              (ctypes.c_int64 * n)(*[q.scales.stride(0) for q in qs]), ptrs(outs), ptrs(parts), ptrs(counters),
              (ctypes.c_int * n)(*[0 if c is None else c.numel() // COUNTER_STRIDE for c in counters]),
              (ctypes.c_int * n)(*[q.n for q in qs]), (ctypes.c_int * n)(*sks), m, k, gs, bucket(m), int(f32))
    return outs


def prompt_tile(m: int, n: int, k: int = 64) -> int:
    """The prompt matmul's tile for ``m`` rows (cuda/kernels/qmm.py:202-205 names the reference's one tile, tuned for
    its chip): 1, 4 or 8 = a four-wave workgroup on 16, 64 or 128 rows x 128 columns; 9 = eight waves on 128 rows x
    512 columns, from 65 rows on, for K in whole steps of 64.  What ``tile=0`` picks."""

    if m <= 16:
        return 1
    if m <= 64:
        return 4
    return 9 if k % 64 == 0 else 8


def prefill_matmul(x: torch.Tensor, q: Q4, *, f32: bool = False, tile: int = 0,
                   out: torch.Tensor | None = None, arith: int | None = None) -> torch.Tensor:
    """Prompt-form x @ W.T on MFMA: every weight is rounded once and K is one fp32 chain, so chunking a prompt never
    changes a row's bits (they differ from ``matmul``'s).  ``arith`` 0: fp16 operands (256 w rounded to fp16;
    activations beyond +-65504 are clamped); 1: the reference's bf16 operands (w rounded to bf16), slower, with
    bf16's range; None: what ``pack`` found the weight's scales and biases to need.  ``tile``: 0 or a ``prompt_tile``
    code; the bits are the same whatever the tile."""

    if tile not in (0, 1, 4, 8, 9):
        raise ValueError("prefill_matmul: tile 0, 1, 4, 8 or 9 (see prompt_tile)")
    x = _check_x(x, q, "prefill_matmul")
    m = int(x.shape[0])
    if out is None:
        out = x.new_empty((m, q.n), dtype=torch.float32 if f32 else torch.bfloat16)
    elif tuple(out.shape) != (m, q.n) or out.dtype != (torch.float32 if f32 else torch.bfloat16) \
            or not out.is_contiguous() or out.device != x.device:
        raise ValueError(f"prefill_matmul: out must be contiguous ({m}, {q.n}) {'fp32' if f32 else 'bf16'}")
    s16, b16 = q.scales.contiguous(), q.biases.contiguous()
    _lib.call("tf_qmm_prefill", _lib.ptr(x), x.stride(0), _lib.ptr(q.weight), _lib.ptr(s16), _lib.ptr(b16),
              _lib.ptr(out), m, q.n, q.k, q.gs, int(f32), tile,
              q.arith if arith is None else int(arith))
    return out


def quantize_rows(x: torch.Tensor, gs: int = 64) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Inputs for ``prefill_matmul8`` (cuda/kernels/qmm.py:245-255): e4m3 bytes [M, K] with every octet of inputs in
    the matrix operand's order, each group's input sum over the row scale (bf16 [M, K / gs]), the row scales (fp32
    [M]: max|x| / 448)."""

    _lib.on_gpu(x)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        raise ValueError("quantize_rows: x must be bf16 (M, K)")
    m, k = (int(v) for v in x.shape)
    if k % gs or k % 32:
        raise ValueError("quantize_rows takes K a multiple of the group and of 32")
    if x.stride(1) != 1 or (m > 1 and x.stride(0) % 8) or x.data_ptr() % 16:
        x = x.clone(memory_format=torch.contiguous_format)
    x8 = torch.empty((m, k), dtype=torch.uint8, device=x.device)
    xs = torch.empty((m, k // gs), dtype=torch.bfloat16, device=x.device)
    a = torch.empty((m,), dtype=torch.float32, device=x.device)
    _lib.call("tf_quantize_rows", _lib.ptr(x), x.stride(0), m, k, gs, _lib.ptr(x8), _lib.ptr(xs), _lib.ptr(a))
    return x8, xs, a


def prefill_matmul8(xq: tuple[torch.Tensor, torch.Tensor, torch.Tensor], q: Q4, *, f32: bool = False, tile: int = 0,
                    out: torch.Tensor | None = None) -> torch.Tensor:
    """FP8 prompt matmul on ``quantize_rows`` output, the 4-bit codes as exact e4m3 operands
    (cuda/kernels/qmm.py:258-268); a row's bits depend only on that row.  K in whole steps of 64."""

    x8, xs, a = xq
    _lib.on_gpu(x8, xs, a)
    if x8.dim() != 2 or x8.shape[1] != q.k:
        raise ValueError(f"prefill_matmul8: inputs must be (M, {q.k})")
    m = int(x8.shape[0])
    if x8.dtype != torch.uint8 or not x8.is_contiguous() or xs.dtype != torch.bfloat16 or not xs.is_contiguous() \
            or tuple(xs.shape) != (m, q.k // q.gs) or a.dtype != torch.float32 or tuple(a.shape) != (m,) \
            or not a.is_contiguous():
        raise ValueError("prefill_matmul8: takes what quantize_rows returned for this weight's group size")
    if q.k % 64:
        raise ValueError("prefill_matmul8 takes K in whole steps of 64 inputs")
    if out is None:
        out = torch.empty((m, q.n), dtype=torch.float32 if f32 else torch.bfloat16, device=x8.device)
    elif tuple(out.shape) != (m, q.n) or out.dtype != (torch.float32 if f32 else torch.bfloat16) \
            or not out.is_contiguous() or out.device != x8.device:
        raise ValueError(f"prefill_matmul8: out must be contiguous ({m}, {q.n}) {'fp32' if f32 else 'bf16'}")
    s16, b16 = q.scales.contiguous(), q.biases.contiguous()
    _lib.call("tf_qmm_prefill8", _lib.ptr(x8), _lib.ptr(xs), _lib.ptr(a), _lib.ptr(q.weight), _lib.ptr(s16),
              _lib.ptr(b16), _lib.ptr(out), m, q.n, q.k, q.gs,
              int(f32), tile)
    return out

