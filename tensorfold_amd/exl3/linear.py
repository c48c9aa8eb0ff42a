"""EXL3 linear layers on MI355X: y = x @ W + bias for 1 to 128 rows, any codebook and width, row-invariant.

Host side of ``tf_exl3_*``; the class and function names follow the reference's operator module
(src/tensorfold/cuda/exl3/linear.py:30-204).  W = diag(suh) H W_q H diag(svh): ``rot_in`` rotates the input once a
call (fp16 out), ``linear`` decodes each pair of k tiles straight into f16 MFMA operands, sums in fp32 in a fixed
order and applies the output Hadamard, svh and the bias.
"""

from __future__ import annotations

import dataclasses

import torch

from .. import _lib
from . import format as fmt

CODEBOOK_IDS = fmt.CODEBOOK_IDS
COUNTER_STRIDE = 16       # ints between two K-split arrival counters (TF_EXL3_COUNTER_STRIDE): each alone in 64 bytes
_DTYPES = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}


def k2_of(bits: float) -> int:
    """Twice the width: the integer the kernels are specialised on."""

    return int(2 * fmt.check_bits(bits))


def plan(k: int, n: int, waves: int = 4096, min_pairs: int = 4) -> tuple[int, int]:
    """(K splits, waves a workgroup) of a K x N layer, from the shape alone so that a layer keeps one reduction
    order at every row count.  The decode is bound by vector arithmetic, every wave of a launch is resident at once,
    and the launch ends with the busiest SIMD: a column block of 128 gets as many waves (splits x waves a workgroup)
    as put just under four on each of an MI355X's 1,024 SIMDs, none of them with fewer than ``min_pairs`` pairs of k
    tiles.  Many waves a block go eight a workgroup, so that the splits' partial sums stay few."""

    pairs, nb = k // 32, n // 128
    slots = max(2, min(waves // max(nb, 1), pairs // min_pairs, 512))
    wk = 8 if slots >= 64 else (4 if slots >= 8 else 2)
    sk = max(1, min(64, slots // wk))
    while wk > 2 and sk * wk > pairs:
        wk //= 2
    return min(sk, max(1, pairs // wk)), wk


def strips(words: torch.Tensor) -> torch.Tensor:
    """Trellis words [K/16, N/16, W] -> [N/128, K/16, 8, W] (a copy): each 128-column block's tiles in k order, the
    order a workgroup walks."""

    return words.unflatten(1, (-1, 8)).movedim(1, 0).contiguous()


def _scale_vector(t: torch.Tensor, size: int, device) -> torch.Tensor:
    """A layer's suh or svh as fp16 [size] on ``device``; older checkpoints store one sign bit an element instead
    (int16 [size / 16]), which become +-1."""

    if t.dtype == torch.int16 and 16 * t.numel() == size:
        t = torch.from_numpy(fmt.unpack_signs(t))
    if t.dtype != torch.float16 or t.numel() != size:
        raise ValueError(f"scales must be fp16 [{size}] or int16 sign words [{size // 16}]")
    return t.to(device).reshape(size).contiguous()


def _decode(words: torch.Tensor, k: int, n: int, strides: tuple[int, int], k2: int, codebook: str,
            out: torch.Tensor | None) -> torch.Tensor:
    """W_q [K, N] fp16 from GPU trellis words laid out with ``strides`` (see ``Exl3Linear.strides``)."""

    if out is None:
        out = words.new_empty((k, n), dtype=torch.float16)
    _lib.call("tf_exl3_unpack", _lib.ptr(words), _lib.ptr(out), k, n, *strides, k2, CODEBOOK_IDS[codebook])
    return out


@dataclasses.dataclass
class Exl3Linear:
    """One EXL3 layer resident on the GPU."""

    words: torch.Tensor           # int32 [N/128, K/16, 8, 8 * bits] ("strips") or [K/16, N/16, 8 * bits] ("stored")
    suh: torch.Tensor             # fp16 [K]
    svh: torch.Tensor             # fp16 [N]
    bias: torch.Tensor | None     # fp16 [N]
    bits: float
    codebook: str
    k: int
    n: int
    layout: str = "strips"
    split: tuple[int, int] | None = None     # (K splits, waves); plan(k, n) when None

    def __post_init__(self) -> None:
        if self.split is None:
            self.split = plan(self.k, self.n)
        self._counters: torch.Tensor | None = None

    @classmethod
    def from_tensors(cls, trellis: torch.Tensor, suh: torch.Tensor, svh: torch.Tensor, codebook: str,
                     bias: torch.Tensor | None = None, device: str | torch.device = "cuda",
                     layout: str = "strips") -> "Exl3Linear":
        """Build from a checkpoint group: trellis int16 [K/16, N/16, 16 * bits]; suh / svh fp16, or the int16 sign
        words of older checkpoints; the codebook's name."""

        if layout not in ("strips", "stored"):
            raise ValueError(f"layout must be 'strips' or 'stored', got {layout!r}")
        bits = fmt.bits_of(trellis.shape)
        fmt.check_pair(bits, codebook)
        k, n = (16 * int(v) for v in trellis.shape[:2])
        if k % fmt.HAD or n % fmt.HAD:
            raise ValueError(f"K={k} and N={n} must be multiples of 128")
        words = trellis.to(device).contiguous().view(torch.int32)
        return cls(words=strips(words) if layout == "strips" else words, suh=_scale_vector(suh, k, device),
                   svh=_scale_vector(svh, n, device),
                   bias=None if bias is None else bias.to(device=device, dtype=torch.float16).contiguous(),
                   bits=bits, codebook=codebook, k=k, n=n, layout=layout)

    @property
    def k2(self) -> int:
        return k2_of(self.bits)

    @property
    def strides(self) -> tuple[int, int]:
        """int32 words from one k tile to the next, and from one 128-column block to the next."""

        if self.layout == "strips":                       # [N/128, K/16, 8, W]
            return self.words.stride(1), self.words.stride(0)
        return self.words.stride(0), 8 * self.words.stride(1)       # [K/16, N/16, W]: a block is 8 tiles side by side

    def nbytes(self) -> int:
        return self.words.numel() * 4

    @property
    def counters(self) -> torch.Tensor:
        """Arrival counters of the K splits, zero between calls."""

        if self._counters is None:
            self._counters = torch.zeros((8 * (self.n // 128) * COUNTER_STRIDE,), dtype=torch.int32, device=self.words.device)
        return self._counters

    def __call__(self, x: torch.Tensor, out: torch.Tensor | None = None, out_dtype: torch.dtype | None = None,
                 xh: torch.Tensor | None = None, z: torch.Tensor | None = None) -> torch.Tensor:
        """y [M, N] for x [M, K], M = 1..128 (fp16, bf16 or fp32 in and out).  ``xh`` (fp16 [M, K]) and ``z`` (fp32
        [splits * M * N]) are scratch, allocated here when not passed."""

        if x.dim() != 2 or x.shape[1] != self.k or not 1 <= x.shape[0] <= 128:
            raise ValueError(f"x must be [1..128, {self.k}], got {tuple(x.shape)}")
        if x.dtype not in _DTYPES:
            raise ValueError("x: expected fp16, bf16 or fp32")
        _lib.on_gpu(x)
        x = x.contiguous()
        m = int(x.shape[0])
        if out is None:
            out = x.new_empty((m, self.n), dtype=out_dtype or x.dtype)
        elif tuple(out.shape) != (m, self.n) or out.dtype not in _DTYPES or not out.is_contiguous():
            raise ValueError(f"out must be contiguous ({m}, {self.n}) fp16, bf16 or fp32")
        else:
            _lib.on_gpu(out)
        sk, wk = self.split
        if xh is None:
            xh = x.new_empty((m, self.k), dtype=torch.float16)
        elif xh.dtype != torch.float16 or xh.numel() < m * self.k or not xh.is_contiguous() or xh.device != x.device:
            raise ValueError(f"xh must hold {m} x {self.k} fp16 values on x's device")
        if sk > 1 and z is None:
            z = x.new_empty((sk * m * self.n,), dtype=torch.float32)
        elif sk > 1 and (z.dtype != torch.float32 or z.numel() < sk * m * self.n or not z.is_contiguous()
                         or z.device != x.device):
            raise ValueError(f"z must hold {sk} x {m} x {self.n} fp32 values on x's device")
        stride_k, stride_nb = self.strides
        _lib.call("tf_exl3_rot_in", _lib.ptr(x), _DTYPES[x.dtype], _lib.ptr(self.suh), _lib.ptr(xh), m, self.k)
        _lib.call("tf_exl3_linear", _lib.ptr(xh), _lib.ptr(self.words), stride_k, stride_nb, _lib.ptr(self.svh),
                  _lib.ptr(self.bias), _lib.ptr(out), _DTYPES[out.dtype], _lib.ptr(z) if sk > 1 else None,
                  _lib.ptr(self.counters), m, self.k, self.n, self.k2, CODEBOOK_IDS[self.codebook], sk, wk)
        return out

    def unpack(self, out: torch.Tensor | None = None) -> torch.Tensor:
        """W_q [K, N] fp16, decoded on the GPU from either layout."""

        return _decode(self.words, self.k, self.n, self.strides, self.k2, self.codebook, out)


@dataclasses.dataclass
class Exl3Stack:
    """Layers of one shape, width, codebook and layout that read the same input (an MLP's gate and up projections),
    laid side by side so that a call is one rotation launch and one linear launch for all of them.  Every layer's
    output has the bits of its own ``Exl3Linear`` call."""

    words: torch.Tensor           # int32 [L, ...one layer's words...]
    suh: torch.Tensor             # fp16 [L, K]
    svh: torch.Tensor             # fp16 [L, N]
    bias: torch.Tensor | None     # fp16 [L, N] (layers without one add zero)
    bits: float
    codebook: str
    k: int
    n: int
    layout: str
    split: tuple[int, int]

    @classmethod
    def of(cls, layers: list[Exl3Linear]) -> "Exl3Stack":
        """A copy of the layers' tensors in one piece (drop the layers afterwards to give their memory back)."""

        first = layers[0]
        same = lambda l: (l.k, l.n, l.bits, l.codebook, l.layout, l.words.shape, tuple(l.split)) == \
            (first.k, first.n, first.bits, first.codebook, first.layout, first.words.shape, tuple(first.split))
        if not 1 <= len(layers) <= 64 or not all(same(l) for l in layers):
            raise ValueError("a stack takes 1 to 64 layers of one shape, width, codebook, layout and K split")
        bias = None
        if any(l.bias is not None for l in layers):
            bias = torch.stack([l.bias if l.bias is not None else torch.zeros_like(first.svh) for l in layers])
        return cls(torch.stack([l.words for l in layers]), torch.stack([l.suh for l in layers]),
                   torch.stack([l.svh for l in layers]), bias, first.bits, first.codebook, first.k, first.n, first.layout,
                   first.split)

    def __post_init__(self) -> None:
        self.counters = torch.zeros((len(self), 8 * (self.n // 128) * COUNTER_STRIDE), dtype=torch.int32,
                                    device=self.words.device)

    def __len__(self) -> int:
        return int(self.words.shape[0])

    def layer(self, i: int) -> Exl3Linear:
        """Layer ``i`` as an ``Exl3Linear`` over the stack's memory."""

        return Exl3Linear(self.words[i], self.suh[i], self.svh[i], None if self.bias is None else self.bias[i],
                          self.bits, self.codebook, self.k, self.n, self.layout, self.split)

    def __call__(self, x: torch.Tensor, out: torch.Tensor | None = None, out_dtype: torch.dtype | None = None,
                 xh: torch.Tensor | None = None, z: torch.Tensor | None = None) -> torch.Tensor:
        """y [L, M, N] for x [M, K], M = 1..128.  ``xh`` (fp16, L * M * K values) and ``z`` (fp32, L * splits * M * N)
        are scratch, allocated here when not passed."""

        if x.dim() != 2 or x.shape[1] != self.k or not 1 <= x.shape[0] <= 128 or x.dtype not in _DTYPES:
            raise ValueError(f"x must be [1..128, {self.k}] fp16, bf16 or fp32, got {tuple(x.shape)} {x.dtype}")
        _lib.on_gpu(x)
        x = x.contiguous()
        count, m = len(self), int(x.shape[0])
        if out is None:
            out = x.new_empty((count, m, self.n), dtype=out_dtype or x.dtype)
        elif tuple(out.shape) != (count, m, self.n) or out.dtype not in _DTYPES or not out.is_contiguous() \
                or out.device != x.device:
            raise ValueError(f"out must be contiguous ({count}, {m}, {self.n}) fp16, bf16 or fp32 on x's device")
        sk, wk = self.split
        if xh is None:
            xh = x.new_empty((count, m, self.k), dtype=torch.float16)
        elif xh.dtype != torch.float16 or xh.numel() < count * m * self.k or not xh.is_contiguous() or xh.device != x.device:
            raise ValueError(f"xh must hold {count} x {m} x {self.k} fp16 values on x's device")
        if sk > 1 and z is None:
            z = x.new_empty((count * sk * m * self.n,), dtype=torch.float32)
        elif sk > 1 and (z.dtype != torch.float32 or z.numel() < count * sk * m * self.n or not z.is_contiguous()
                         or z.device != x.device):
            raise ValueError(f"z must hold {count} x {sk} x {m} x {self.n} fp32 values on x's device")
        stride_k, stride_nb = self.layer(0).strides
        _lib.call("tf_exl3_rot_in_stacked", _lib.ptr(x), _DTYPES[x.dtype], _lib.ptr(self.suh), _lib.ptr(xh), count, m,
                  self.k)
        _lib.call("tf_exl3_linear_stacked", _lib.ptr(xh), _lib.ptr(self.words), stride_k, stride_nb,
                  self.words.stride(0), _lib.ptr(self.svh), _lib.ptr(self.bias), _lib.ptr(out), _DTYPES[out.dtype],
                  _lib.ptr(z) if sk > 1 else None, _lib.ptr(self.counters), count, m, self.k, self.n, k2_of(self.bits),
                  CODEBOOK_IDS[self.codebook], sk, wk)
        return out


@dataclasses.dataclass
class Exl3MLP:
    """down(silu(gate(x)) * up(x)) in three launches: the input rotation for gate and up, their linear launch — whose
    workgroups also apply the SwiGLU and the down projection's input rotation to every column block they complete —
    and the down projection's linear launch.  The elementwise steps round as they would on tensors of ``mid_dtype``
    (gate and up's outputs, silu, the product); the bits are those of ``Exl3Stack`` + ``swiglu_rot_in`` + the down
    layer's linear launch."""

    gate_up: Exl3Stack            # gate first
    down: Exl3Linear

    @classmethod
    def of(cls, gate: Exl3Linear, up: Exl3Linear, down: Exl3Linear) -> "Exl3MLP":
        if down.k != gate.n or down.n != gate.k:
            raise ValueError(f"down must be {gate.n} -> {gate.k}, got {down.k} -> {down.n}")
        return cls(Exl3Stack.of([gate, up]), down)

    def scratch(self, m: int, device=None) -> dict[str, torch.Tensor]:
        """Buffers of a call on up to ``m`` rows: rotated inputs of both stages and the K splits' partial sums."""

        g, d = self.gate_up, self.down
        device = device or g.words.device
        floats = max(2 * g.split[0] * m * g.n, d.split[0] * m * d.n)
        return {"xh": torch.empty((2, m, g.k), dtype=torch.float16, device=device),
                "hh": torch.empty((m, g.n), dtype=torch.float16, device=device),
                "z": torch.empty((floats,), dtype=torch.float32, device=device)}

    def __call__(self, x: torch.Tensor, out: torch.Tensor | None = None, mid_dtype: torch.dtype = torch.float16,
                 scratch: dict[str, torch.Tensor] | None = None, mid: torch.Tensor | None = None) -> torch.Tensor:
        """y [M, D] for x [M, D], M = 1..128.  ``mid`` ([2, M, I] of ``mid_dtype``), when given, receives gate's and
        up's outputs as well."""

        g, d = self.gate_up, self.down
        if x.dim() != 2 or x.shape[1] != g.k or not 1 <= x.shape[0] <= 128 or x.dtype not in _DTYPES:
            raise ValueError(f"x must be [1..128, {g.k}] fp16, bf16 or fp32, got {tuple(x.shape)} {x.dtype}")
        if mid_dtype not in _DTYPES:
            raise ValueError("mid_dtype: fp16, bf16 or fp32")
        _lib.on_gpu(x)
        x = x.contiguous()
        m = int(x.shape[0])
        s = scratch or self.scratch(m, x.device)
        if s["xh"].numel() < 2 * m * g.k or s["hh"].numel() < m * g.n or \
                s["z"].numel() < max(2 * g.split[0] * m * g.n, d.split[0] * m * d.n):
            raise ValueError(f"the scratch does not hold {m} rows")
        if out is None:
            out = x.new_empty((m, d.n))
        elif tuple(out.shape) != (m, d.n) or out.dtype not in _DTYPES or not out.is_contiguous() or out.device != x.device:
            raise ValueError(f"out must be contiguous ({m}, {d.n}) fp16, bf16 or fp32 on x's device")
        if mid is not None and (tuple(mid.shape) != (2, m, g.n) or mid.dtype != mid_dtype or not mid.is_contiguous()
                                or mid.device != x.device):
            raise ValueError(f"mid must be contiguous (2, {m}, {g.n}) {mid_dtype} on x's device")
        (sk, wk), (dsk, dwk) = g.split, d.split
        stride_k, stride_nb = g.layer(0).strides
        _lib.call("tf_exl3_rot_in_stacked", _lib.ptr(x), _DTYPES[x.dtype], _lib.ptr(g.suh), _lib.ptr(s["xh"]), 2, m, g.k)
        _lib.call("tf_exl3_gate_up", _lib.ptr(s["xh"]), _lib.ptr(g.words), stride_k, stride_nb, g.words.stride(0),
                  _lib.ptr(g.svh), _lib.ptr(g.bias), _lib.ptr(mid), _DTYPES[mid_dtype], _lib.ptr(s["z"]),
                  _lib.ptr(g.counters), _lib.ptr(d.suh), _lib.ptr(s["hh"]), m, g.k, g.n, k2_of(g.bits),
                  CODEBOOK_IDS[g.codebook], sk, wk)
        stride_k, stride_nb = d.strides
        _lib.call("tf_exl3_linear", _lib.ptr(s["hh"]), _lib.ptr(d.words), stride_k, stride_nb, _lib.ptr(d.svh),
                  _lib.ptr(d.bias), _lib.ptr(out), _DTYPES[out.dtype], _lib.ptr(s["z"]) if dsk > 1 else None,
                  _lib.ptr(d.counters), m, d.k, d.n, d.k2, CODEBOOK_IDS[d.codebook], dsk, dwk)
        return out


def swiglu_rot_in(y: torch.Tensor, suh: torch.Tensor, xh: torch.Tensor | None = None) -> torch.Tensor:
    """The rotated input of a down projection from a stack's gate and up outputs ``y`` [2, M, I] (a launch of its own;
    ``Exl3MLP`` folds it into the stack's): fp16 [M, I]."""

    _lib.on_gpu(y, suh)
    if y.dim() != 3 or y.shape[0] != 2 or y.dtype not in _DTYPES or not y.is_contiguous() or y.shape[2] % 128:
        raise ValueError("y must be a contiguous [2, M, I] fp16, bf16 or fp32, I a multiple of 128")
    if suh.dtype != torch.float16 or tuple(suh.shape) != (y.shape[2],) or not suh.is_contiguous():
        raise ValueError(f"suh must be fp16 [{y.shape[2]}]")
    m, n = int(y.shape[1]), int(y.shape[2])
    if xh is None:
        xh = torch.empty((m, n), dtype=torch.float16, device=y.device)
    elif xh.dtype != torch.float16 or tuple(xh.shape) != (m, n) or not xh.is_contiguous() or xh.device != y.device:
        raise ValueError(f"xh must be a contiguous fp16 ({m}, {n}) on y's device")
    _lib.call("tf_exl3_swiglu_rot_in", _lib.ptr(y), _DTYPES[y.dtype], _lib.ptr(suh), _lib.ptr(xh), m, n)
    return xh


def unpack_gpu(trellis: torch.Tensor, codebook: str) -> torch.Tensor:
    """W_q [K, N] fp16 from trellis int16 [K/16, N/16, 16 * bits], decoded on the GPU from the stored order."""

    bits = fmt.bits_of(trellis.shape)
    fmt.check_pair(bits, codebook)
    words = trellis.cuda().contiguous().view(torch.int32)
    kt, nt, tile = words.shape
    return _decode(words, 16 * kt, 16 * nt, (nt * tile, 8 * tile), k2_of(bits), codebook, None)


unpack_cuda = unpack_gpu      # the name the reference's callers use (torch keeps the "cuda" device name on ROCm)
