"""ctypes binding of the C oracle (oracle/orc.c).  Test infrastructure only."""

from __future__ import annotations

import ctypes
import subprocess
from functools import lru_cache
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "liborc.so"


def build(force: bool = False) -> Path:
    """Compile orc.c with gcc (``make -C oracle``); rebuilt when the source is newer than the library."""

    src = HERE / "orc.c"
    if force or not LIB.exists() or LIB.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(HERE), "-B", "liborc.so"], check=True, capture_output=True)
    return LIB


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


@lru_cache(maxsize=1)
def lib() -> ctypes.CDLL:
    if not LIB.exists():
        build()
    so = ctypes.CDLL(str(LIB))
    so.orc_threads.restype = ctypes.c_int
    so.orc_double_to_half.restype = ctypes.c_uint16
    so.orc_double_to_half.argtypes = [ctypes.c_double]
    so.orc_half_to_double.restype = ctypes.c_double
    so.orc_half_to_double.argtypes = [ctypes.c_uint16]
    return so


def threads() -> int:
    return int(lib().orc_threads())


def set_threads(n: int) -> None:
    lib().orc_set_threads(ctypes.c_int(n))


def _u16(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint16)


def _u32(a) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint32)


def affine_dequant(words, scales_bits, biases_bits, gs: int) -> np.ndarray:
    words = _u32(words)
    n, k = int(np.prod(words.shape[:-1])), words.shape[-1] * 8
    out = np.empty((*words.shape[:-1], k), dtype=np.float32)
    lib().orc_affine_dequant(_p(words), _p(_u16(scales_bits)), _p(_u16(biases_bits)), ctypes.c_int64(n),
                             ctypes.c_int(k), ctypes.c_int(gs), _p(out))
    return out


def affine_linear(x_bits, words, scales_bits, biases_bits, gs: int, *, prefill: bool | int = False) -> np.ndarray:
    """fp32 [M, N]; x, scales, biases as bf16 bit patterns (uint16).  ``prefill`` 1 (True): every weight rounded once as
    this build's fp16 prompt form does; 2: as the reference's bf16 prompt form does; 0: not at all."""

    x_bits, words = _u16(x_bits), _u32(words)
    m, k = x_bits.shape
    n = words.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    lib().orc_affine_linear(_p(x_bits), ctypes.c_int(m), _p(words), _p(_u16(scales_bits)), _p(_u16(biases_bits)),
                            ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(gs), ctypes.c_int(int(prefill)), _p(y))
    return y


def moe_layer(x_bits, picks, wts, gate, up, down, gs: int, *, limit: float = 0.0, prefill: bool = False,
              want_pairs: bool = False):
    """The whole routed layer on the CPU.  gate/up/down = (words [E, n, k/8], scale bits, bias bits); gate may be None.
    Returns out bf16 bits [rows, d] (and act bits [P, ni], y fp32 [P, d] with ``want_pairs``)."""

    x_bits = _u16(x_bits)
    rows, d = x_bits.shape
    picks = np.ascontiguousarray(picks, dtype=np.int32)
    wts = np.ascontiguousarray(wts, dtype=np.float32)
    slots = picks.shape[1]
    ni = up[0].shape[1]
    out = np.empty((rows, d), dtype=np.uint16)
    act = np.empty((rows * slots, ni), dtype=np.uint16) if want_pairs else None
    y = np.empty((rows * slots, d), dtype=np.float32) if want_pairs else None
    g = (None, None, None) if gate is None else (_u32(gate[0]), _u16(gate[1]), _u16(gate[2]))
    u = (_u32(up[0]), _u16(up[1]), _u16(up[2]))
    dn = (_u32(down[0]), _u16(down[1]), _u16(down[2]))
    lib().orc_moe_layer(_p(x_bits), ctypes.c_int(rows), ctypes.c_int(d), _p(picks), _p(wts), ctypes.c_int(slots),
                        _p(g[0]), _p(g[1]), _p(g[2]), _p(u[0]), _p(u[1]), _p(u[2]), _p(dn[0]), _p(dn[1]), _p(dn[2]),
                        ctypes.c_int(ni), ctypes.c_int(gs), ctypes.c_float(limit), ctypes.c_int(int(prefill)),
                        _p(act), _p(y), _p(out))
    return (out, act, y) if want_pairs else out


def exl3_codebook(cb: int) -> np.ndarray:
    table = np.empty(65536, dtype=np.uint16)
    lib().orc_exl3_codebook(ctypes.c_int(cb), _p(table))
    return table.view(np.float16)


def exl3_unpack(trellis, k2: int, cb: int) -> np.ndarray:
    t = np.ascontiguousarray(trellis, dtype=np.int16)
    kt, nt = t.shape[:2]
    w = np.empty((16 * kt, 16 * nt), dtype=np.uint16)
    lib().orc_exl3_unpack(_p(t), ctypes.c_int(kt), ctypes.c_int(nt), ctypes.c_int(k2), ctypes.c_int(cb), _p(w))
    return w.view(np.float16)


def exl3_linear(x_half, trellis, suh, svh, k2: int, cb: int, bias=None) -> np.ndarray:
    """fp32 [M, N] = ((((x * suh) H) W_q) H) * svh + bias with the rotated input rounded to fp16."""

    x = np.ascontiguousarray(x_half, dtype=np.float16)
    t = np.ascontiguousarray(trellis, dtype=np.int16)
    m, k = x.shape
    n = 16 * t.shape[1]
    y = np.empty((m, n), dtype=np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16)
    lib().orc_exl3_linear(_p(x), ctypes.c_int(m), _p(t), _p(np.ascontiguousarray(suh, dtype=np.float16)),
                          _p(np.ascontiguousarray(svh, dtype=np.float16)), _p(b), ctypes.c_int(k), ctypes.c_int(n),
                          ctypes.c_int(k2), ctypes.c_int(cb), _p(y))
    return y
