"""Conversions between torch tensors and the oracle's numpy conventions, and the error measures the tests state."""

from __future__ import annotations

import json
import struct

import numpy as np
import torch

SAFETENSORS_NAMES = {torch.int32: "I32", torch.uint32: "U32", torch.bfloat16: "BF16", torch.float16: "F16",
                     torch.uint8: "U8", torch.bool: "BOOL", torch.float32: "F32", torch.int16: "I16",
                     torch.float64: "F64", torch.int64: "I64"}


def write_safetensors(path, tensors: dict[str, torch.Tensor], shift: int = 0) -> None:
    """A safetensors file written by hand (u64 header length, JSON header, the tensors' bytes back to back).  A
    0-dimensional tensor is a scalar (shape []).  ``shift`` pads the header so that the data starts that many bytes
    past a 4 KiB edge."""

    header, blobs, at = {}, [], 0
    for name, t in tensors.items():
        raw = t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": SAFETENSORS_NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    text = json.dumps(header).encode()
    if shift:
        text += b" " * ((shift - 8 - len(text)) % 4096)
    path.write_bytes(struct.pack("<Q", len(text)) + text + b"".join(blobs))


def f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def bits16(t: torch.Tensor) -> np.ndarray:
    """bf16 / fp16 tensor -> its bit patterns as uint16."""

    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def u32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def rel_l2(got, want) -> float:
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def max_abs(got, want) -> float:
    return float(np.abs(np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)).max())
