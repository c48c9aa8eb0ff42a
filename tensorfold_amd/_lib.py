"""ctypes prototypes of ``include/tfmi.h`` and the call helper every op goes through."""

from __future__ import annotations

import contextlib
import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p
from functools import lru_cache
from pathlib import Path

import torch

from . import build

P, I, L, F = c_void_p, c_int, c_int64, c_float

# name -> argument types, in the header's order (the trailing stream included)
PROTOTYPES = {
    "tf_qmm_pack": [P, P, P, I, I, I, P, P, P, P],
    "tf_qmm_unpack": [P, P, P, I, I, I, P, P, P, P],
    "tf_group_sums": [P, L, I, I, I, P, P],
    "tf_qmm": [P, L, P, P, P, P, L, P, P, P, I, I, I, I, I, I, I, I, I, P],
    "tf_qmm_static": [P, L, P, P, P, P, L, P, I, I, I, I, I, I, I, P],
    "tf_qmm_group": [P, L, P, I, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, P],
    "tf_qmm_prefill": [P, L, P, P, P, P, I, I, I, I, I, I, I, P],
    "tf_quantize_rows": [P, L, I, I, I, P, P, P, P],
    "tf_qmm_prefill8": [P, P, P, P, P, P, P, I, I, I, I, I, I, P],
    "tf_experts_pack": [P, P, P, I, I, I, I, P, P],
    "tf_experts_unpack": [P, L, I, I, I, I, P, P, P, P],
    "tf_experts_plan": [P, L, I, I, P, P, P, P, P, P],
    "tf_experts_run": [I, I, P, L, I, P, I, I, P, P, P, P, I, F, L, P],
    "tf_experts_run_desc": [I, I, P, L, I, P, I, I, P, P, P, I, F, L, P],
    "tf_experts_prefill": [I, I, P, L, I, P, I, I, P, P, P, P, I, F, L, I, I, P],
    "tf_moe_route_up": [P, L, I, I, I, I, I, I, P, L, P, I, I, P, P, P, P, P, P, P, F, I, P, I, P],
    "tf_moe_down_combine": [I, P, I, I, P, I, I, P, P, P, P, P, I, P],
    "tf_moe_decode_sliced": [P, L, I, I, I, I, I, I, P, L, P, P, I, I, P, P, P, P, P, P, P, P, P, P, P, F, I, P],
    "tf_moe_route_decode": [P, L, I, I, I, I, P, P, P, P, P, P, P, I, P],
    "tf_moe_decode_experts": [I, I, P, L, I, I, P, P, I, I, P, P, P, P, P, P, P, P, P, F, I, P],
    "tf_moe_router": [P, L, P, P, I, I, I, P],
    "tf_moe_topk": [P, L, I, I, I, I, P, P, P],
    "tf_moe_combine": [P, I, P, P, I, I, I, P],
    "tf_exl3x_rot_in": [P, I, L, P, P, P, P, P, I, I, I, I, P],
    "tf_exl3x_grouped": [P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P],
    "tf_exl3x_gateup_epilogue": [P, P, P, P, P, P, I, I, I, I, F, I, P],
    "tf_exl3x_down_combine": [P, P, P, P, P, P, I, I, I, I, I, P],
    "tf_exl3x_plan_rot_in": [P, I, L, P, P, P, P, P, I, I, I, I, I, P, P, P, P],
    "tf_add_norm": [P, P, I, P, I, I, P, F, P, P, P, I, I, I, P],
    "tf_exl3_rot_in": [P, I, P, P, I, I, P],
    "tf_exl3_linear": [P, P, L, L, P, P, P, I, P, P, I, I, I, I, I, I, I, P],
    "tf_exl3_rot_in_stacked": [P, I, P, P, I, I, I, P],
    "tf_exl3_linear_stacked": [P, P, L, L, L, P, P, P, I, P, P, I, I, I, I, I, I, I, I, P],
    "tf_exl3_gate_up": [P, P, L, L, L, P, P, P, I, P, P, P, P, I, I, I, I, I, I, I, P],
    "tf_exl3_swiglu_rot_in": [P, I, P, P, I, I, P],
    "tf_exl3_unpack": [P, P, I, I, L, L, I, I, P],
    "tf_exl3_unpack_k8": [P, P, I, I, L, L, I, I, P],
    "tf_exl3_gemm": [P, P, P, P, P, I, L, I, I, I, P],
}


def _declare(so: ctypes.CDLL) -> ctypes.CDLL:
    so.tf_last_error.restype = ctypes.c_char_p
    so.tf_last_error.argtypes = []
    so.tf_version.restype = c_int
    so.tf_check_device.restype = c_int
    for name, args in PROTOTYPES.items():
        fn = getattr(so, name)
        fn.argtypes = args
        fn.restype = c_int
    return so


@lru_cache(maxsize=1)
def lib() -> ctypes.CDLL:
    return _declare(build.load())


_other: ctypes.CDLL | None = None


@contextlib.contextmanager
def through(path):
    """Route ``call`` through another build of the library (the timeline build) inside the block; yields it.  The
    other build must carry the digest of the sources beside it: one built before an entry point changed its
    arguments would be called with shifted pointers."""

    global _other
    if not Path(path).exists():
        raise RuntimeError(f"tensorfold-amd: {path} is missing (build.timeline_lib() builds the timeline library)")
    if build.built_id(Path(path)) != build.source_id():
        raise RuntimeError(f"tensorfold-amd: {path} was built from other sources than the ones beside it")
    _other = _declare(ctypes.CDLL(str(path)))
    try:
        yield _other
    finally:
        _other = None


@lru_cache(maxsize=1)
def _ready() -> bool:
    """First GPU call: the device must be the one the kernels were built for."""

    if not torch.cuda.is_available():
        raise RuntimeError("tensorfold-amd: its kernels run on an MI355X GPU only; none is available "
                           "(there is no CPU path)")
    so = lib()
    if so.tf_check_device():
        raise RuntimeError(so.tf_last_error().decode())
    return True


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def call(name: str, *args) -> None:
    """Run entry point ``name`` on the current stream; a non-zero status raises with the library's sentence."""

    _ready()
    so = _other or lib()
    if getattr(so, name)(*args, stream()):
        raise RuntimeError(so.tf_last_error().decode())


def on_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("tensorfold-amd: expected a GPU tensor (its kernels have no CPU path)")
