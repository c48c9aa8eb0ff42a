"""Build and load ``libtfmi.so``: hipcc for gfx950, nothing else (the counterpart of the reference's cuda/build.py).

The reference JIT-builds one pybind11 module per kernel family for whatever NVIDIA GPU is present and refuses GPUs
under compute capability 8.9 (cuda/build.py:20-69).  Here one shared library with a C ABI is compiled ahead of
time, in the tree, for the one target this package supports, and a GPU that is not gfx950 is refused by name.
"""

from __future__ import annotations

import ctypes
import shutil
import subprocess
import sys
from functools import lru_cache
from pathlib import Path

ARCH = "gfx950"
HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libtfmi.so"
TIMELINE_LIB = HERE / "libtfmi_timeline.so"      # the same kernels with per-workgroup timestamps (see compile)
SOURCES = ("api.hip", "pack.hip", "decode.hip", "fused.hip", "route.hip", "norm.hip", "prefill.hip", "prefill8.hip", "exl3.hip", "exl3_experts.hip")
# packed-fp32 VALU forms are switched off for the device pass (the host pass warns that it does not know the feature)
FLAGS = ("-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")


def say(text: str) -> None:
    print(f"[tensorfold-amd] {text}", file=sys.stderr, flush=True)


def hipcc() -> str | None:
    return shutil.which("hipcc") or (str(Path("/opt/rocm/bin/hipcc")) if Path("/opt/rocm/bin/hipcc").exists() else None)


def source_id() -> str:
    """16 hex digits over every file the library is built from and the compiler flags."""

    import hashlib

    h = hashlib.sha256(" ".join(FLAGS).encode())
    for path in [CSRC / s for s in SOURCES] + sorted(CSRC.glob("*.h")) + [HERE.parent / "include" / "tfmi.h"]:
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()[:16]


def built_id(path: Path = LIB) -> str | None:
    """The digest a library file carries (``tf_build_id``), read from the file without loading it."""

    if not path.exists():
        return None
    blob, mark = path.read_bytes(), b"TFMI_BUILD_ID="
    at = blob.find(mark)
    return None if at < 0 else blob[at + len(mark):at + len(mark) + 16].decode(errors="replace")


def stale() -> bool:
    """Whether the library is missing or was built from other sources than the ones beside it."""

    if LIB.exists() and not (CSRC / SOURCES[0]).exists():
        return False                       # a library shipped without its sources is taken as it is
    return built_id() != source_id()


def timeline_lib() -> Path:
    """``libtfmi_timeline.so`` for the sources beside it: built on request only (``bench_configs.py timeline*`` asks),
    and again whenever its digest is not the sources'.  A timeline build of other sources is never loaded: its entry
    points may take other arguments than the prototypes of this tree."""

    if built_id(TIMELINE_LIB) != source_id():
        if hipcc() is None:
            raise RuntimeError(f"tensorfold-amd: {TIMELINE_LIB} is missing or was built from other sources, and there "
                               "is no hipcc to build it")
        compile(timeline=True)
    return TIMELINE_LIB


def compile(verbose: bool = False, timeline: bool = False) -> Path:
    """Compile every kernel for gfx950 into ``libtfmi.so`` (cross-compiles without a GPU): one hipcc per source,
    side by side, then a link.  ``timeline``: the same sources with -DTF_TIMELINE into ``libtfmi_timeline.so``, whose
    decode expert kernels note per-workgroup timestamps (an instrument: only ``timeline_lib`` builds it)."""

    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    cc = hipcc()
    if cc is None:
        raise RuntimeError("tensorfold-amd: hipcc was not found; ROCm's compiler is needed to build libtfmi.so")
    target = TIMELINE_LIB if timeline else LIB
    say(f"building {target.name} for {ARCH} (about half a minute)")
    noise = "packed-fp32-ops"

    def run(cmd: list[str]) -> str:
        done = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(line for line in done.stderr.splitlines() if noise not in line)
        if done.returncode:
            raise RuntimeError(f"tensorfold-amd: hipcc failed:\n{err}")
        return err

    compile_flags = [f for f in FLAGS if f != "-shared"] + [f'-DTF_BUILD_ID="{source_id()}"']
    if timeline:
        compile_flags.append("-DTF_TIMELINE")
    with tempfile.TemporaryDirectory(prefix="tfmi-build-") as tmp:
        objects = [str(Path(tmp) / (Path(s).stem + ".o")) for s in SOURCES]
        with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
            logs = list(pool.map(lambda so: run([cc, *compile_flags, "-c", str(CSRC / so[0]), "-o", so[1]]),
                                 zip(SOURCES, objects)))
        logs.append(run([cc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(target), *objects]))
    if verbose:
        for text in logs:
            if text:
                say(text)
    return target


@lru_cache(maxsize=1)
def load() -> ctypes.CDLL:
    """The library, built first if it is missing or out of date (its digest differs from the sources') and hipcc is
    here; a missing or stale library never falls back to anything."""

    if stale():
        if hipcc() is None:
            what = "is missing" if not LIB.exists() else "was built from other sources than the ones beside it"
            raise RuntimeError(f"tensorfold-amd: {LIB} {what} and there is no hipcc to build it; "
                               "run `python -c 'import __graft_entry__ as g; g.build()'` where ROCm is installed")
        compile()
    return ctypes.CDLL(str(LIB))


def refuse_other_gpu() -> None:
    """With a GPU present, refuse by name one the kernels were not built for (cuda/build.py:35-46 in spirit)."""

    import torch

    if not torch.cuda.is_available():
        return
    lib = load()
    lib.tf_last_error.restype = ctypes.c_char_p
    if lib.tf_check_device():
        raise ValueError(lib.tf_last_error().decode())
