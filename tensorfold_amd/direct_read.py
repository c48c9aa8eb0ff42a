"""Checkpoint bytes from disk into host memory or onto the GPU: what feeds ``qmm.pack``, ``experts.make`` and
``Exl3Linear.from_tensors``.

The interface is the reference's reader (src/tensorfold/cuda/direct_read.py:28-199: ``Reader.read``, ``read_header``,
``SafeTensors``, ``ReadAhead``, ``in_background`` / ``wait_all``); how the bytes travel is this package's.  A safetensors
file is a little-endian u64 header length, a JSON header (name -> dtype, shape, byte range) and the tensors' bytes
back to back.  An MI355X holds 288 GB, so a checkpoint is read once and whole, and the page cache only gets in the
way: a file is opened with O_DIRECT and walked in block-aligned pieces (``pieces``).  On these machines a direct
read cannot land in page-locked memory (the kernel answers EFAULT: the driver's page-locked mappings are not ones
block I/O can pin, and registering ordinary memory after the fact is refused too), so a piece is read into an
ordinary block-aligned buffer and copied by the CPU into page-locked staging that was allocated as such.  For the
GPU a ring of ``RING`` staging pieces takes turns: one uploads on the caller's stream while the next piece is read
and copied.  A file system that refuses O_DIRECT (tmpfs, some overlays) answers EINVAL once; from then on the reader
goes through the page cache.
"""

from __future__ import annotations

import errno
import json
import os
import pathlib
import struct
from concurrent.futures import Future, ThreadPoolExecutor

import torch

PIECE = 64 << 20      # bytes one direct read asks for, and the size of a staging piece (a multiple of ALIGN)
ALIGN = 4096          # O_DIRECT wants the file offset, the length and the buffer address on this boundary
RING = 2              # staging pieces an upload cycles through

_NAMES = "BOOL:bool U8:uint8 I8:int8 U16:uint16 I16:int16 U32:uint32 I32:int32 U64:uint64 I64:int64 " \
         "F16:float16 BF16:bfloat16 F32:float32 F64:float64 F8_E4M3:float8_e4m3fn F8_E5M2:float8_e5m2"
DTYPES = {theirs: getattr(torch, ours) for theirs, ours in (pair.split(":") for pair in _NAMES.split())}


def pieces(offset: int, n: int, size: int):
    """File bytes [offset, offset + n) of a file of ``size`` bytes as block-aligned reads of at most PIECE bytes:
    yields (lo, hi, a, b) — read blocks [lo, hi); file bytes [a, b) of them are wanted.  The last block of a file may
    be short on disk; its read is still asked for whole."""

    end, last_block = offset + n, -(-size // ALIGN) * ALIGN
    lo = offset - offset % ALIGN
    while lo < end:
        hi = min(lo + PIECE, -(-end // ALIGN) * ALIGN, last_block)
        yield lo, hi, max(lo, offset), min(hi, end)
        lo = hi


def _block_aligned(n: int) -> torch.Tensor:
    """``n`` bytes of ordinary memory that start on an ALIGN boundary (the allocator does not promise one)."""

    block = torch.empty((n + ALIGN,), dtype=torch.uint8)
    lead = -block.data_ptr() % ALIGN
    return block[lead:lead + n]


def _drop_pinned_cache() -> None:
    """Give freed page-locked memory back to the system, where this torch can (it otherwise stays cached)."""

    release = getattr(torch._C, "_host_emptyCache", None)
    if release is not None:
        release()


class _Direct:
    """One file open with O_DIRECT."""

    def __init__(self, path, offset: int, n: int) -> None:
        self.path, self.fd = path, os.open(path, os.O_RDONLY | os.O_DIRECT)
        self.size = os.fstat(self.fd).st_size
        if offset + n > self.size:
            os.close(self.fd)
            raise IOError(f"short read of {path}: bytes {offset}-{offset + n} lie past its end ({self.size})")

    def fill(self, into: torch.Tensor, lo: int, need: int) -> None:
        """Read the blocks at ``lo`` into ``into`` (as long as the blocks) until ``need`` bytes are there."""

        view, have = memoryview(into.numpy()), 0
        while have < need:
            got = os.preadv(self.fd, [view[have:]], lo + have)
            if got <= 0:
                raise IOError(f"short read of {self.path} at byte {lo + have}")
            have += got


class Reader:
    """Byte ranges of files as new uint8 tensors.  ``direct`` turns False for good the first time O_DIRECT is refused."""

    def __init__(self) -> None:
        self.direct = hasattr(os, "O_DIRECT")
        self.ring: list[list] = []            # [page-locked piece, event of its last upload or None] per slot
        self.turn = 0
        self.landing: torch.Tensor | None = None      # where an upload's direct reads land before they are staged

    def read(self, path, offset: int, n: int, device="cpu", *, pinned: bool = False) -> torch.Tensor:
        """Bytes [offset, offset + n) of ``path`` on ``device``.  ``pinned`` asks for page-locked host memory (direct
        reads only), for an upload that does not block."""

        device = torch.device(device)
        if n == 0:
            return torch.empty((0,), dtype=torch.uint8, device=device)
        if self.direct:
            try:
                f = _Direct(path, offset, n)
                try:
                    return self._onto_gpu(f, offset, n, device) if device.type == "cuda" else self._onto_host(f, offset, n, pinned)
                finally:
                    os.close(f.fd)
            except OSError as refused:
                if refused.errno != errno.EINVAL:
                    raise
                self.direct = False
        out = torch.empty((n,), dtype=torch.uint8)
        view = memoryview(out.numpy())
        with open(path, "rb", buffering=0) as f:                  # through the page cache, a piece a call
            f.seek(offset)
            have = 0
            while have < n:
                got = f.readinto(view[have:min(n, have + PIECE)])
                if not got:
                    raise IOError(f"short read of {path} at byte {offset + have}")
                have += got
        return out.to(device) if device.type == "cuda" else out

    @staticmethod
    def _onto_host(f: _Direct, offset: int, n: int, pinned: bool) -> torch.Tensor:
        """All pieces into one buffer, side by side as in the file."""

        cuts = list(pieces(offset, n, f.size))
        base = cuts[0][0]
        span = _block_aligned(cuts[-1][1] - base)
        for lo, hi, _, b in cuts:
            f.fill(span[lo - base:hi - base], lo, b - lo)
        out = span[offset - base:offset - base + n]
        if pinned:
            return torch.empty((n,), dtype=torch.uint8, pin_memory=True).copy_(out)
        return out if out.data_ptr() % 8 == 0 else out.clone()      # a view as a wider dtype needs an aligned start

    def _onto_gpu(self, f: _Direct, offset: int, n: int, device: torch.device) -> torch.Tensor:
        """Piece by piece: a direct read lands, its wanted bytes are staged in a ring slot whose last upload is done,
        and the slot is uploaded while the next piece is read."""

        if self.landing is None or self.landing.numel() < PIECE:
            self.landing = _block_aligned(PIECE)
        while len(self.ring) < RING:
            self.ring.append([torch.empty((PIECE,), dtype=torch.uint8, pin_memory=True), None])
        out = torch.empty((n,), dtype=torch.uint8, device=device)
        stream = torch.cuda.current_stream(device)
        for lo, hi, a, b in pieces(offset, n, f.size):
            f.fill(self.landing[:hi - lo], lo, b - lo)
            slot = self.ring[self.turn % len(self.ring)]
            self.turn += 1
            if slot[1] is not None:
                slot[1].synchronize()
            staged = slot[0][:b - a].copy_(self.landing[a - lo:b - lo])
            out[a - offset:b - offset].copy_(staged, non_blocking=True)
            slot[1] = torch.cuda.Event()
            slot[1].record(stream)
        return out

    def close(self) -> None:
        """Wait for the uploads in flight and hand the staging pieces back to the system."""

        for _, sent in self.ring:
            if sent is not None:
                sent.synchronize()
        self.ring.clear()
        self.landing = None
        _drop_pinned_cache()


def read_header(path) -> tuple[int, dict]:
    """(file offset of the first tensor byte, the JSON header) of a safetensors file."""

    with open(path, "rb") as f:
        (length,) = struct.unpack("<Q", f.read(8))
        return 8 + length, json.loads(f.read(length))


class SafeTensors:
    """Tensors by name over several safetensors files (of a name in two files the later file's wins)."""

    def __init__(self, files, reader: Reader | None = None) -> None:
        self.reader = reader if reader is not None else Reader()
        self.where: dict[str, tuple] = {}       # name -> (file, first byte, bytes, dtype name, shape)
        for path in map(pathlib.Path, files):
            start, header = read_header(path)
            header.pop("__metadata__", None)
            for name, entry in header.items():
                first, end = entry["data_offsets"]
                self.where[name] = (path, start + first, end - first, entry["dtype"], [int(v) for v in entry["shape"]])

    def keys(self) -> list[str]:
        return list(self.where)

    def __contains__(self, name: str) -> bool:
        return name in self.where

    def get(self, name: str, device="cpu") -> torch.Tensor:
        path, first, nbytes, dtype, shape = self.where[name]
        if dtype not in DTYPES:
            raise ValueError(f"{name}: no torch dtype for safetensors' {dtype}")
        return self.reader.read(path, first, nbytes, device).view(DTYPES[dtype]).reshape(shape)

    def close(self) -> None:
        self.reader.close()


def _runs(items: list, run: int, gap: int) -> list[list]:
    """Items of one file (key, path, first byte, end byte, meta) sorted by position and cut into runs: a new run
    starts where the next item lies more than ``gap`` past the run's end or would stretch the run over ``run`` bytes."""

    out: list[list] = []
    end = 0
    for item in sorted(items, key=lambda it: it[2]):
        if out and item[2] - end <= gap and item[3] - out[-1][0][2] <= run:
            out[-1].append(item)
            end = max(end, item[3])
        else:
            out.append([item])
            end = item[3]
    return out


class _Run:
    """One read of neighbouring tensors: what it covers, and once read, its tensors and (on a GPU) the upload's event."""

    def __init__(self, path: str, items: list) -> None:
        self.path, self.items = path, items
        self.lo, self.hi = items[0][2], max(item[3] for item in items)
        self.tensors: dict = {}
        self.sent = None
        self.job: Future | None = None

    def read(self, reader: Reader, device, stream, cut) -> "_Run":
        slices = lambda raw: {key: cut(raw[a - self.lo:b - self.lo], meta) for key, _, a, b, meta in self.items}
        if device is None:
            self.tensors = slices(reader.read(self.path, self.lo, self.hi - self.lo))
            return self
        host = reader.read(self.path, self.lo, self.hi - self.lo, pinned=True)
        with torch.cuda.device(device), torch.cuda.stream(stream):
            self.tensors = slices(host.to(device, non_blocking=True))
            self.sent = torch.cuda.Event()
            self.sent.record(stream)
        return self


class ReadAhead:
    """Tensors requested before they are needed: worker threads read runs of neighbouring tensors with one read each;
    for a GPU each run is uploaded once, on a side stream of default priority, and cut up there."""

    def __init__(self, reader: Reader | None = None, threads: int = 8, run: int = 128 << 20, gap: int = 1 << 20) -> None:
        self.reader = reader if reader is not None else Reader()
        self.threads, self.run, self.gap = threads, run, gap
        self.ahead: dict = {}               # key -> the _Run that holds (or will hold) its tensor
        self.pool: ThreadPoolExecutor | None = None
        self.stream: torch.cuda.Stream | None = None

    def queue(self, items, device=None, cut=None) -> None:
        """Start on the ``items`` (key, path, first byte, end byte, meta) that are not queued already.  ``cut(raw,
        meta)`` makes an item's tensor out of its slice of the run's bytes (a copy of the slice when not given)."""

        cut = cut if cut is not None else (lambda raw, meta: raw.clone())
        device = torch.device(device) if device is not None and torch.device(device).type == "cuda" else None
        if self.pool is None:
            self.pool = ThreadPoolExecutor(self.threads, thread_name_prefix="read-ahead")
        if device is not None and self.stream is None:
            self.stream = torch.cuda.Stream(device)
        per_file: dict[str, list] = {}
        for item in items:
            if item[0] not in self.ahead:
                per_file.setdefault(str(item[1]), []).append(item)
        for path, mine in per_file.items():
            for group in _runs(mine, self.run, self.gap):
                one = _Run(path, group)
                one.job = self.pool.submit(one.read, self.reader, device, self.stream, cut)
                self.ahead.update((item[0], one) for item in group)

    def take(self, key):
        """The tensor queued under ``key`` (waits for its read; on a GPU the current stream then waits for the
        upload), or None when nothing is queued under it."""

        one = self.ahead.pop(key, None)
        if one is None:
            return None
        t = one.job.result().tensors.pop(key)
        if one.sent is not None:
            stream = torch.cuda.current_stream(t.device)
            stream.wait_event(one.sent)
            t.record_stream(stream)
        return t

    def drop(self, keys) -> None:
        """Forget queued tensors that nobody will take; their memory goes once their run has been read."""

        for key in keys:
            one = self.ahead.pop(key, None)
            if one is not None:
                one.job.add_done_callback(lambda _, run=one, k=key: run.tensors.pop(k, None))

    def close(self) -> None:
        """Cancel what has not started, wait for what has, and give the uploads' page-locked memory back."""

        self.ahead.clear()
        if self.pool is not None:
            self.pool.shutdown(wait=True, cancel_futures=True)
            self.pool = None
        if self.stream is not None:
            self.stream.synchronize()
            self.stream = None
            _drop_pinned_cache()


def in_background(job, futures: list) -> None:
    """Run ``job`` on a thread of its own; its future is appended to ``futures`` for ``wait_all``."""

    pool = ThreadPoolExecutor(1, thread_name_prefix="background-read")
    futures.append(pool.submit(job))
    pool.shutdown(wait=False)


def wait_all(futures: list) -> None:
    """Wait until none of ``futures`` is running, empty the list, then raise the first error among them."""

    done = [f.exception() for f in futures]
    del futures[:]
    for error in done:
        if error is not None:
            raise error
