"""The checkpoint reader on the host.  Whichever way the bytes travel — O_DIRECT blocks, the page cache, runs read
ahead on threads — a tensor read by name must equal what the ``safetensors`` package itself returns for the file.
(The properties the reference's tests/test_direct_read.py asks of its reader.)"""

import errno
import json
import os
import struct

import numpy as np
import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from tensorfold_amd import direct_read as dr
from tests.helpers import write_safetensors

WAYS = ("o_direct", "page cache")


def bag() -> dict[str, torch.Tensor]:
    """Tensors of every dtype a checkpoint of this path holds; sizes that straddle blocks and pieces; one empty; the
    last one ends the file, so the final block read is short."""

    rng = np.random.default_rng(11)
    return {
        "layer.weight": torch.from_numpy(rng.integers(0, 2 ** 32, (41, 13), dtype=np.uint32)),
        "layer.scales": torch.from_numpy(rng.standard_normal((41, 3)).astype(np.float32)).to(torch.bfloat16),
        "layer.signed": torch.from_numpy(rng.integers(-2 ** 31, 2 ** 31, (7, 9), dtype=np.int64).astype(np.int32)),
        "layer.trellis": torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, (8, 8, 48), dtype=np.int16)),
        "layer.suh": torch.from_numpy(rng.standard_normal(128).astype(np.float16)),
        "bytes.odd": torch.from_numpy(rng.integers(0, 256, 12289, dtype=np.uint8)),
        "flags": torch.from_numpy(rng.integers(0, 2, 17).astype(bool)),
        "wide": torch.from_numpy(rng.standard_normal((1200, 31)).astype(np.float32)),
        "nothing": torch.zeros((0, 8)),
        "doubles": torch.from_numpy(rng.standard_normal(5)),
        "tail": torch.from_numpy(rng.standard_normal(3).astype(np.float32)),
    }


def raw(t: torch.Tensor) -> bytes:
    return t.contiguous().view(torch.uint8).numpy().tobytes()


def check(got: torch.Tensor, want: torch.Tensor, name: str) -> None:
    assert (got.dtype, got.shape, raw(got)) == (want.dtype, want.shape, raw(want)), name


@pytest.fixture
def stored(tmp_path, monkeypatch):
    """The bag saved by the safetensors package, read in pieces of two blocks so that a tensor takes several reads."""

    monkeypatch.setattr(dr, "PIECE", 2 * dr.ALIGN)
    path = tmp_path / "model.safetensors"
    save_file(bag(), str(path))
    return path


def opened(path, way: str) -> dr.SafeTensors:
    files = dr.SafeTensors([path])
    if way == "page cache":
        files.reader.direct = False
    return files


@pytest.mark.parametrize("way", WAYS)
def test_any_range_of_a_file_reads_back(tmp_path, monkeypatch, way):
    """Drawn (offset, length) pairs against the file's own bytes, pieces of one, two and sixteen blocks."""

    rng = np.random.default_rng(3)
    blob = rng.integers(0, 256, 150_003, dtype=np.uint8)
    path = tmp_path / "blob.bin"
    path.write_bytes(blob.tobytes())
    for blocks in (1, 2, 16):
        monkeypatch.setattr(dr, "PIECE", blocks * dr.ALIGN)
        reader = dr.Reader()
        reader.direct = reader.direct and way == "o_direct"
        edges = [0, 1, 4095, 4096, 4097, 8192, 150_002, 150_003]
        starts = list(rng.integers(0, blob.size, 20)) + edges[:-1]
        for first in starts:
            for n in (int(rng.integers(0, blob.size - first + 1)), min(4096, blob.size - first), blob.size - first):
                got = reader.read(path, int(first), n)
                assert got.dtype == torch.uint8 and np.array_equal(got.numpy(), blob[first:first + n]), (blocks, first, n)
        with pytest.raises(IOError, match="short read"):
            reader.read(path, blob.size - 10, 11)


def test_pieces_cover_a_range_once_in_whole_blocks(monkeypatch):
    monkeypatch.setattr(dr, "PIECE", 2 * dr.ALIGN)
    for offset, n, size in ((0, 1, 1), (13, 30_000, 40_000), (8192, 8192, 16384), (4095, 2, 9000), (20_000, 5, 20_005)):
        cuts = list(dr.pieces(offset, n, size))
        assert all(lo % dr.ALIGN == 0 and hi % dr.ALIGN == 0 and 0 < hi - lo <= dr.PIECE for lo, hi, _, _ in cuts)
        assert all(lo <= a < b <= hi for lo, hi, a, b in cuts)
        assert [c[0] for c in cuts[1:]] == [c[1] for c in cuts[:-1]]              # block ranges follow one another
        assert cuts[0][2] == offset and cuts[-1][3] == offset + n
        assert [c[2] for c in cuts[1:]] == [c[3] for c in cuts[:-1]]              # and so do the wanted bytes


@pytest.mark.parametrize("way", WAYS)
def test_every_tensor_equals_the_safetensors_package(stored, way):
    files = opened(stored, way)
    with safe_open(str(stored), framework="pt") as theirs:
        assert sorted(files.keys()) == sorted(theirs.keys()) and "wide" in files and "narrow" not in files
        for name in theirs.keys():
            check(files.get(name), theirs.get_tensor(name), name)
    files.close()
    if way == "o_direct" and not files.reader.direct:
        pytest.skip("this file system refuses O_DIRECT; the page-cache path was checked instead")


def test_a_later_file_wins_a_name(tmp_path):
    write_safetensors(tmp_path / "a.safetensors", {"x": torch.zeros(4), "y": torch.ones(2)})
    write_safetensors(tmp_path / "b.safetensors", {"x": torch.full((3,), 7.0)})
    files = dr.SafeTensors([tmp_path / "a.safetensors", tmp_path / "b.safetensors"])
    assert files.get("x").tolist() == [7.0] * 3 and files.get("y").tolist() == [1.0, 1.0]


@pytest.mark.parametrize("way", WAYS)
def test_tensors_that_start_on_odd_bytes(tmp_path, monkeypatch, way):
    """Data 13 bytes past a block edge: no tensor starts aligned, and each still comes back viewable as its dtype."""

    monkeypatch.setattr(dr, "PIECE", 2 * dr.ALIGN)
    path = tmp_path / "model.safetensors"
    write_safetensors(path, bag(), shift=13)
    assert dr.read_header(path)[0] % 4096 == 13
    files = opened(path, way)
    for name, t in bag().items():
        check(files.get(name), t, name)


def test_unknown_dtypes_are_refused(tmp_path):
    path = tmp_path / "model.safetensors"
    text = json.dumps({"x": {"dtype": "F4", "shape": [2], "data_offsets": [0, 1]}}).encode()
    path.write_bytes(struct.pack("<Q", len(text)) + text + b"\0")
    with pytest.raises(ValueError, match="F4"):
        dr.SafeTensors([path]).get("x")


@pytest.mark.parametrize("way", WAYS)
def test_a_cut_off_file_is_a_short_read(stored, way):
    files = opened(stored, way)
    first = files.where["wide"][1]
    with open(stored, "r+b") as f:
        f.truncate((first + 5 * 4096) // 4096 * 4096)          # on a block edge inside "wide"
    with pytest.raises(IOError, match="short read"):
        files.get("wide")
    before = min((name for name in files.keys() if files.where[name][2]), key=lambda name: files.where[name][1])
    assert before != "wide"
    check(files.get(before), bag()[before], "what lies before the cut still reads")


def test_a_refusal_of_o_direct_is_remembered(stored, monkeypatch):
    if not hasattr(os, "O_DIRECT"):
        pytest.skip("this platform has no O_DIRECT")
    plain_open, asked = os.open, []

    def refusing(p, flags, *rest):
        if flags & os.O_DIRECT:
            asked.append(p)
            raise OSError(errno.EINVAL, "no O_DIRECT here")
        return plain_open(p, flags, *rest)

    monkeypatch.setattr(os, "open", refusing)
    files = dr.SafeTensors([stored])
    check(files.get("wide"), bag()["wide"], "wide")
    assert files.reader.direct is False and len(asked) == 1
    check(files.get("tail"), bag()["tail"], "tail")
    assert len(asked) == 1                                      # not asked again


def test_other_errors_are_not_swallowed(tmp_path):
    with pytest.raises(OSError):
        dr.Reader().read(tmp_path / "absent.safetensors", 0, 16)


def test_runs_join_neighbours_only():
    item = lambda key, a, b: (key, "f", a, b, None)
    items = [item("c", 5000, 6000), item("a", 0, 1000), item("b", 1000, 3000), item("d", 90000, 90010)]
    keys = lambda runs: [[it[0] for it in run] for run in runs]
    assert keys(dr._runs(items, run=1 << 20, gap=4096)) == [["a", "b", "c"], ["d"]]
    assert keys(dr._runs(items, run=1 << 20, gap=0)) == [["a", "b"], ["c"], ["d"]]
    assert keys(dr._runs(items, run=2500, gap=4096)) == [["a"], ["b"], ["c"], ["d"]]      # a and b together span 3,000


@pytest.mark.parametrize("run,gap", [(1 << 20, 1 << 20), (4096, 0)])          # one read for all; about one a tensor
def test_reading_ahead_gives_the_same_tensors(stored, run, gap):
    files = dr.SafeTensors([stored])
    ahead = dr.ReadAhead(files.reader, threads=3, run=run, gap=gap)
    items = [(name, p, first, first + n, None) for name, (p, first, n, _, _) in files.where.items()]
    ahead.queue(items)
    ahead.queue(items[:2])                                      # queued already: nothing new starts
    ahead.drop(["nothing", "flags"])
    for name, want in bag().items():
        got = ahead.take(name)
        if name in ("nothing", "flags"):
            assert got is None
        else:
            check(got.view(want.dtype).reshape(want.shape), want, name)
    assert not ahead.ahead and ahead.take("wide") is None
    ahead.close()


def test_background_jobs_report_the_first_error():
    done, futures = [], []
    dr.in_background(lambda: done.append(1), futures)
    dr.in_background(lambda: 1 // 0, futures)
    with pytest.raises(ZeroDivisionError):
        dr.wait_all(futures)
    assert done == [1] and futures == []
