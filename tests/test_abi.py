"""The C ABI and the host logic, without a GPU: libtfmi.so loads and exports every symbol include/tfmi.h declares,
the ctypes table matches the header, shape-only planners are pure functions, argument errors surface as the
reference's do, and nothing in the product imports the oracle."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

from tensorfold_amd import _lib, build, experts, qmm
from tensorfold_amd.exl3 import format as fmt
from tensorfold_amd.exl3 import linear

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "tfmi.h").read_text()
DECLARED = re.findall(r"^(?:int|const char\*)\s+(tf_\w+)\(", HEADER, flags=re.M)


def test_library_exports_the_header():
    assert len(DECLARED) >= 19
    so = build.load()
    for name in DECLARED:
        assert hasattr(so, name), name
    so.tf_version.restype = ctypes.c_int
    assert so.tf_version() == 3
    # the library says which sources it was built from, and the loader only hands out one built from these
    so.tf_build_id.restype = ctypes.c_char_p
    assert so.tf_build_id().decode() == build.source_id() == build.built_id() and not build.stale()
    so.tf_last_error.restype = ctypes.c_char_p
    assert so.tf_last_error() == b""


def test_ctypes_table_covers_the_header():
    compute = [n for n in DECLARED if n not in ("tf_last_error", "tf_version", "tf_build_id", "tf_check_device")]
    assert sorted(compute) == sorted(_lib.PROTOTYPES)
    for name, args in _lib.PROTOTYPES.items():                 # argument counts against the header's text
        decl = re.search(name + r"\((.*?)\);", HEADER, flags=re.S).group(1)
        assert len(args) == decl.count(",") + 1, name


def test_host_constants_are_the_headers():
    """The counter layouts the host allocates are the ones the kernels index: the header's defines and the Python
    constants agree."""

    from tensorfold_amd import moe

    define = lambda name: int(re.search(r"^#define " + name + r" (\d+)", HEADER, flags=re.M).group(1))
    assert define("TF_DESC_TILE") == moe.DESC_TILE
    assert define("TF_DONE_STRIDE") == moe.DONE_STRIDE
    assert define("TF_ARRIVE_STRIDE") == moe.ARRIVE_STRIDE
    assert define("TF_EXL3_COUNTER_STRIDE") == linear.COUNTER_STRIDE
    assert [moe.arrive_stride(r) for r in (1, 64, 65, 1024)] == [moe.ARRIVE_STRIDE, moe.ARRIVE_STRIDE, 1, 1]


def test_no_gpu_means_a_loud_error_not_a_fallback():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(RuntimeError, match="no CPU path"):
        qmm.group_sums(torch.zeros((1, 64), dtype=torch.bfloat16))
    with pytest.raises(RuntimeError):
        experts.pack(torch.zeros((1, 32, 8), dtype=torch.int32), torch.zeros((1, 32, 1)).bfloat16(),
                     torch.zeros((1, 32, 1)).bfloat16(), 64)


def test_the_product_never_imports_the_oracle():
    for path in (ROOT / "tensorfold_amd").rglob("*"):
        if path.suffix in (".py", ".hip", ".h"):
            text = path.read_text()
            assert "oracle" not in text.replace("no oracle", ""), path


def test_argument_errors_come_before_the_gpu():
    with pytest.raises(ValueError, match="32 or 64"):
        experts.pack(torch.zeros((1, 32, 8), dtype=torch.int32), torch.zeros((1, 32, 4)), torch.zeros((1, 32, 4)), 16)
    with pytest.raises(ValueError, match="does not pack"):
        experts.pack(torch.zeros((1, 33, 8), dtype=torch.int32), torch.zeros((1, 33, 1)), torch.zeros((1, 33, 1)), 64)
    with pytest.raises(ValueError, match="at least one row"):
        qmm.bucket(0)
    with pytest.raises(ValueError, match="gate and an up"):
        experts.make([], (), 64)
    with pytest.raises(ValueError):
        fmt.check_bits(4.5)                       # a dense layer's checkpoint never holds it (the routed experts take it)
    with pytest.raises(ValueError):
        fmt.bits_of((4, 4, 36))


def test_planners_are_functions_of_the_shape():
    assert [qmm.bucket(m) for m in (1, 16, 17, 32, 33, 500)] == [16, 16, 32, 32, 64, 64]
    for n, k in [(48, 5120), (1024, 5120), (4096, 4096), (17408, 5120), (5120, 17408), (248320, 5120)]:
        sk = qmm.split_k(n, k)
        assert sk == qmm.split_k(n, k) and (k // 64) % sk == 0 and sk in (1, 2, 4, 8, 16)
    assert experts.max_items(48, 128) == 48 and experts.max_items(45056, 513, 64) == 513 + 704      # never more items than pairs
    assert experts.block_words(64) == 288 and experts.block_words(32) == 160
    for k, n in ((128, 128), (256, 256), (5120, 17408), (17408, 5120), (4096, 12288), (4096, 152576)):
        sk, wk = linear.plan(k, n)
        assert (sk, wk) == linear.plan(k, n) and sk * wk <= k // 32 and wk in (2, 4, 8)
    assert linear.plan(17408, 5120)[0] > linear.plan(5120, 17408)[0]      # the narrow layer splits K further


def test_format_facts():
    assert fmt.tile_words(3) == 48 and fmt.bits_of((320, 1088, 48)) == 3 and fmt.bits_of((4, 4, 40)) == 2.5
    assert linear.k2_of(3) == 6 and linear.k2_of(2.5) == 5
    import numpy as np

    signs = np.array([0b1000_0000_0000_0101, 0], dtype=np.uint16).view(np.int16)
    want = np.ones(32, dtype=np.float16)
    want[[0, 2, 15]] = -1
    assert np.array_equal(fmt.unpack_signs(signs), want)
    t = torch.arange(2 * 16 * 4, dtype=torch.int32).reshape(2, 16, 4)
    s = linear.strips(t)
    assert s.shape == (2, 2, 8, 4) and torch.equal(s[1, 0], t[0, 8:16]) and torch.equal(s[0, 1], t[1, 0:8])


def test_host_wrappers_reject_scratch_that_is_too_small():
    """A caller's buffer that cannot hold what the kernel writes must stop in Python, before any launch."""

    import inspect

    from tensorfold_amd import experts, qmm
    from tensorfold_amd.exl3 import linear

    assert "part must hold" in inspect.getsource(qmm.matmul)
    assert "z must hold" in inspect.getsource(linear.Exl3Linear.__call__)
    plan = experts.Plan.__new__(experts.Plan)
    plan.rows, plan.slots = 4, 3
    with pytest.raises(ValueError):
        experts._fits(plan, 5, 5, 15)
    with pytest.raises(ValueError):
        experts._fits(plan, 4, 3, 12)
    with pytest.raises(ValueError):
        experts._fits(plan, 4, 4, 11)
    experts._fits(plan, 4, 4, 12)
