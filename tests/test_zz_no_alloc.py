"""The entry point that allocates nothing, ``tf_qmm_static``, against ``tf_qmm`` through the C ABI: same bits on two
calls in a row, the second smaller than the first (the library's built-in array keeps the first call's contents)."""

import pytest
import torch

from tensorfold_amd import _lib, qmm, synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda"


def both(x, q, sk, f32):
    """(tf_qmm's result, tf_qmm_static's result) for the same operands, each through the C ABI."""

    m = int(x.shape[0])
    xs = qmm.group_sums(x, q.gs)
    dtype = torch.float32 if f32 else torch.bfloat16
    want = torch.full((m, q.n), 7.0, device=DEV, dtype=dtype)
    got = torch.full((m, q.n), -7.0, device=DEV, dtype=dtype)
    part = torch.empty((sk, m, q.n), device=DEV, dtype=torch.float32)
    common = (_lib.ptr(x), x.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales), _lib.ptr(q.biases),
              q.scales.stride(0))
    shape = (m, q.n, q.k, sk, q.gs, qmm.bucket(m), int(f32))
    _lib.call("tf_qmm", *common, _lib.ptr(want), _lib.ptr(part), None, 0, *shape, 1)      # no arrival counters
    _lib.call("tf_qmm_static", *common, _lib.ptr(got), *shape)
    torch.cuda.synchronize()
    return want, got


@pytest.mark.parametrize("f32", [False, True])
def test_static_scratch_matches_the_part_buffer_twice(f32):
    n, k, gs = 1536, 4096, 64
    q = qmm.pack(*(t.to(DEV) for t in synthetic.affine_general(n, k, gs, 77)), gs)
    sk = qmm.split_k(n, k, gs)
    assert sk > 1
    # more than 8 rows: the split launch and its reduce run, so the K slices really pass through the array
    for rows, seed in ((40, 1), (12, 2)):
        x = synthetic.activations(rows, k, seed).to(DEV)
        want, got = both(x, q, sk, f32)
        assert torch.equal(want, got), (rows, f32)
    # up to eight rows finish in one launch: the library's own arrival counters there, tf_qmm (given none) in its
    # one-launch form; the counters are back at zero after each call, so calls in a row agree
    for rows, seed in ((3, 3), (8, 4), (1, 5), (1, 6), (5, 7)):
        x = synthetic.activations(rows, k, seed).to(DEV)
        want, got = both(x, q, sk, f32)
        assert torch.equal(want, got), (rows, f32)


def test_static_scratch_host_wrapper_and_limit():
    n, k, gs = 1024, 2048, 32
    q = qmm.pack(*(t.to(DEV) for t in synthetic.affine_general(n, k, gs, 5)), gs)
    x = synthetic.activations(20, k, 9).to(DEV)
    xs = qmm.group_sums(x, gs)
    out = torch.empty((20, n), device=DEV, dtype=torch.bfloat16)
    assert torch.equal(qmm.matmul_static(x, q, xs, out), qmm.matmul(x, q, xs))
    # beyond the built-in array: refused by the library with a sentence, nothing launched
    big = qmm.STATIC_FLOATS // (16 * n) + 1
    xb = torch.zeros((big, k), device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="exceed"):
        qmm.matmul_static(xb, q, qmm.group_sums(xb, gs), torch.empty((big, n), device=DEV, dtype=torch.bfloat16), sk=16)
    so = _lib.lib()
    rc = so.tf_qmm_static(_lib.ptr(xb), xb.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales),
                          _lib.ptr(q.biases), q.scales.stride(0), _lib.ptr(out), big, n, k, 16, gs, 64, 0, _lib.stream())
    assert rc != 0 and b"exceed" in so.tf_last_error()


def test_static_scratch_allocates_nothing():
    """What the entry point is for: calls of both paths (more than eight rows: split launch + reduce; up to eight:
    one launch on the built-in counters) leave the device's free memory and torch's pools exactly where they were.
    The built-in counters being back at zero shows in the runs of few-row calls above, which would sum wrongly
    otherwise."""

    n, k, gs = 1536, 4096, 64
    q = qmm.pack(*(t.to(DEV) for t in synthetic.affine_general(n, k, gs, 78)), gs)
    sk = qmm.split_k(n, k, gs)
    so = _lib.lib()
    cases = []
    for rows in (40, 5):
        x = synthetic.activations(rows, k, rows).to(DEV)
        xs = qmm.group_sums(x, gs)
        out = torch.empty((rows, n), device=DEV, dtype=torch.bfloat16)
        cases.append((x, xs, out, rows, qmm.matmul(x, q, xs)))
    stream = _lib.stream()

    def run(x, xs, out, rows, _):
        rc = so.tf_qmm_static(_lib.ptr(x), x.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales),
                              _lib.ptr(q.biases), q.scales.stride(0), _lib.ptr(out), rows, n, k, sk, gs,
                              qmm.bucket(rows), 0, stream)
        assert rc == 0, so.tf_last_error()

    for c in cases:                      # first calls on this device: the array's address is looked up here
        run(*c)
    torch.cuda.synchronize()
    before = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    for _ in range(20):
        for c in cases:
            run(*c)
    torch.cuda.synchronize()
    after = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert before == after, (before, after)
    for c in cases:
        assert torch.equal(c[2], c[4]), c[3]
