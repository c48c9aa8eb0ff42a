"""Dense 4-bit lane matmul on the GPU against the CPU oracle (properties after the reference's tests/cuda/test_qmm.py)."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from oracle import native
from tensorfold_amd import qmm, synthetic
from tests.helpers import bits16, f32, max_abs, rel_l2, u32

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3          # relative L2 bound on bf16 outputs (fp32 accumulation), as the benchmark states


def gpu(*ts):
    return tuple(t.to(DEV) for t in ts)


@pytest.mark.parametrize("n,k,gs", [(48, 5120, 64), (1024, 5120, 64), (200, 1024, 32), (1536, 2048, 32)])
def test_pack_round_trip(n, k, gs):
    w = gpu(*synthetic.affine_general(n, k, gs, n + k))
    back = qmm.unpack(qmm.pack(*w, gs))
    assert all(torch.equal(a, b) for a, b in zip(back, w))


@pytest.mark.parametrize("n,k,gs", [(128, 5120, 64), (200, 1024, 32)])
def test_every_nibble_decodes_exactly(n, k, gs):
    """One-hot rows read back each stored nibble (scale 1, bias 0), through every K split, decode and prefill form."""

    words = synthetic.affine_general(n, k, gs, 29)[0].to(DEV)
    ones = torch.ones((n, k // gs), device=DEV).bfloat16()
    zeros = torch.zeros_like(ones)
    q = qmm.pack(words, ones, zeros, gs)
    want = torch.from_numpy(ora.nibbles(u32(words)).astype(np.float32).T.copy())            # (k, n): every code
    assert set(want.unique().tolist()) == set(range(16))
    eye = torch.eye(k, device=DEV).bfloat16()
    for f in (False, True):
        assert torch.equal(qmm.matmul(eye, q, f32=f).float().cpu(), want), f
        assert torch.equal(qmm.matmul(eye, q, f32=f, sk=1).float().cpu(), want), f
        assert torch.equal(qmm.prefill_matmul(eye, q, f32=f).float().cpu(), want), f


def test_config0_single_linear_matches_the_oracle():
    """benchmark configuration 0: N = K = 4096, g64, one row; bf16 out against dequant-then-matmul."""

    n = k = 4096
    w = synthetic.affine(n, k, 64, 1000)
    x = synthetic.activations(1, k, 1001)
    q = qmm.pack(*gpu(*w), 64)
    y = qmm.matmul(x.to(DEV), q)
    ref = native.affine_linear(bits16(x), u32(w[0]), bits16(w[1]), bits16(w[2]), 64)
    want = ora.bf16(ref)
    err = rel_l2(f32(y), want)
    print(f"config 0 decode: rel-L2 {err:.2e}, max-abs {max_abs(f32(y), want):.3e}")
    assert err <= TOL
    yp = qmm.prefill_matmul(x.to(DEV), q)
    errp = rel_l2(f32(yp), want)
    print(f"config 0 prefill form: rel-L2 {errp:.2e}, max-abs {max_abs(f32(yp), want):.3e}")
    assert errp <= TOL
    # numpy statement of the same oracle agrees with the C one
    assert rel_l2(ora.linear(f32(x), u32(w[0]), f32(w[1]), f32(w[2]), 64, f32=True), ref) < 1e-5


@pytest.mark.parametrize("n,k,gs", [(1024, 5120, 64), (512, 2048, 32), (200, 1024, 32)])
def test_accuracy_matches_fp32_reference(n, k, gs):
    w = synthetic.affine_general(n, k, gs, 11 * n + k)
    x = synthetic.activations(16, k, 5)
    q = qmm.pack(*gpu(*w), gs)
    ref = native.affine_linear(bits16(x), u32(w[0]), bits16(w[1]), bits16(w[2]), gs)
    y = f32(qmm.matmul(x.to(DEV), q))
    assert max_abs(y, ref) <= np.abs(ref).max() * 2 ** -7          # the reference's own bound (test_qmm.py:64-70)
    assert rel_l2(y, ref) <= TOL
    y32 = f32(qmm.matmul(x.to(DEV), q, f32=True))
    assert rel_l2(y32, ref) <= 1e-5
    refp = native.affine_linear(bits16(x), u32(w[0]), bits16(w[1]), bits16(w[2]), gs, prefill=True)
    yp = f32(qmm.prefill_matmul(x.to(DEV), q, f32=True))
    assert rel_l2(yp, refp) <= 1e-5                                  # same once-rounded weights, fp32 chain
    assert rel_l2(f32(qmm.prefill_matmul(x.to(DEV), q)), ref) <= TOL


ROWS = [1, 2, 3, 4, 5, 7, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 129, 200]


@pytest.mark.parametrize("n,k,gs", [(48, 5120, 64), (1024, 2048, 64), (200, 1024, 32)])
def test_rows_do_not_depend_on_row_count(n, k, gs):
    q = qmm.pack(*gpu(*synthetic.affine_general(n, k, gs, 3 * n + k)), gs)
    x = synthetic.activations(max(ROWS), k, 7).to(DEV)
    alone = torch.cat([qmm.matmul(x[r:r + 1], q) for r in range(max(ROWS))])
    alone_p = torch.cat([qmm.prefill_matmul(x[r:r + 1], q) for r in range(max(ROWS))])
    for m in ROWS:
        assert torch.equal(qmm.matmul(x[:m], q), alone[:m]), f"{n}x{k}: rows differ at M={m}"
        assert torch.equal(qmm.prefill_matmul(x[:m], q), alone_p[:m]), f"{n}x{k}: prefill rows differ at M={m}"
    perm = torch.randperm(max(ROWS), generator=torch.Generator().manual_seed(3)).to(DEV)
    assert torch.equal(qmm.matmul(x[perm], q), alone[perm])
    f32_ = qmm.matmul(x[:40], q, f32=True)
    assert torch.equal(torch.cat([qmm.matmul(x[r:r + 1], q, f32=True) for r in range(40)]), f32_)


@pytest.mark.parametrize("n,k,gs", [(4096, 4096, 64), (200, 1024, 32), (1536, 2048, 32)])
def test_the_slices_added_in_the_matmuls_own_launch(n, k, gs):
    """Up to eight rows with a weight's arrival counters: the last workgroup of a tile adds the K slices up; without
    them the one-launch form runs (or, past eight rows, a second launch).  The same bits, the counters zero again
    afterwards, also on replays of a graph; more rows take the other forms whatever is passed."""

    from tensorfold_amd import _lib

    q = qmm.pack(*gpu(*synthetic.affine_general(n, k, gs, n + k)), gs)
    sk = qmm.split_k(n, k, gs)
    assert sk > 1
    x = synthetic.activations(65, k, 12).to(DEV)

    def two_launches(rows, f32=False):
        xs, m = qmm.group_sums(rows, gs), int(rows.shape[0])
        out = torch.empty((m, n), device=DEV, dtype=torch.float32 if f32 else torch.bfloat16)
        part = torch.empty((sk, m, n), device=DEV, dtype=torch.float32)
        _lib.call("tf_qmm", _lib.ptr(rows), rows.stride(0), _lib.ptr(xs), _lib.ptr(q.weight), _lib.ptr(q.scales),
                  _lib.ptr(q.biases), q.scales.stride(0), _lib.ptr(out), _lib.ptr(part), None, 0, m, n, k, sk, gs,
                  qmm.bucket(m), int(f32), 1)
        return out

    for m in (1, 2, 3, 4, 5, 6, 7, 8, 9, 11, 13, 17, 65):
        assert torch.equal(qmm.matmul(x[:m], q), two_launches(x[:m])), m
        assert not q.counters.any(), m
    for r in (5, 64):
        assert torch.equal(qmm.matmul(x[r:r + 1], q)[0], two_launches(x[:65])[r]), r
    assert torch.equal(qmm.matmul(x[:3], q, f32=True), two_launches(x[:3], f32=True))
    out, part = torch.empty((3, n), device=DEV, dtype=torch.bfloat16), torch.empty((sk, 3, n), device=DEV)
    xs = qmm.group_sums(x[:3], gs)
    qmm.matmul(x[:3], q, xs, out=out, part=part)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(3):
            qmm.matmul(x[:3], q, xs, out=out, part=part)
    want = two_launches(x[:3])
    for _ in range(3):
        out.zero_()
        graph.replay()
        assert torch.equal(out, want) and not q.counters.any()


def test_split_depends_only_on_shape():
    for n, k in [(48, 5120), (1024, 5120), (5120, 6144), (17408, 5120), (5120, 17408), (248320, 5120), (4096, 4096)]:
        sk = qmm.split_k(n, k)
        assert sk == qmm.split_k(n, k) and (k // 64) % sk == 0


def test_strided_rows_buffers_and_unreduced_slices():
    n, k, gs = 640, 8192, 64
    q = qmm.pack(*gpu(*synthetic.affine_general(n, k, gs, 17)), gs)
    wide = synthetic.activations(24, k + 64, 9).to(DEV)
    x = wide[:, :k]                                   # rows 16-byte aligned, stride k + 64
    want = qmm.matmul(x.contiguous(), q)
    assert torch.equal(qmm.matmul(x, q), want)
    out = torch.empty_like(want)
    assert qmm.matmul(x, q, out=out) is out and torch.equal(out, want)
    sk = qmm.split_k(n, k)
    assert sk > 1
    slices = qmm.matmul(x, q, reduce=False, f32=True)
    assert slices.shape == (sk, 24, n)
    total = slices[0]
    for s in range(1, sk):
        total = total + slices[s]
    assert torch.equal(total, qmm.matmul(x, q, f32=True))


@pytest.mark.parametrize("m", [1, 3, 17])
def test_grouped_launch_has_the_bits_of_single_calls(m):
    """Up to four weights against one x in one launch (after tests/cuda/test_qmm_group.py): each output equals
    matmul's bit for bit, for mixed widths and slice counts, bf16 and fp32."""

    k = 2048
    x = gpu(synthetic.activations(m, k, 50 + m))[0]
    for gs, ns in ((64, (256, 1024, 96, 4096)), (32, (128, 640)), (64, (512,))):
        qs = [qmm.pack(*gpu(*synthetic.affine_general(n, k, gs, 60 + n)), gs) for n in ns]
        for f32 in (False, True):
            got = qmm.matmul_group(x, qs, f32=f32)
            for q, y in zip(qs, got):
                assert torch.equal(y, qmm.matmul(x, q, f32=f32)), (gs, q.n, f32)
        sks = [1] + [2] * (len(qs) - 1)
        got = qmm.matmul_group(x, qs, sks=sks)
        for q, sk, y in zip(qs, sks, got):
            assert torch.equal(y, qmm.matmul(x, q, sk=sk))
    with pytest.raises(ValueError):
        qmm.matmul_group(x, [])
    with pytest.raises(ValueError):
        qmm.matmul_group(x, [qs[0]] * 5)


def test_group_sums():
    x = synthetic.activations(5, 2048, 3).to(DEV)
    for gs in (32, 64):
        got = f32(qmm.group_sums(x, gs))
        want = ora.group_sums(f32(x), gs)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_bad_arguments_raise():
    w = gpu(*synthetic.affine_general(64, 256, 64, 1))
    with pytest.raises(ValueError):
        qmm.pack(*w, 48)
    q = qmm.pack(*w, 64)
    with pytest.raises(ValueError):
        qmm.matmul(torch.zeros((1, 128), device=DEV).bfloat16(), q)
    with pytest.raises(ValueError):
        qmm.matmul(torch.zeros((1, 256), device=DEV), q)
    with pytest.raises(RuntimeError, match="whole groups"):
        qmm.matmul(torch.zeros((1, 256), device=DEV).bfloat16(), q, sk=3)
    x = torch.zeros((2, 256), device=DEV).bfloat16()
    with pytest.raises(ValueError, match="part must hold"):
        qmm.matmul(x, q, sk=4, part=torch.empty((2, 2, 64), device=DEV))       # room for 2 of the 4 slices
    with pytest.raises(ValueError, match="out must be"):
        qmm.matmul(x, q, out=torch.empty((1, 64), device=DEV, dtype=torch.bfloat16))


def test_the_bf16_prompt_form_is_the_references_arithmetic():
    """``arith=1``: every weight bf16(fma(q, s, b)), bf16 activations, bf16 MFMA, one fp32 chain (the reference's
    kernels/qmm_prefill.cu:116-117).  Equal to the oracle with the same once-rounded weights to fp32 rounding, rows
    independent of the row count, and (with eight times the fp16 form's weight rounding) further from the fp32-weight
    oracle than the fp16 form is."""

    for n, k, gs in ((512, 2048, 32), (200, 1024, 64)):
        w = synthetic.affine_general(n, k, gs, 5 * n + k)
        x = synthetic.activations(70, k, 6)
        q = qmm.pack(*gpu(*w), gs)
        assert q.arith == 0                                     # these scales and biases fit the fp16 form
        want = native.affine_linear(bits16(x), u32(w[0]), bits16(w[1]), bits16(w[2]), gs, prefill=2)
        got = qmm.prefill_matmul(x.to(DEV), q, f32=True, arith=1)
        assert rel_l2(f32(got), want) <= 1e-5
        exact = native.affine_linear(bits16(x), u32(w[0]), bits16(w[1]), bits16(w[2]), gs)
        e16, e_bf = rel_l2(f32(qmm.prefill_matmul(x.to(DEV), q, f32=True)), exact), rel_l2(f32(got), exact)
        print(f"{n}x{k} g{gs}: fp16 form {e16:.2e}, bf16 form {e_bf:.2e} from the fp32-weight oracle")
        assert e16 < e_bf <= 8e-3
        for m in (1, 16, 17, 64, 65):
            assert torch.equal(qmm.prefill_matmul(x[:m].to(DEV), q, f32=True, arith=1), got[:m]), m


def test_prompt_form_beyond_the_range_of_fp16():
    """Scales around 300 and activations around 1e5: 256 x scale has no fp16 value, so ``pack`` marks the weight for
    the bf16 form and ``prefill_matmul`` takes it by itself; the result matches the oracle (2e-3 against the oracle
    with the same once-rounded weights is loose: it measures 1e-6; against fp32 weights the bf16 rounding shows).
    With a table that fits, the fp16 form clamps activations beyond +-65504, no more and no less."""

    n, k, gs = 256, 1024, 64
    g = torch.Generator().manual_seed(91)
    words = synthetic.affine_general(n, k, gs, 92)[0]
    scales = (torch.rand((n, k // gs), generator=g) * 200 + 200).bfloat16()               # 200 to 400
    biases = (scales.float() * -7.5).bfloat16()
    x = (torch.randn((40, k), generator=g) * 1e5).bfloat16()
    q = qmm.pack(words.to(DEV), scales.to(DEV), biases.to(DEV), gs)
    assert q.arith == 1
    got = qmm.prefill_matmul(x.to(DEV), q, f32=True)
    assert torch.isfinite(got).all()
    same = native.affine_linear(bits16(x), u32(words), bits16(scales), bits16(biases), gs, prefill=2)
    exact = native.affine_linear(bits16(x), u32(words), bits16(scales), bits16(biases), gs)
    err, err_exact = rel_l2(f32(got), same), rel_l2(f32(got), exact)
    print(f"beyond fp16: rel-L2 {err:.2e} (same rounded weights), {err_exact:.2e} (fp32 weights), "
          f"max-abs {max_abs(f32(got), same):.3e} of {np.abs(same).max():.3e}")
    assert err <= 1e-5 and err_exact <= 8e-3
    assert rel_l2(f32(qmm.matmul(x.to(DEV), q, f32=True)), exact) <= 1e-5            # the decode form never minded
    # a table that fits fp16 with activations that do not: the fp16 form is the matmul of the clamped activations
    small = synthetic.affine_general(n, k, gs, 93)
    q2 = qmm.pack(*gpu(*small), gs)
    assert q2.arith == 0
    clamped = x.float().clamp(-65504, 65504).bfloat16()
    assert not torch.equal(clamped, x)
    want = native.affine_linear(bits16(clamped), u32(small[0]), bits16(small[1]), bits16(small[2]), gs, prefill=True)
    unclamped = native.affine_linear(bits16(x), u32(small[0]), bits16(small[1]), bits16(small[2]), gs, prefill=2)
    got16 = f32(qmm.prefill_matmul(x.to(DEV), q2, f32=True))
    # (the oracle's clamp lands on bf16's 65536, the kernel's on fp16's 65504: 5e-4 apart)
    assert rel_l2(got16, want) <= 1e-3 and rel_l2(got16, unclamped) > 0.1
    assert rel_l2(f32(qmm.prefill_matmul(x.to(DEV), q2, f32=True, arith=1)), unclamped) <= 1e-5
