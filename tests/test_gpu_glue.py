"""The fused producers (residual add + RMSNorm + group sums) on the GPU against the CPU oracle: the residual stream h
bit for bit (no reduction enters it), the normed row and its group sums within bf16 / fp32 rounding of the oracle's
float64 mean square, rows independent of the window."""

import numpy as np
import pytest
import torch

from oracle import affine as ora
from tensorfold_amd import glue
from tests.helpers import bits16, f32, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = 2e-3          # relative L2 of the bf16 outputs


def case(rows, d, slots, seed):
    rng = np.random.default_rng(seed)
    h = ora.bf16(rng.standard_normal((rows, d)).astype(np.float32))
    y = (rng.standard_normal((rows, slots, d)) * 0.5).astype(np.float32)
    wts = ora.bf16(rng.random((rows, slots)).astype(np.float32) * 0.5 + 0.05)
    w = ora.bf16((rng.random(d) + 0.5).astype(np.float32))
    return h, y, wts, w


def bf(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).to(DEV)


def check_norm(got_y, got_xs, want_y, want_xs, gs):
    got_y, got_xs = f32(got_y), got_xs.cpu().numpy()
    assert rel_l2(got_y, want_y) <= TOL
    # the mean square is summed in another order than the oracle's float64: a value may land one bf16 step away
    assert np.abs(got_y - want_y).max() <= 2 ** -7 * np.abs(want_y).max()
    assert (got_y == want_y).mean() > 0.98
    # the group sums are the sums of the row the kernel stored, to fp32 rounding of gs terms
    own = got_y.reshape(got_y.shape[0], -1, gs).astype(np.float64).sum(axis=2)
    assert np.abs(got_xs - own).max() <= 1e-5 * max(1.0, np.abs(own).max())
    assert np.abs(got_xs - want_xs).max() <= 2 ** -6 * np.abs(want_y).max() * gs ** 0.5 + 1e-5


@pytest.mark.parametrize("rows,d,gs", [(1, 64, 64), (8, 2688, 64), (3, 2048, 32), (32, 4096, 64), (5, 5120, 128),
                                        (2, 16384, 64), (7, 96, 32), (4, 1152, 128)])
def test_add_rmsnorm_matches_the_oracle(rows, d, gs):
    h, y, _, w = case(rows, d, 1, 100 + d)
    r = ora.bf16(y[:, 0])
    want_h, want_y, want_xs = ora.add_rmsnorm(h, r, w, 1e-5, gs)
    got_h, got_y, got_xs = glue.add_rmsnorm(bf(h), bf(r), bf(w), 1e-5, gs)
    assert np.array_equal(bits16(got_h), ora.bf16_bits(want_h))
    check_norm(got_y, got_xs, want_y, want_xs, gs)
    # without a residual h is x itself and nothing is written to it
    x = bf(h)
    same, got_y, got_xs = glue.add_rmsnorm(x, None, bf(w), 1e-5, gs)
    assert same is x
    _, want_y, want_xs = ora.add_rmsnorm(h, None, w, 1e-5, gs)
    check_norm(got_y, got_xs, want_y, want_xs, gs)


@pytest.mark.parametrize("rows,d,slots,top_k,ybf", [(8, 2688, 7, 6, False), (1, 2688, 7, 6, False), (32, 2048, 11, 10, False),
                                                     (4, 4096, 9, 8, True), (3, 256, 20, 17, False), (2, 128, 1, 1, False),
                                                     (2, 128, 2, 0, True), (5, 1024, 8, 8, False)])
def test_add_moe_norm_matches_the_oracle(rows, d, slots, top_k, ybf):
    h, y, wts, w = case(rows, d, slots, 200 + d + slots)
    if ybf:
        y = ora.bf16(y)
    want_h, want_y, want_xs = ora.add_moe_norm(h, y, wts, w, 1e-5, top_k)
    yt = torch.from_numpy(y.reshape(rows * slots, d)).to(DEV)
    got_h, got_y, got_xs = glue.add_moe_norm(bf(h), yt.to(torch.bfloat16) if ybf else yt,
                                             torch.from_numpy(wts).to(DEV), bf(w), 1e-5, top_k)
    assert np.array_equal(bits16(got_h), ora.bf16_bits(want_h))          # products and sums in the oracle's order
    check_norm(got_y, got_xs, want_y, want_xs, 64)


def test_rows_do_not_depend_on_the_window():
    h, y, wts, w = case(16, 2688, 7, 7)
    yt = torch.from_numpy(y.reshape(16 * 7, 2688)).to(DEV)
    wt = torch.from_numpy(wts).to(DEV)
    full = glue.add_moe_norm(bf(h), yt, wt, bf(w), 1e-5, 6)
    for r in (0, 5, 15):
        one = glue.add_moe_norm(bf(h[r:r + 1]), yt[7 * r:7 * r + 7], wt[r:r + 1], bf(w), 1e-5, 6)
        for a, b in zip(full, one):
            assert torch.equal(a[r:r + 1], b)


def test_the_group_sums_feed_the_decode_matmul():
    """xs from the producer equals qmm.group_sums of the stored row to fp32 rounding: the matmul may take either."""

    from tensorfold_amd import qmm

    h, y, _, w = case(8, 4096, 1, 9)
    _, out, xs = glue.add_rmsnorm(bf(h), bf(ora.bf16(y[:, 0])), bf(w), 1e-5, 64)
    ref = qmm.group_sums(out, 64)
    assert torch.allclose(xs, ref, rtol=1e-5, atol=1e-4)


def test_bad_arguments_raise():
    h, y, wts, w = case(2, 128, 3, 1)
    with pytest.raises(ValueError):
        glue.add_rmsnorm(bf(h).float(), None, bf(w), 1e-5)
    with pytest.raises(ValueError):
        glue.add_rmsnorm(bf(h), None, bf(w)[:64], 1e-5)
    with pytest.raises(ValueError):
        glue.add_rmsnorm(bf(h), None, bf(w), 1e-5, gs=48)
    with pytest.raises(ValueError):
        glue.add_rmsnorm(bf(h), bf(h)[:1], bf(w), 1e-5)
    yt = torch.from_numpy(y.reshape(6, 128)).to(DEV)
    with pytest.raises(ValueError):
        glue.add_moe_norm(bf(h), yt[:5], torch.from_numpy(wts).to(DEV), bf(w), 1e-5, 2)
    with pytest.raises(ValueError):
        glue.add_moe_norm(bf(h), yt, torch.from_numpy(wts).to(DEV), bf(w), 1e-5, 4)
    with pytest.raises(ValueError):
        glue.add_moe_norm(bf(h), yt, torch.from_numpy(wts).double().to(DEV), bf(w), 1e-5, 2)
