"""Pins of the oracle's tensor kernels against PyTorch CPU ops, closed forms and
brute force (the reference holds no test vectors for them)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from util import bilinear_tol, normal, pool_out, rel_err, torch_bn_stats, torch_im2col, torch_maxpool, uniform

IM2COL_CASES = [
    # (N, C, H, W, kernel, pad, stride, dil)
    (2, 3, 8, 8, (3, 3), (1, 1), (1, 1), (1, 1)),
    (1, 2, 7, 9, (3, 2), (0, 1), (2, 1), (1, 1)),
    (2, 2, 11, 10, (2, 3), (2, 2), (1, 2), (2, 1)),
    (1, 1, 5, 5, (5, 5), (2, 2), (1, 1), (1, 1)),
    (4, 8, 56, 56, (3, 3), (1, 1), (1, 1), (1, 1)),
]


@pytest.mark.parametrize("case", IM2COL_CASES, ids=str)
def test_im2col_vs_torch_unfold(case):
    n, c, h, w, k, p, s, d = case
    x = uniform((n, c, h, w), 1)
    got = O.im2col(x.reshape(n * c, h, w).numpy(), k, p, s, d)
    want = torch_im2col(x, k, p, s, d).numpy()  # [N, C*kh*kw, L]
    assert np.array_equal(got.reshape(want.shape), want)


def test_im2col_centre_tap_is_the_image():
    x = uniform((6, 9, 12), 2).numpy()
    col = O.im2col(x, (3, 3), (1, 1), (1, 1)).reshape(6, 9, 9, 12)
    assert np.array_equal(col[:, 4], x)
    assert np.all(col[:, 0, 0, :] == 0) and np.all(col[:, 8, -1, :] == 0)  # padded border taps


POOL_CASES = [
    (2, 3, 8, 8, (3, 3), (2, 2), (1, 1), (1, 1)),
    (1, 2, 9, 7, (2, 2), (2, 2), (0, 0), (1, 1)),
    (2, 2, 13, 11, (3, 2), (1, 2), (1, 1), (2, 1)),
    (1, 1, 6, 6, (3, 3), (1, 1), (1, 1), (1, 1)),
    (2, 4, 112, 112, (3, 3), (2, 2), (1, 1), (1, 1)),
    (2, 4, 64, 64, (2, 2), (2, 2), (0, 0), (1, 1)),
]


@pytest.mark.parametrize("case", POOL_CASES, ids=str)
def test_max_pool_vs_torch(case):
    n, c, h, w, k, s, p, d = case
    x = uniform((n, c, h, w), 3)
    val, idx = O.max_pool(x.numpy(), k, s, p, d)
    tv, ti = torch_maxpool(x, k, s, p, d)
    assert np.array_equal(val, tv.numpy())
    assert np.array_equal(idx, ti.numpy())


def test_max_pool_ties_keep_first_index_and_nan_wins():
    x = torch.full((1, 1, 8, 8), 0.25)
    val, idx = O.max_pool(x.numpy(), (3, 3), (2, 2), (1, 1))
    tv, ti = torch_maxpool(x, (3, 3), (2, 2), (1, 1))
    assert np.array_equal(idx, ti.numpy())
    # first in-bounds element of every window
    want = np.array([[max(2 * ph - 1, 0) * 8 + max(2 * pw - 1, 0) for pw in range(4)] for ph in range(4)])
    assert np.array_equal(idx[0, 0], want)
    y = uniform((1, 2, 8, 8), 4)
    y[0, 0, 3, 3] = float("nan")
    y[0, 1, 0, 0] = float("-inf")
    y[0, 1, 5, 5] = float("inf")
    val, idx = O.max_pool(y.numpy(), (3, 3), (2, 2), (1, 1))
    tv, ti = torch_maxpool(y, (3, 3), (2, 2), (1, 1))
    assert np.array_equal(idx, ti.numpy())
    assert np.array_equal(val, tv.numpy(), equal_nan=True)


def test_max_pool_bruteforce_small():
    x = uniform((1, 1, 7, 7), 5).numpy()
    val, idx = O.max_pool(x, (3, 3), (2, 2), (1, 1))
    for ph in range(pool_out(7, 3, 2, 1)):
        for pw in range(pool_out(7, 3, 2, 1)):
            best, where = -np.inf, None
            for h in range(2 * ph - 1, 2 * ph + 2):
                for w in range(2 * pw - 1, 2 * pw + 2):
                    if 0 <= h < 7 and 0 <= w < 7 and x[0, 0, h, w] > best:
                        best, where = x[0, 0, h, w], h * 7 + w
            assert val[0, 0, ph, pw] == best and idx[0, 0, ph, pw] == where


@pytest.mark.parametrize("shape,out", [((2, 3, 5, 7), (10, 14)), ((1, 2, 4, 4), (7, 9)), ((1, 1, 6, 5), (3, 4)),
                                       ((2, 2, 56, 56), (112, 112))])
def test_upsample_nearest_vs_torch(shape, out):
    x = uniform(shape, 6)
    got = O.upsample_nearest2d(x.numpy(), out)
    want = torch.nn.functional.interpolate(x, size=out, mode="nearest").numpy()
    assert np.array_equal(got, want)


def test_upsample_2x_closed_form():
    x = uniform((2, 3, 6, 8), 7).numpy()
    got = O.upsample_nearest2d(x, (12, 16))
    hh, ww = np.meshgrid(np.arange(12) >> 1, np.arange(16) >> 1, indexing="ij")
    assert np.array_equal(got, x[:, :, hh, ww])


BILINEAR_CASES = [((2, 3, 5, 7), (10, 14)), ((1, 2, 4, 4), (7, 9)), ((1, 1, 6, 5), (3, 4)), ((2, 2, 56, 56), (112, 112)),
                  ((1, 1, 3, 3), (3, 3)), ((1, 1, 8, 8), (1, 1)), ((1, 2, 1, 5), (4, 5)), ((1, 3, 50, 50), (77, 131)),
                  ((4, 8, 28, 28), (42, 60)), ((1, 1, 6, 8), (12, 24))]


@pytest.mark.parametrize("align", [False, True])
@pytest.mark.parametrize("shape,out", BILINEAR_CASES)
def test_upsample_bilinear_vs_torch(shape, out, align):
    """PyTorch CPU associates the four products differently and rounds the source index
    differently, so agreement is to rounding (bound: util.bilinear_tol)."""
    x = uniform(shape, 6)
    got = O.upsample_bilinear2d(x.numpy(), out, align)
    want = torch.nn.functional.interpolate(x, size=out, mode="bilinear", align_corners=align).numpy()
    assert np.abs(got - want).max() <= bilinear_tol(shape[2:], out, align)


def test_upsample_bilinear_closed_forms():
    x = uniform((2, 3, 6, 8), 7).numpy()
    assert np.array_equal(O.upsample_bilinear2d(x, (6, 8), False), x)            # same size: a copy
    c = np.full((1, 2, 5, 7), 0.375, dtype=np.float32)
    assert np.array_equal(O.upsample_bilinear2d(c, (11, 9), False), np.full((1, 2, 11, 9), 0.375, dtype=np.float32))
    # align_corners on a 2 x 2 image: corners are kept, the centre of a 3 x 3 output is the mean
    q = np.array([[[[0.0, 1.0], [2.0, 4.0]]]], dtype=np.float32)
    o = O.upsample_bilinear2d(q, (3, 3), True)
    assert o[0, 0, 0, 0] == 0.0 and o[0, 0, 0, 2] == 1.0 and o[0, 0, 2, 0] == 2.0 and o[0, 0, 2, 2] == 4.0
    assert o[0, 0, 1, 1] == 1.75 and o[0, 0, 0, 1] == 0.5 and o[0, 0, 1, 0] == 1.0
    # exact 2x without align_corners: interior weights are 0.25 / 0.75
    r = np.arange(8, dtype=np.float32).reshape(1, 1, 1, 8)
    o = O.upsample_bilinear2d(r, (1, 16), False)[0, 0, 0]
    assert o[0] == 0.0 and o[1] == 0.25 and o[2] == 0.75 and o[3] == 1.25 and o[15] == 7.0


@pytest.mark.parametrize("n,nbins,lo,hi", [(100000, 1024, 0.0, 1.0), (5000, 16, 0.0, 1.0), (70001, 256, -2.0, 2.0),
                                           (4096, 1, 0.0, 1.0)])
def test_histc_vs_torch_and_numpy(n, nbins, lo, hi):
    x = uniform((n,), 8, lo, hi)
    x[:3] = torch.tensor([lo, hi, (lo + hi) / 2])  # both edges are counted, max goes to the last bin
    got = O.histc(x.numpy(), nbins, lo, hi)
    want = torch.histc(x, nbins, lo, hi).numpy()
    assert np.array_equal(got, want)
    assert got.sum() == n
    if (lo, hi) == (0.0, 1.0):  # power-of-two bins: floor(v * nbins) is exact in fp32
        ref, _ = np.histogram(x.numpy().astype(np.float64), bins=nbins, range=(lo, hi))
        assert np.array_equal(got, ref.astype(np.float32))


def test_histc_ignores_out_of_range():
    x = torch.tensor([-0.5, 0.0, 0.999, 1.0, 1.5, float("nan")])
    got = O.histc(x.numpy(), 4, 0.0, 1.0)
    assert got.tolist() == [1.0, 0.0, 0.0, 2.0]


@pytest.mark.parametrize("shape", [(4, 3, 50), (32, 8, 784), (2, 5, 7)])
def test_bn_stats_vs_f64_and_torch(shape):
    x = normal(shape, 9)
    mean, inv = O.bn_stats(x.numpy(), 1e-5)
    m64, i64 = O.bn_stats_f64(x.numpy(), 1e-5)
    assert rel_err(mean, m64) < 1e-5 and rel_err(inv, i64) < 1e-5
    tm, ti = torch_bn_stats(x.reshape(shape[0], shape[1], shape[2], 1), 1e-5)
    assert rel_err(tm.numpy(), m64) < 1e-5 and rel_err(ti.numpy(), i64) < 1e-5
    # independent float64 witness of the two-pass oracle
    xd = x.double()
    assert np.allclose(m64, xd.mean(dim=(0, 2)).numpy(), rtol=1e-12)
    assert np.allclose(i64, 1.0 / np.sqrt(xd.var(dim=(0, 2), unbiased=False).numpy() + 1e-5), rtol=1e-12)


def test_bn_stats_invariants():
    c = torch.full((4, 2, 30), 3.5)
    mean, inv = O.bn_stats(c.numpy(), 1e-5)
    assert np.allclose(mean, 3.5) and np.allclose(inv, 1.0 / np.sqrt(1e-5), rtol=1e-6)
    x = normal((8, 3, 100), 10)
    m1, i1 = O.bn_stats(x.numpy(), 0.0)
    m2, i2 = O.bn_stats((x * 4.0 + 1.0).numpy(), 0.0)  # shift/scale equivariance
    assert rel_err(m2, m1 * 4.0 + 1.0) < 1e-5 and rel_err(i2, i1 / 4.0) < 1e-5
