"""GPU parity of the five tensor kernels, native and fused, through the C-ABI.
Bit-exact against the oracle / PyTorch CPU ops for im2col, max_pool (values and
int64 argmax), upsample and histogram counts; 1e-5 relative for batch-norm
mean / invstd (tolerance of the fp32 Welford tree against the fp64 two-pass)."""
import numpy as np
import os

import pytest
import torch

from hfuse_amd import _lib as L
from hfuse_amd import launcher as H
from oracle import oracle as O
from util import bilinear_tol, normal, pool_out, rel_err, torch_bn_stats, torch_im2col, torch_maxpool, uniform

pytestmark = pytest.mark.gpu
BN_TOL = 1e-5


# ------------------------------------------------------------------ helpers
class Im2col:
    def __init__(self, dev, n, c, h, w, k=(3, 3), p=(1, 1), s=(1, 1), d=(1, 1), seed=1):
        self.geom = (k, p, s, d)
        self.x = uniform((n, c, h, w), seed)
        hc = (h + 2 * p[0] - (d[0] * (k[0] - 1) + 1)) // s[0] + 1
        wc = (w + 2 * p[1] - (d[1] * (k[1] - 1) + 1)) // s[1] + 1
        self.xd = self.x.to(dev)
        self.out = torch.full((n, c * k[0] * k[1], hc * wc), float("nan"), device=dev)
        self.args = H.im2col_args(self.xd, self.out, k, p, s, d)

    def check(self):
        k, p, s, d = self.geom
        want = torch_im2col(self.x, k, p, s, d)
        got = self.out.cpu()
        assert torch.equal(got, want), f"im2col mismatch: {(got != want).sum().item()} of {want.numel()}"
        self.out.fill_(float("nan"))


class MaxPool:
    def __init__(self, dev, n, c, h, w, k, s, p, d=(1, 1), seed=2, x=None):
        self.geom = (k, s, p, d)
        self.x = uniform((n, c, h, w), seed) if x is None else x
        ph, pw = pool_out(h, k[0], s[0], p[0], d[0]), pool_out(w, k[1], s[1], p[1], d[1])
        self.xd = self.x.to(dev)
        self.val = torch.full((n, c, ph, pw), float("nan"), device=dev)
        self.idx = torch.full((n, c, ph, pw), -7, dtype=torch.int64, device=dev)
        self.args = H.maxpool_args(self.xd, self.val, self.idx, k, s, p, d)

    def check(self):
        k, s, p, d = self.geom
        tv, ti = torch_maxpool(self.x, k, s, p, d)
        assert torch.equal(self.idx.cpu(), ti), "argmax mismatch"
        assert np.array_equal(self.val.cpu().numpy(), tv.numpy(), equal_nan=True), "max value mismatch"
        self.val.fill_(float("nan"))
        self.idx.fill_(-7)


class Upsample:
    def __init__(self, dev, n, c, h, w, out_hw, seed=3):
        self.x = uniform((n, c, h, w), seed)
        self.out_hw = out_hw
        self.xd = self.x.to(dev)
        self.out = torch.full((n, c) + tuple(out_hw), float("nan"), device=dev)
        self.args = H.upsample_nearest_args(self.xd, self.out)

    def check(self):
        want = torch.nn.functional.interpolate(self.x, size=self.out_hw, mode="nearest")
        assert torch.equal(self.out.cpu(), want), "upsample mismatch"
        assert np.array_equal(self.out.cpu().numpy(), O.upsample_nearest2d(self.x.numpy(), self.out_hw))
        self.out.fill_(float("nan"))


class Bilinear:
    def __init__(self, dev, n, c, h, w, out_hw, align=False, seed=13):
        self.x = uniform((n, c, h, w), seed)
        self.out_hw, self.align = out_hw, align
        self.xd = self.x.to(dev)
        self.out = torch.full((n, c) + tuple(out_hw), float("nan"), device=dev)
        self.args = H.upsample_bilinear_args(self.xd, self.out, align)

    def check(self):
        got = self.out.cpu().numpy()
        assert np.array_equal(got, O.upsample_bilinear2d(self.x.numpy(), self.out_hw, self.align)), "bilinear mismatch"
        want = torch.nn.functional.interpolate(self.x, size=self.out_hw, mode="bilinear", align_corners=self.align)
        assert np.abs(got - want.numpy()).max() <= bilinear_tol(self.x.shape[2:], self.out_hw, self.align)
        self.out.fill_(float("nan"))


class BnStats:
    def __init__(self, dev, n, c, h, w, seed=4, x=None):
        self.x = normal((n, c, h, w), seed) if x is None else x
        self.xd = self.x.to(dev)
        self.mean = torch.full((c,), float("nan"), device=dev)
        self.inv = torch.full((c,), float("nan"), device=dev)
        self.args = H.bn_stats_args(self.xd, self.mean, self.inv, 1e-5, 0.0)

    def check(self):
        n, c = self.x.shape[:2]
        m64, i64 = O.bn_stats_f64(self.x.reshape(n, c, -1).numpy(), 1e-5)
        gm, gi = self.mean.cpu().numpy(), self.inv.cpu().numpy()
        assert rel_err(gm, m64) < BN_TOL, rel_err(gm, m64)
        assert rel_err(gi, i64) < BN_TOL, rel_err(gi, i64)
        tm, ti = torch_bn_stats(self.x, 1e-5)
        assert rel_err(gm, tm.numpy()) < 2 * BN_TOL and rel_err(gi, ti.numpy()) < 2 * BN_TOL
        self.mean.fill_(float("nan"))
        self.inv.fill_(float("nan"))


class Histc:
    def __init__(self, dev, n, nbins=1024, lo=0.0, hi=1.0, seed=5, x=None):
        self.x = uniform((n,), seed, lo, hi) if x is None else x
        self.p = (nbins, lo, hi)
        self.xd = self.x.to(dev)
        self.out = torch.zeros(nbins, device=dev)
        self.args = H.histc_args(self.xd, self.out, nbins, lo, hi)

    def check(self):
        nbins, lo, hi = self.p
        want = torch.histc(self.x, nbins, lo, hi)
        got = self.out.cpu()
        assert torch.equal(got, want), f"histogram mismatch in {(got != want).sum().item()} bins"
        assert np.array_equal(got.numpy(), O.histc(self.x.numpy(), nbins, lo, hi))
        self.out.zero_()


def sync():
    torch.cuda.synchronize()


# ------------------------------------------------------------------ native kernels
@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (1, 5, 12, 20), (32, 64, 56, 56)], ids=str)
def test_im2col_3x3(cuda, shape):
    t = Im2col(cuda, *shape)
    H.launch_native("im2col_kernel", t.args)
    sync()
    t.check()


@pytest.mark.parametrize("case", [
    (2, 3, 7, 9, (3, 2), (0, 1), (2, 1), (1, 1)),
    (2, 2, 11, 10, (2, 3), (2, 2), (1, 2), (2, 1)),
    (1, 1, 5, 5, (5, 5), (2, 2), (1, 1), (1, 1)),
    (3, 2, 9, 10, (3, 3), (1, 1), (1, 1), (1, 1)),  # width not a multiple of 4: general path
    (1, 2, 6, 8, (1, 1), (0, 0), (1, 1), (1, 1)),
], ids=str)
def test_im2col_general(cuda, case):
    n, c, h, w, k, p, s, d = case
    t = Im2col(cuda, n, c, h, w, k, p, s, d)
    H.launch_native("im2col_kernel", t.args, grid_blocks=3, block_threads=64)  # forces the stride loop
    sync()
    t.check()


@pytest.mark.parametrize("case", [
    (32, 64, 112, 112, (3, 3), (2, 2), (1, 1)),   # benchmark config 1
    (16, 128, 64, 64, (2, 2), (2, 2), (0, 0)),    # benchmark config 3
    (2, 3, 16, 24, (3, 3), (2, 2), (1, 1)),
    (1, 2, 8, 8, (2, 2), (2, 2), (0, 0)),
    (2, 3, 9, 7, (2, 2), (2, 2), (0, 0)),          # odd sizes: general path
    (2, 2, 13, 11, (3, 2), (1, 2), (1, 1)),
    (1, 1, 6, 6, (3, 3), (1, 1), (1, 1)),
], ids=str)
def test_maxpool(cuda, case):
    n, c, h, w, k, s, p = case
    t = MaxPool(cuda, n, c, h, w, k, s, p)
    H.launch_native("MaxPoolForward", t.args)
    sync()
    t.check()


@pytest.mark.parametrize("case", [
    (2, 3, 16, 24, (3, 3), (2, 2), (1, 1)),        # 3x3 / 2 / 1: two outputs per item
    (3, 5, 18, 20, (2, 2), (2, 2), (0, 0)),        # 2x2 / 2: two outputs per item, two items in flight per trip
    (1, 1, 2, 4, (2, 2), (2, 2), (0, 0)),          # a single item
    (4, 7, 30, 62, (2, 2), (2, 2), (0, 0)),
], ids=str)
@pytest.mark.parametrize("grid,block", [(1, 64), (3, 128), (2, 1024), (61, 256)])
def test_maxpool_on_fewer_threads_than_items(cuda, case, grid, block):
    """A caller's small grid makes every thread loop over its items; odd and even trip counts, and threads whose
    second item of a trip does not exist, give the same result as the one-item-per-thread launch."""
    n, c, h, w, k, s, p = case
    t = MaxPool(cuda, n, c, h, w, k, s, p, seed=grid + block)
    H.launch_native("MaxPoolForward", t.args, grid, block)
    sync()
    t.check()


def test_maxpool_dilated(cuda):
    t = MaxPool(cuda, 2, 2, 13, 11, (3, 2), (1, 2), (1, 1), (2, 1))
    H.launch_native("MaxPoolForward", t.args, grid_blocks=2, block_threads=64)
    sync()
    t.check()


@pytest.mark.parametrize("k,p", [((3, 3), (1, 1)), ((2, 2), (0, 0))])
def test_maxpool_ties_nan_inf(cuda, k, p):
    """Ties keep the first index; NaN wins; -inf planes return the first in-bounds element."""
    x = torch.full((2, 3, 16, 16), 0.25)
    x[0, 1] = float("-inf")
    x[1, 0, 5, 5] = float("nan")
    x[1, 0, 6, 6] = float("nan")
    x[1, 1, 3, 4] = float("inf")
    x[1, 2] = uniform((16, 16), 11).round(decimals=1)  # many exact ties
    t = MaxPool(cuda, 2, 3, 16, 16, k, (2, 2), p, x=x)
    H.launch_native("MaxPoolForward", t.args)
    sync()
    t.check()


@pytest.mark.parametrize("shape,out", [((32, 64, 56, 56), (112, 112)), ((2, 3, 8, 12), (16, 24)),
                                       ((2, 3, 5, 7), (10, 14)), ((1, 2, 4, 4), (7, 9)), ((1, 1, 6, 5), (3, 4))],
                         ids=str)
def test_upsample_nearest(cuda, shape, out):
    t = Upsample(cuda, *shape, out)
    H.launch_native("upsample_nearest2d_out_frame", t.args)
    sync()
    t.check()


@pytest.mark.parametrize("align", [False, True])
@pytest.mark.parametrize("shape,out", [((8, 16, 56, 56), (112, 112)), ((2, 3, 5, 7), (10, 14)), ((1, 2, 4, 4), (7, 9)),
                                       ((1, 1, 6, 5), (3, 4)), ((2, 2, 8, 12), (8, 12)), ((1, 2, 9, 9), (1, 1)),
                                       # exact 2x with an even input width: the shifted-lane path, rows of 1, 3, 65
                                       # and 100 work items so wavefront boundaries fall inside and between rows
                                       ((1, 1, 1, 2), (2, 4)), ((2, 3, 5, 6), (10, 12)), ((3, 2, 7, 130), (14, 260)),
                                       ((1, 5, 33, 200), (66, 400)), ((2, 2, 1, 64), (2, 128)),
                                       ((1, 1, 6, 8), (12, 24)), ((1, 1, 6, 8), (18, 16)),
                                       # more exact-2x shapes (with align_corners the sources drift by half a pixel across
                                       # the image; the rows and columns an output blends stay those of align_corners off)
                                       ((1, 1, 2, 2), (4, 4)), ((2, 3, 9, 14), (18, 28)), ((1, 2, 64, 66), (128, 132)),
                                       # two input rows per work item: one, two and three rows, wide and tall planes
                                       ((2, 2, 2, 4), (4, 8)), ((1, 3, 3, 8), (6, 16)), ((1, 1, 2, 4096), (4, 8192)),
                                       ((1, 1, 3001, 2), (6002, 4)), ((5, 1, 4, 2), (8, 4)),
                                       # four columns x four rows per work item: heights 1, 2, 3, 5, 13 leave partial row blocks
                                       ((3, 5, 7, 12), (13, 20)), ((2, 2, 3, 4), (1, 8)), ((1, 3, 2, 6), (2, 12)),
                                       ((1, 1, 4, 4), (3, 4)), ((2, 1, 9, 16), (5, 8)), ((4, 8, 28, 28), (56, 60))], ids=str)
def test_upsample_bilinear(cuda, shape, out, align):
    """Bit-exact against the oracle (no fused multiply-adds on either side), 2 ulp against PyTorch CPU."""
    t = Bilinear(cuda, *shape, out, align)
    H.launch_native("upsample_bilinear2d_out_frame", t.args)
    sync()
    t.check()


def test_upsample_bilinear_signed_zeros(cuda):
    """Bit patterns, not values: -0.0 inputs and the zero weights of the clamped edges."""
    x = uniform((2, 2, 6, 8), 23)
    x[x.abs() < 0.3] = 0.0
    x[(x > 0.3) & (x < 0.5)] = -0.0
    out = torch.empty((2, 2, 12, 16), device=cuda)
    H.launch_native("upsample_bilinear2d_out_frame", H.upsample_bilinear_args(x.to(cuda), out, False))
    sync()
    want = O.upsample_bilinear2d(x.numpy(), (12, 16), False)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("align", [False, True])
@pytest.mark.parametrize("offset", [1, 2, 3])
def test_upsample_bilinear_input_off_the_vector_boundary(cuda, offset, align):
    """An exact-2x shape whose input starts 4, 8 or 12 bytes past a 16-byte boundary: 8-byte-aligned inputs keep the
    shifted-lane path, the others take the gathered loads; the bits are the same either way."""
    n, c, h, w = 2, 3, 10, 12
    x = uniform((n * c * h * w + offset,), 41 + offset)
    xd = x.to(cuda)
    view = xd[offset:].view(n, c, h, w)
    out = torch.full((n, c, 2 * h, 2 * w), float("nan"), device=cuda)
    H.launch_native("upsample_bilinear2d_out_frame", H.upsample_bilinear_args(view, out, align))
    sync()
    want = O.upsample_bilinear2d(x[offset:].view(n, c, h, w).numpy(), (2 * h, 2 * w), align)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_upsample_bilinear_strided_output(cuda):
    x = uniform((2, 3, 6, 6), 17)
    xd = x.to(cuda)
    big = torch.zeros((2, 3, 12, 16), device=cuda)
    view = big[:, :, :, 2:14]
    H.launch_native("upsample_bilinear2d_out_frame", H.upsample_bilinear_args(xd, view, False))
    sync()
    assert np.array_equal(view.cpu().numpy(), O.upsample_bilinear2d(x.numpy(), (12, 12), False))
    assert float(big[:, :, :, :2].abs().sum()) == 0.0 and float(big[:, :, :, 14:].abs().sum()) == 0.0


def test_reference_ml_pairs_with_bilinear(cuda):
    """The four pairs of the reference's ml_fusion.yaml that contain the bilinear kernel."""
    from test_host_config import REFERENCE_ML_FUSION, REFERENCE_ML_KERNELS, REFERENCE_ML_PAIRS
    ref_cfg = H.Config(REFERENCE_ML_FUSION, REFERENCE_ML_KERNELS)
    made = []
    makers = {
        "im2col_kernel": lambda: Im2col(cuda, 2, 4, 12, 12),
        "MaxPoolForward": lambda: MaxPool(cuda, 2, 4, 16, 16, (3, 3), (2, 2), (1, 1)),
        "batch_norm_collect_statistics_kernel": lambda: BnStats(cuda, 4, 9, 6, 6),
        "upsample_bilinear2d_out_frame": lambda: Bilinear(cuda, 4, 8, 28, 28, (56, 56) if len(made) % 2 else (42, 60)),
        "kernelHistogram1D": lambda: Histc(cuda, 50000),
    }
    for i, (k1, k2) in enumerate(REFERENCE_ML_PAIRS):
        for preset, idx in (("hfuse", L.HF_SPLIT_TABLE), ("hfuse", 0), ("vfuse", L.HF_SPLIT_TABLE)):
            a, b = makers[k1](), makers[k2]()
            made.append(i)
            ref_cfg.plan(i, preset, idx).launch(a.args, b.args)
            sync()
            a.check()
            b.check()


@pytest.mark.parametrize("shape", [(32, 256, 28, 28), (4, 3, 5, 10), (2, 5, 7, 1), (3, 2, 3, 3), (64, 7, 4, 4)],
                         ids=str)
@pytest.mark.parametrize("block", [512, 64, 1024])
def test_bn_stats(cuda, shape, block):
    t = BnStats(cuda, *shape)
    H.launch_native("batch_norm_collect_statistics_kernel", t.args, block_threads=block)
    sync()
    t.check()


def test_bn_stats_fewer_blocks_than_planes_and_constant_input(cuda):
    t = BnStats(cuda, 4, 37, 6, 6)
    H.launch_native("batch_norm_collect_statistics_kernel", t.args, grid_blocks=5, block_threads=128)
    sync()
    t.check()
    c = BnStats(cuda, 4, 3, 8, 8, x=torch.full((4, 3, 8, 8), 3.5))
    H.launch_native("batch_norm_collect_statistics_kernel", c.args)
    sync()
    assert torch.allclose(c.mean.cpu(), torch.full((3,), 3.5))
    assert rel_err(c.inv.cpu().numpy(), np.full(3, 1.0 / np.sqrt(1e-5))) < BN_TOL


def test_bn_stats_strided_input(cuda):
    """A channel-sliced (non-contiguous) input goes down the general path."""
    big = normal((4, 10, 6, 5), 21)
    bd = big.to(cuda)
    view = bd[:, 2:7]
    mean = torch.empty(5, device=cuda)
    inv = torch.empty(5, device=cuda)
    a = L.BnStatsArgs()
    a.input.data = view.data_ptr()
    a.input.sizes[:] = [4, 5, 30]
    a.input.strides[:] = [view.stride(0), view.stride(1), 1]
    a.epsilon = 1e-5
    for acc, tt in ((a.save_mean, mean), (a.save_transformed_var, inv)):
        acc.data, acc.sizes[0], acc.strides[0] = tt.data_ptr(), 5, 1
    H.launch_native("batch_norm_collect_statistics_kernel", a)
    sync()
    m64, i64 = O.bn_stats_f64(big[:, 2:7].reshape(4, 5, 30).contiguous().numpy(), 1e-5)
    assert rel_err(mean.cpu().numpy(), m64) < BN_TOL and rel_err(inv.cpu().numpy(), i64) < BN_TOL


@pytest.mark.parametrize("n,nbins,lo,hi", [(1 << 20, 1024, 0.0, 1.0), (100003, 1024, 0.0, 1.0), (5000, 16, 0.0, 1.0),
                                           (70001, 256, -2.0, 2.0), (4096, 1, 0.0, 1.0), (3, 8, 0.0, 1.0)])
def test_histc(cuda, n, nbins, lo, hi):
    t = Histc(cuda, n, nbins, lo, hi)
    t.x[:3] = torch.tensor([lo, hi, (lo + hi) / 2])
    t.xd.copy_(t.x)
    H.launch_native("kernelHistogram1D", t.args)
    sync()
    t.check()


@pytest.mark.parametrize("offset", [1, 2, 3])
@pytest.mark.parametrize("n", [1, 2, 3, 5, 4099, 100001])
def test_histc_unaligned_input(cuda, offset, n):
    """A contiguous input that starts 4, 8 or 12 bytes past a 16-byte boundary still streams with
    16-byte loads; the elements before the boundary and the tail are counted by scalar loads."""
    x = uniform((n + offset,), 31 + n, 0.0, 1.0)
    xd = x.to(cuda)
    out = torch.zeros(64, device=cuda)
    H.launch_native("kernelHistogram1D", H.histc_args(xd[offset:], out, 64, 0.0, 1.0))
    sync()
    assert np.array_equal(out.cpu().numpy(), O.histc(x[offset:].numpy(), 64, 0.0, 1.0))


@pytest.mark.parametrize("block", [256, 1024])          # eight / four KiB-chunks in flight per wave
@pytest.mark.parametrize("grid", [1, 3, 256])
@pytest.mark.parametrize("n", [2047, 2048, 2049, 8191, 8192 * 5 + 3, 8192 * 4 * 7 + 4096 + 5])
def test_histc_chunk_boundaries(cuda, n, grid, block):
    """The input is read in per-wave chunks of four or eight KiB dealt over waves and workgroups; sizes one
    element either side of a chunk, fewer chunks than waves and more chunks than one pass of the grid all count every
    element once, with values outside the range (they go to a spare word of the table) mixed in."""
    x = uniform((n + 1,), 77 + n, -0.25, 1.25)
    x[::97] = float("nan")
    x[5::131] = float("inf")
    xd = x.to(cuda)
    for off in (0, 1):
        out = torch.zeros(100, device=cuda)
        view = xd[off:off + n]
        H.launch_native("kernelHistogram1D", H.histc_args(view, out, 100, 0.0, 1.0), grid, block)
        sync()
        want = O.histc(x[off:off + n].numpy(), 100, 0.0, 1.0)
        assert np.array_equal(out.cpu().numpy(), want), (off, int(np.abs(out.cpu().numpy() - want).sum()))


@pytest.mark.parametrize("nbins,lo,hi", [(1000, 0.0, 3.0), (7, -0.7, 0.0), (15360, 0.0, 10.0), (1024, 0.1, 0.9),
                                         (100, -5.0, 123.0), (3, 1e-3, 1e3), (1024, 0.0, 1.0),
                                         # power-of-two widths (the division is folded into the scale factor)
                                         (1000, -3.0, 5.0), (777, 0.25, 0.75), (15360, -1.0, 1.0), (5, 0.0, 2.0 ** -20),
                                         (1023, -2.0 ** 20, 2.0 ** 20)])
def test_histc_bin_edges_with_any_range(cuda, nbins, lo, hi):
    """Ranges whose width is not a power of two go through the real fp32 division of the bin
    formula.  The inputs sit on and one ulp either side of every bin edge (where the rounding
    of (v - lo) * nbins / (hi - lo) decides the bin) plus uniform draws."""
    k = np.arange(nbins + 1, dtype=np.float64)
    edges = (lo + k * (hi - lo) / nbins).astype(np.float32)
    parts = [edges, np.nextafter(edges, np.float32(np.inf)), np.nextafter(edges, np.float32(-np.inf)),
             np.nextafter(np.nextafter(edges, np.float32(np.inf)), np.float32(np.inf)),
             uniform((50000,), 77, lo, hi).numpy()]
    x = torch.from_numpy(np.concatenate(parts).astype(np.float32))
    t = Histc(cuda, x.numel(), nbins, lo, hi, x=x)
    H.launch_native("kernelHistogram1D", t.args)
    sync()
    got = t.out.cpu().numpy()
    assert np.array_equal(got, O.histc(x.numpy(), nbins, lo, hi))


@pytest.mark.parametrize("nbins,n", [(15361, 200000), (100000, 300000), (1 << 20, 50000)])
def test_histc_more_bins_than_lds_holds(cuda, nbins, n):
    """Beyond 15360 bins the counts go straight to global memory (the original also switches from
    shared to global memory by what fits); alone and fused with batch norm in every partition mode."""
    t = Histc(cuda, n, nbins, 0.0, 1.0)
    H.launch_native("kernelHistogram1D", t.args)
    sync()
    t.check()
    cfg = hfuse_amd_default()
    i = cfg.find_fusion("kernelHistogram1D", "batch_norm_collect_statistics_kernel")
    for mode in (None, L.HF_BARRIER_MATCHED, L.HF_BARRIER_BLOCKIDX):
        plan = cfg.plan(i)
        if mode is not None:
            plan.set_barrier_mode(mode)
        bn = BnStats(cuda, 4, 9, 6, 6)
        plan.launch(t.args, bn.args)
        sync()
        t.check()
        bn.check()


def hfuse_amd_default():
    import hfuse_amd
    return hfuse_amd.default_config()


def test_histc_out_of_range_and_accumulation(cuda):
    x = torch.tensor([-0.5, 0.0, 0.999, 1.0, 1.5, float("nan"), 0.3, 0.3])
    t = Histc(cuda, 8, 4, 0.0, 1.0, x=x)
    H.launch_native("kernelHistogram1D", t.args)
    H.launch_native("kernelHistogram1D", t.args)  # counts accumulate into `a`, as in the original
    sync()
    assert t.out.cpu().tolist() == [2.0, 4.0, 0.0, 4.0]


def test_histc_full_benchmark_size(cuda):
    n = 1 << 26
    g = torch.Generator().manual_seed(7)
    x = torch.rand(n, generator=g, dtype=torch.float32)
    t = Histc(cuda, n, 1024, 0.0, 1.0, x=x)
    H.launch_native("kernelHistogram1D", t.args)
    sync()
    assert t.out.sum().item() == n  # every element lands in exactly one bin
    t.check()


# ------------------------------------------------------------------ fused pairs
def _plans(cfg, k1, k2):
    i = cfg.find_fusion(k1, k2)
    plans = [("table", cfg.plan(i))]
    for idx in range(cfg.num_splits(i)):
        try:
            plans.append((f"idx{idx}", cfg.plan(i, "hfuse", idx)))
        except Exception:
            pass
    return plans


def test_fused_im2col_maxpool(cuda, cfg):
    for label, plan in _plans(cfg, "im2col_kernel", "MaxPoolForward"):
        for a, b in ((Im2col(cuda, 32, 64, 56, 56), MaxPool(cuda, 32, 64, 112, 112, (3, 3), (2, 2), (1, 1))),
                     (Im2col(cuda, 2, 3, 9, 10), MaxPool(cuda, 2, 3, 9, 7, (2, 2), (2, 2), (0, 0)))):
            plan.launch(a.args, b.args)
            sync()
            a.check()
            b.check()


def test_fused_bn_upsample(cuda, cfg):
    for label, plan in _plans(cfg, "batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame"):
        for a, b in ((BnStats(cuda, 32, 256, 28, 28), Upsample(cuda, 32, 64, 56, 56, (112, 112))),
                     (BnStats(cuda, 4, 37, 6, 5), Upsample(cuda, 1, 2, 4, 4, (7, 9)))):
            for grid in (0, 7):
                plan.launch(a.args, b.args, grid_blocks=grid)
                sync()
                a.check()
                b.check()


def test_fused_histc_maxpool(cuda, cfg):
    for label, plan in _plans(cfg, "kernelHistogram1D", "MaxPoolForward"):
        for a, b in ((Histc(cuda, 1 << 22), MaxPool(cuda, 16, 128, 64, 64, (2, 2), (2, 2), (0, 0))),
                     (Histc(cuda, 70001, 256, -2.0, 2.0), MaxPool(cuda, 2, 2, 13, 11, (3, 2), (1, 2), (1, 1)))):
            plan.launch(a.args, b.args)
            sync()
            a.check()
            b.check()


def test_fused_histc_maxpool_full_benchmark_size(cuda, cfg):
    """Benchmark configuration 3 at its full shape through the fused kernel: 2^26 values into 1024 bins
    next to max_pool2d [16,128,64,64] 2x2 s2; counts, values and argmax against PyTorch CPU and the oracle."""
    n = 1 << 26
    g = torch.Generator().manual_seed(11)
    x = torch.rand(n, generator=g, dtype=torch.float32)
    i = cfg.find_fusion("kernelHistogram1D", "MaxPoolForward")
    a, b = Histc(cuda, n, 1024, 0.0, 1.0, x=x), MaxPool(cuda, 16, 128, 64, 64, (2, 2), (2, 2), (0, 0))
    for plan in (cfg.plan(i), cfg.plan(i, "vfuse")):
        plan.launch(a.args, b.args)
        sync()
        assert a.out.sum().item() == n
        a.check()
        b.check()


def test_bounded_builds_at_every_wave_count(cuda, cfg):
    """The register-bounded builds of the thread partitions -- the benchmarked pairs at each of 5, 6, 7 and 8 waves
    per SIMD, three more shipped pairs at their formula's value and at 8 -- give the same bits as the plain build."""
    cases = [("im2col_kernel", "MaxPoolForward", lambda: Im2col(cuda, 4, 16, 56, 56),
              lambda: MaxPool(cuda, 4, 16, 112, 112, (3, 3), (2, 2), (1, 1)), (5, 6, 7, 8)),
             ("kernelHistogram1D", "MaxPoolForward", lambda: Histc(cuda, 1 << 20),
              lambda: MaxPool(cuda, 4, 32, 64, 64, (2, 2), (2, 2), (0, 0)), (5, 6, 7, 8)),
             ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame", lambda: BnStats(cuda, 8, 32, 28, 28),
              lambda: Upsample(cuda, 8, 16, 56, 56, (112, 112)), (5, 6, 7, 8)),
             ("im2col_kernel", "upsample_nearest2d_out_frame", lambda: Im2col(cuda, 4, 16, 56, 56),
              lambda: Upsample(cuda, 8, 16, 56, 56, (112, 112)), (6, 8)),
             ("im2col_kernel", "kernelHistogram1D", lambda: Im2col(cuda, 4, 16, 56, 56), lambda: Histc(cuda, 1 << 20), (7, 8)),
             ("im2col_kernel", "upsample_bilinear2d_out_frame", lambda: Im2col(cuda, 4, 16, 56, 56),
              lambda: Bilinear(cuda, 4, 16, 56, 56, (112, 112)), (6, 8))]
    for k1, k2, m1, m2, built in cases:
        plan = cfg.plan(cfg.find_fusion(k1, k2), "hfuse", 0)       # the thread partition at the table's shape
        plan.set_block(256, 256)
        for waves in built:
            plan.set_launch_waves(waves)
            assert plan.launch_waves[1] == waves
            a, b = m1(), m2()
            plan.launch(a.args, b.args)
            sync()
            a.check()
            b.check()


def test_three_kernel_fusions(cuda):
    """The reference's three-kernel lists (configs/im2col_maxpool_norm.yaml, maxpool_summary_norm.yaml) as one
    fused kernel each: horizontal at the shipped block shape, other shapes, a caller's grid, the vertical
    baseline; every output against PyTorch CPU and the oracle as for the pairs."""
    import hfuse_amd
    t = hfuse_amd.triples_config()
    i = t.find_fusion_n("im2col_kernel", "MaxPoolForward", "batch_norm_collect_statistics_kernel")
    j = t.find_fusion_n("MaxPoolForward", "kernelHistogram1D", "batch_norm_collect_statistics_kernel")
    shapes = [(lambda: Im2col(cuda, 32, 64, 56, 56), lambda: MaxPool(cuda, 32, 64, 112, 112, (3, 3), (2, 2), (1, 1)),
               lambda: BnStats(cuda, 32, 256, 28, 28)),
              (lambda: Im2col(cuda, 2, 3, 9, 10), lambda: MaxPool(cuda, 2, 3, 9, 7, (2, 2), (2, 2), (0, 0)),
               lambda: BnStats(cuda, 4, 37, 6, 5))]
    for mk in shapes:
        for preset, block, grid in (("hfuse", None, 0), ("hfuse", (512, 256, 256), 0), ("hfuse", (64, 64, 64), 0),
                                    ("hfuse", (128, 192, 704), 5), ("hfuse_lb", None, 0), ("vfuse", None, 0), ("vfuse_lb", None, 3)):
            plan = t.plan(i, preset)
            if block:
                plan.set_block_n(*block)
            a, b, c = (m() for m in mk)
            plan.launch_n([a.args, b.args, c.args], grid_blocks=grid)
            sync()
            a.check()
            b.check()
            c.check()
    for preset, block in (("hfuse", None), ("hfuse", (256, 512, 256)), ("vfuse", None)):
        plan = t.plan(j, preset)
        if block:
            plan.set_block_n(*block)
        for n in (1 << 22, 70001):
            a = MaxPool(cuda, 8, 32, 64, 64, (2, 2), (2, 2), (0, 0))
            b = Histc(cuda, n)
            c = BnStats(cuda, 8, 40, 14, 14)
            plan.launch_n([a.args, b.args, c.args])
            sync()
            a.check()
            b.check()
            c.check()
    # timing helper: natives back to back and the fused kernel both run the real kernels
    plan = t.plan(i)
    for mode in (2, 3):
        a, b, c = (m() for m in shapes[1])
        assert plan.time_n(mode, [[a.args, b.args, c.args]], 1, 2) > 0
        sync()
        a.check()
        b.check()
        c.check()
    with pytest.raises(H.HfuseError):
        plan.time_n(0, [[a.args, b.args, c.args]], 0, 1)
    # the launch-bound presets of a three-kernel list run its build bounded for 8 waves per SIMD
    assert t.plan(i, "hfuse_lb").launch_waves[1] == 8 and t.plan(i, "vfuse_lb").launch_waves[1] == 8 and t.plan(i).launch_waves[1] == 0
    # empty work in one part
    a, c = Im2col(cuda, 2, 3, 9, 10), BnStats(cuda, 4, 37, 6, 5)
    b = MaxPool(cuda, 2, 3, 9, 7, (2, 2), (2, 2), (0, 0))
    plan.launch_n([a.args, b.args, c.args], grid_blocks=1)
    sync()
    a.check(); b.check(); c.check()


@pytest.mark.parametrize("order", [(2, 0, 1), (1, 2, 0), (2, 1, 0), (0, 2, 1)])
def test_three_kernel_lists_in_any_order(cuda, order):
    """The Context partitions a block among the kernels in the order the list names them
    (include/KernelFusion.h:45-80): the reference's three-kernel lists with their kernels permuted run the same
    instantiation with other thread bounds, the arguments following the list's order."""
    import hfuse_amd
    kernels = open(os.path.join(hfuse_amd.CONFIG_DIR, "gfx950_kernels.yaml")).read()
    lists = [("im2col_kernel", "MaxPoolForward", "batch_norm_collect_statistics_kernel"),
             ("MaxPoolForward", "kernelHistogram1D", "batch_norm_collect_statistics_kernel")]
    make = {"im2col_kernel": lambda: Im2col(cuda, 4, 16, 24, 24),
            "MaxPoolForward": lambda: MaxPool(cuda, 4, 16, 48, 48, (3, 3), (2, 2), (1, 1)),
            "batch_norm_collect_statistics_kernel": lambda: BnStats(cuda, 4, 37, 6, 8),
            "kernelHistogram1D": lambda: Histc(cuda, 300001)}
    for names in lists:
        listed = [names[k] for k in order]
        text = "- File: permuted\n  Kernels:\n" + "".join(f"    - {k}\n" for k in listed) + "  Blocks: [128, 256, 192]\n"
        cfg = H.Config(text, kernels)
        for preset, grid in (("hfuse", 0), ("hfuse", 7), ("vfuse", 0), ("hfuse_lb", 0)):
            plan = cfg.plan(0, preset)
            q = plan.partition_n
            if preset != "vfuse":
                assert list(q.lo)[:3] == [0, 128, 384] and list(q.hi)[:3] == [128, 384, 576]
            work = [make[k]() for k in listed]
            plan.launch_n([w.args for w in work], grid_blocks=grid)
            sync()
            for w in work:
                w.check()


def test_time_pair_continues_the_rotation(cuda, cfg):
    """hf_time_pair's first_set: repetition r uses set (first_set + r) % nsets, so short calls chained
    through a Rotation touch every set.  Three sets of a tiny histogram; each launch adds its set's
    element count to that set's bins, which shows which sets ran."""
    i = cfg.find_fusion("kernelHistogram1D", "MaxPoolForward")
    plan = cfg.plan(i)
    hs = [Histc(cuda, 1000 * (k + 1), 16, 0.0, 1.0, seed=50 + k) for k in range(3)]
    ps = [MaxPool(cuda, 1, 1, 8, 8, (2, 2), (2, 2), (0, 0), seed=60 + k) for k in range(3)]
    a1, a2 = [h.args for h in hs], [p.args for p in ps]
    rot = H.Rotation()
    plan.time(3, a1, a2, 0, 1, rotation=rot)       # set 0
    plan.time(3, a1, a2, 1, 1, rotation=rot)       # warm-up on set 1, timed on set 2
    sync()
    assert [h.out.sum().item() for h in hs] == [1000.0, 2000.0, 3000.0]
    plan.time(0, a1, a2, 0, 2, rotation=rot)       # native histogram on sets 0 and 1
    sync()
    assert [h.out.sum().item() for h in hs] == [2000.0, 4000.0, 3000.0]
    assert rot.cursor == 2
    with pytest.raises(H.HfuseError):
        check = H.check
        import ctypes as C
        n = 3
        p1 = (C.c_void_p * n)(*[C.addressof(a) for a in a1])
        p2 = (C.c_void_p * n)(*[C.addressof(a) for a in a2])
        ms = C.c_float()
        check(H.L.lib().hf_time_pair(plan._h, 3, p1, p2, n, 3, 0, 1, 0, None, C.byref(ms)))   # first_set out of range


@pytest.mark.parametrize("lend", [True, False])
def test_wave_lending_gives_identical_results(cuda, cfg, lend):
    """Blocks beyond one half's grid: with lending the idle half runs the partner's body,
    without it those waves end at once; both must produce the same bits."""
    cases = [
        ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame",
         lambda: BnStats(cuda, 8, 5, 14, 14), lambda: Upsample(cuda, 8, 16, 28, 28, (56, 56))),
        ("upsample_nearest2d_out_frame", "batch_norm_collect_statistics_kernel",
         lambda: Upsample(cuda, 8, 16, 28, 28, (56, 56)), lambda: BnStats(cuda, 8, 5, 14, 14)),
        ("kernelHistogram1D", "MaxPoolForward",
         lambda: Histc(cuda, 30000), lambda: MaxPool(cuda, 8, 32, 64, 64, (2, 2), (2, 2), (0, 0))),
        ("im2col_kernel", "MaxPoolForward",
         lambda: Im2col(cuda, 1, 2, 8, 8), lambda: MaxPool(cuda, 8, 32, 64, 64, (3, 3), (2, 2), (1, 1))),
        ("im2col_kernel", "MaxPoolForward",
         lambda: Im2col(cuda, 8, 16, 56, 56), lambda: MaxPool(cuda, 1, 2, 8, 8, (2, 2), (2, 2), (0, 0))),
    ]
    for k1, k2, m1, m2 in cases:
        plan = cfg.plan(cfg.find_fusion(k1, k2))
        plan.set_lending(lend)
        for grids in ((0, 0), (3, 11), (11, 3)):
            plan.set_grids(*grids)
            a, b = m1(), m2()
            plan.launch(a.args, b.args)
            sync()
            a.check()
            b.check()


@pytest.mark.parametrize("block", [(64, 64), (128, 384), (512, 512), (256, 768), (960, 64)])
def test_fused_block_shapes(cuda, cfg, block):
    """Every legal shape of the fused block gives the same bits (all three benchmarked tensor pairs)."""
    cases = [
        ("im2col_kernel", "MaxPoolForward",
         lambda: Im2col(cuda, 4, 16, 56, 56), lambda: MaxPool(cuda, 4, 16, 112, 112, (3, 3), (2, 2), (1, 1))),
        ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame",
         lambda: BnStats(cuda, 16, 24, 28, 28), lambda: Upsample(cuda, 4, 16, 56, 56, (112, 112))),
        ("kernelHistogram1D", "MaxPoolForward",
         lambda: Histc(cuda, 1 << 21), lambda: MaxPool(cuda, 4, 32, 64, 64, (2, 2), (2, 2), (0, 0))),
    ]
    for k1, k2, m1, m2 in cases:
        plan = cfg.plan(cfg.find_fusion(k1, k2))
        plan.set_block(*block)
        assert plan.partition.launch_threads == sum(block)
        a, b = m1(), m2()
        plan.launch(a.args, b.args)
        sync()
        a.check()
        b.check()


@pytest.mark.parametrize("preset", ["vfuse", "vfuse_lb"])
def test_vertical_baseline_presets(cuda, cfg, preset):
    """The reference's baseline: the same threads run kernel 1, then kernel 2 (block = max(d1, d2))."""
    cases = [
        ("im2col_kernel", "MaxPoolForward",
         lambda: Im2col(cuda, 4, 16, 56, 56), lambda: MaxPool(cuda, 4, 16, 112, 112, (3, 3), (2, 2), (1, 1))),
        ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame",
         lambda: BnStats(cuda, 16, 24, 28, 28), lambda: Upsample(cuda, 4, 16, 56, 56, (112, 112))),
        ("kernelHistogram1D", "MaxPoolForward",
         lambda: Histc(cuda, 1 << 21), lambda: MaxPool(cuda, 4, 32, 64, 64, (2, 2), (2, 2), (0, 0))),
        ("kernelHistogram1D", "batch_norm_collect_statistics_kernel",
         lambda: Histc(cuda, 1 << 20), lambda: BnStats(cuda, 8, 64, 14, 14)),
    ]
    for k1, k2, m1, m2 in cases:
        plan = cfg.plan(cfg.find_fusion(k1, k2), preset)
        part = plan.partition
        assert list(part.lo) == [0, 0] and part.launch_threads == max(part.hi)
        for grid in (0, 5):
            a, b = m1(), m2()
            plan.launch(a.args, b.args, grid_blocks=grid)
            sync()
            a.check()
            b.check()


def test_fused_barrier_modes(cuda, cfg):
    """hist + bn both synchronise: subset counters, the shared hardware barrier and the
    blockIdx fallback must all give the same results."""
    i = cfg.find_fusion("kernelHistogram1D", "batch_norm_collect_statistics_kernel")
    for mode in (L.HF_BARRIER_SUBSET, L.HF_BARRIER_MATCHED, L.HF_BARRIER_BLOCKIDX):
        plan = cfg.plan(i)
        plan.set_barrier_mode(mode)
        a, b = Histc(cuda, 1 << 20), BnStats(cuda, 8, 64, 14, 14)
        plan.launch(a.args, b.args)
        sync()
        a.check()
        b.check()
    j = cfg.find_fusion("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame")
    plan = cfg.plan(j)
    plan.set_barrier_mode(L.HF_BARRIER_BLOCKIDX)
    a, b = BnStats(cuda, 8, 64, 14, 14), Upsample(cuda, 4, 8, 28, 28, (56, 56))
    plan.launch(a.args, b.args)
    sync()
    a.check()
    b.check()


def test_every_shipped_tensor_pair(cuda, cfg):
    """All tensor pairs of the shipped fusion list, small shapes, default split."""
    makers = {
        "im2col_kernel": lambda: Im2col(cuda, 2, 4, 12, 12),
        "MaxPoolForward": lambda: MaxPool(cuda, 2, 4, 16, 16, (3, 3), (2, 2), (1, 1)),
        "batch_norm_collect_statistics_kernel": lambda: BnStats(cuda, 4, 9, 6, 6),
        "upsample_nearest2d_out_frame": lambda: Upsample(cuda, 2, 3, 8, 8, (16, 16)),
        "kernelHistogram1D": lambda: Histc(cuda, 50000),
    }
    n = 0
    for i, (_, k1, k2) in enumerate(cfg.fusions()):
        if k1 in makers and k2 in makers:
            a, b = makers[k1](), makers[k2]()
            cfg.plan(i).launch(a.args, b.args)
            sync()
            a.check()
            b.check()
            # the register-bounded build of the same pair, horizontal and vertical
            for preset in ("hfuse", "vfuse"):
                plan = cfg.plan(i, preset)
                plan.set_launch_bound(True)
                a, b = makers[k1](), makers[k2]()
                plan.launch(a.args, b.args)
                sync()
                a.check()
                b.check()
            n += 1
    assert n == 11  # the ten pairs of the reference list plus bn+upsample in benchmark order


def test_time_pair_modes_leave_correct_results(cuda, cfg):
    """All five timing modes (natives, back to back, fused, two streams) run the real kernels."""
    i = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    plan = cfg.plan(i)
    for mode in range(5):
        a, b = Im2col(cuda, 2, 4, 12, 12), MaxPool(cuda, 2, 4, 16, 16, (3, 3), (2, 2), (1, 1))
        assert plan.time(mode, [a.args], [b.args], 1, 3) > 0
        sync()
        if mode != 1:
            a.check()
        if mode != 0:
            b.check()
    with pytest.raises(H.HfuseError):
        plan.time(5, [a.args], [b.args], 0, 1)


def test_empty_work_is_a_no_op(cuda, cfg):
    """Zero work items (im2col with n = 0, a histogram of nothing) return without touching their
    outputs, alone and as one half of a fused launch; kernels whose PyTorch callers refuse empty
    tensors (pooling, upsampling) refuse them here too."""
    buf = torch.zeros(4096, device=cuda)
    out = torch.full((4096,), 7.0, device=cuda)
    a = H.im2col_args(buf[:64].reshape(1, 8, 8), out)
    a.n = 0
    H.launch_native("im2col_kernel", a)
    h = H.histc_args(buf[:64], out[:16], 16, 0.0, 1.0)
    h.total_elements = 0
    h.b.sizes[0] = 0
    H.launch_native("kernelHistogram1D", h)
    sync()
    assert float(out.min()) == 7.0 and float(out.max()) == 7.0
    idx = torch.zeros(16, dtype=torch.int64, device=cuda)
    m = H.maxpool_args(buf[:64].reshape(1, 1, 8, 8), out[:16].reshape(1, 1, 4, 4), idx.reshape(1, 1, 4, 4),
                       (2, 2), (2, 2), (0, 0))
    m.nthreads = 0
    m.num = 0
    u = H.upsample_nearest_args(buf[:64].reshape(1, 1, 8, 8), out[:256].reshape(1, 1, 16, 16))
    u.nc = 0
    for name, args in (("MaxPoolForward", m), ("upsample_nearest2d_out_frame", u)):
        with pytest.raises(H.HfuseError) as e:
            H.launch_native(name, args)
        assert e.value.code == L.HF_EINVAL
    # an empty half next to a working one, thread partition and block-index partition
    i = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    j = cfg.find_fusion("kernelHistogram1D", "MaxPoolForward")
    for mode in (None, L.HF_BARRIER_BLOCKIDX):
        for fusion, empty in ((i, a), (j, h)):
            plan = cfg.plan(fusion)
            if mode is not None:
                plan.set_barrier_mode(mode)
            pool = MaxPool(cuda, 2, 4, 16, 16, (2, 2), (2, 2), (0, 0))
            plan.launch(empty, pool.args)
            sync()
            pool.check()
    assert float(out.min()) == 7.0 and float(out.max()) == 7.0


def test_launches_can_be_captured_in_a_graph(cuda, cfg):
    """Native and fused launches only enqueue kernels on the caller's stream (no allocation, no
    synchronisation, no memset), so a stream capture records them; every replay must give the
    eager result, with eager work and synchronisations between the replays."""
    i = cfg.find_fusion("kernelHistogram1D", "batch_norm_collect_statistics_kernel")
    j = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    hist, bn = Histc(cuda, 100000), BnStats(cuda, 4, 9, 6, 6)
    col, pool = Im2col(cuda, 2, 4, 12, 12), MaxPool(cuda, 2, 4, 16, 16, (3, 3), (2, 2), (1, 1))
    up = Upsample(cuda, 2, 3, 8, 8, (16, 16))
    p1, p2 = cfg.plan(i), cfg.plan(j)
    p1.launch(hist.args, bn.args)          # warm-up outside the capture (first-use initialisation)
    p2.launch(col.args, pool.args)
    H.launch_native("upsample_nearest2d_out_frame", up.args)
    sync()
    side = torch.cuda.Stream()             # default priority
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            hist.out.zero_()               # a fill kernel, not a memset node
            p1.launch(hist.args, bn.args)
            p2.launch(col.args, pool.args)
            H.launch_native("upsample_nearest2d_out_frame", up.args)
    for t in (hist, bn, col, pool, up):    # the warm-up results; check() also scrubs the outputs
        t.check()
    hist.out.fill_(5.0)                    # the captured fill kernel has to clear this
    for replay in range(3):
        graph.replay()
        sync()
        for t in (hist, bn, col, pool, up):
            t.check()                      # eager copies, comparisons and fills between the replays


def test_three_kernel_launch_can_be_captured_in_a_graph(cuda):
    """hf_launch_fused_n only enqueues one kernel as well: captured, then replayed three times with eager work between."""
    import hfuse_amd
    t = hfuse_amd.triples_config()
    plan = t.plan(t.find_fusion_n("MaxPoolForward", "kernelHistogram1D", "batch_norm_collect_statistics_kernel"))
    pool, hist, bn = MaxPool(cuda, 2, 4, 16, 16, (2, 2), (2, 2), (0, 0)), Histc(cuda, 50000), BnStats(cuda, 4, 9, 6, 6)
    plan.launch_n([pool.args, hist.args, bn.args])   # warm-up outside the capture
    sync()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            hist.out.zero_()                         # a fill kernel, not a memset node
            plan.launch_n([pool.args, hist.args, bn.args])
    for x in (pool, hist, bn):
        x.check()
    hist.out.fill_(3.0)
    for replay in range(3):
        graph.replay()
        sync()
        for x in (pool, hist, bn):
            x.check()


# ------------------------------------------------------------------ sizes at and beyond 2^31 elements
# The general loops use 32-bit indices below 2^31 elements and 64-bit ones from there on.  These
# cases sit above the limit; the expected values come from PyTorch's own GPU operators (at these
# sizes a CPU run of the oracle would take minutes), so they are cross-checks, not oracle parity.
def test_upsample_nearest_beyond_2_31_elements(cuda):
    x = torch.rand((1 << 13, 1 << 6, 1 << 10), device=cuda)          # 2^29 elements, 2 GiB
    out = torch.empty((1 << 13, 1 << 6, 1 << 12), device=cuda)       # 2^31 elements, 8 GiB
    a = H.upsample_nearest_args(x.unsqueeze(0), out.unsqueeze(0))
    H.launch_native("upsample_nearest2d_out_frame", a)
    sync()
    for lo in range(0, 1 << 13, 1 << 10):                            # closed form: out[.., x] = in[.., x // 4]
        assert torch.equal(out[lo:lo + (1 << 10)], x[lo:lo + (1 << 10)].repeat_interleave(4, dim=-1))
    del x, out
    torch.cuda.empty_cache()


def test_maxpool_beyond_2_31_elements(cuda):
    x = torch.rand((8, 1 << 10, 512, 512), device=cuda)              # 2^31 elements, 8 GiB
    val = torch.empty((8, 1 << 10, 256, 256), device=cuda)
    idx = torch.empty((8, 1 << 10, 256, 256), dtype=torch.int64, device=cuda)
    H.launch_native("MaxPoolForward", H.maxpool_args(x, val, idx, (2, 2), (2, 2), (0, 0)))
    sync()
    for n in range(8):
        tv, ti = torch.nn.functional.max_pool2d(x[n], (2, 2), (2, 2), 0, return_indices=True)
        assert torch.equal(val[n], tv) and torch.equal(idx[n], ti)
    del x, val, idx
    torch.cuda.empty_cache()


def test_im2col_beyond_2_31_elements(cuda):
    x = torch.rand((64, 64, 256, 256), device=cuda)                  # 2^28 elements; 9 x that = 2.4e9 columns
    col = torch.empty((64, 576, 65536), device=cuda)
    H.launch_native("im2col_kernel", H.im2col_args(x, col))
    sync()
    for n in range(0, 64, 8):
        assert torch.equal(col[n:n + 8], torch.nn.functional.unfold(x[n:n + 8], 3, padding=1))
    del x, col
    torch.cuda.empty_cache()


def test_two_host_threads_on_their_own_streams(cuda, cfg):
    """The C-ABI is thread-compatible: one plan per thread, launches on the thread's own stream
    (ctypes drops the GIL during a call, so the two threads really overlap in the library)."""
    import threading
    errors = []

    def worker(seed, fusion, make_a, make_b):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                plan = cfg.plan(fusion)
                for rep in range(20):
                    a, b = make_a(seed + rep), make_b(seed + rep)
                    plan.launch(a.args, b.args, stream=stream)
                    H.launch_native("upsample_nearest2d_out_frame", up[seed % 2].args, stream=stream)
                    stream.synchronize()
                    a.check()
                    b.check()
        except Exception as e:  # surfaced in the main thread below
            errors.append(e)

    up = [Upsample(cuda, 2, 3, 8, 8, (16, 16), seed=40), Upsample(cuda, 2, 3, 8, 8, (16, 16), seed=41)]
    i = cfg.find_fusion("im2col_kernel", "MaxPoolForward")
    j = cfg.find_fusion("kernelHistogram1D", "batch_norm_collect_statistics_kernel")
    t1 = threading.Thread(target=worker, args=(100, i, lambda s: Im2col(cuda, 2, 4, 12, 12, seed=s),
                                               lambda s: MaxPool(cuda, 2, 4, 16, 16, (3, 3), (2, 2), (1, 1), seed=s)))
    t2 = threading.Thread(target=worker, args=(201, j, lambda s: Histc(cuda, 50000, seed=s), lambda s: BnStats(cuda, 4, 9, 6, 6, seed=s)))
    t1.start()
    t2.start()
    t1.join()
    t2.join()
    assert not errors, errors
    sync()
    for u in up:
        u.check()


def test_random_fused_configurations(cuda, cfg):
    """Seeded random walk over the tensor pairs of the shipped list: random small shapes (fast and
    general paths), fused block shapes, lending on / off, every partition mode legal for the pair,
    per-half grids; every launch is checked against the oracle / PyTorch CPU like the native kernels."""
    import random
    rng = random.Random(0xF05E)

    def rand_im2col():
        k = rng.choice([(3, 3), (3, 3), (1, 1), (2, 3), (5, 5)])
        p = (1, 1) if k == (3, 3) and rng.random() < 0.7 else (rng.randint(0, k[0] // 2), rng.randint(0, k[1] // 2))
        s = (1, 1) if rng.random() < 0.7 else (rng.randint(1, 2), rng.randint(1, 2))
        h, w = rng.randint(5, 14), rng.choice([8, 12, 16, 7, 9, 13])
        return Im2col(cuda, rng.randint(1, 3), rng.randint(1, 5), h, w, k, p, s, (1, 1), seed=rng.randint(0, 999))

    def rand_pool():
        k, s, p = rng.choice([((3, 3), (2, 2), (1, 1)), ((2, 2), (2, 2), (0, 0)), ((3, 2), (1, 2), (1, 0)), ((2, 2), (1, 1), (1, 1))])
        h, w = rng.choice([8, 12, 16, 9, 11]), rng.choice([8, 16, 24, 10, 13])
        return MaxPool(cuda, rng.randint(1, 3), rng.randint(1, 4), h, w, k, s, p, seed=rng.randint(0, 999))

    class BnStatsSmall(BnStats):
        """Planes of a few elements can have a mean next to zero, where an element-wise relative error
        says nothing; the mean is held to 1e-5 of the plane's scale max(|mean|, std) instead."""

        def check(self):
            n, c = self.x.shape[:2]
            m64, i64 = O.bn_stats_f64(self.x.reshape(n, c, -1).numpy(), 1e-5)
            gm, gi = self.mean.cpu().numpy().astype(np.float64), self.inv.cpu().numpy()
            assert np.max(np.abs(gm - m64) / np.maximum(np.abs(m64), 1.0 / i64)) < BN_TOL
            assert rel_err(gi, i64) < BN_TOL, rel_err(gi, i64)
            self.mean.fill_(float("nan"))
            self.inv.fill_(float("nan"))

    def rand_bn():
        return BnStatsSmall(cuda, rng.randint(1, 5), rng.randint(1, 12), rng.randint(1, 7), rng.choice([1, 3, 4, 8]), seed=rng.randint(0, 999))

    def rand_up():
        h, w = rng.randint(1, 9), rng.choice([2, 4, 6, 8, 5, 7])
        out = (2 * h, 2 * w) if rng.random() < 0.6 else (rng.randint(1, 20), rng.randint(1, 20))
        return Upsample(cuda, rng.randint(1, 3), rng.randint(1, 4), h, w, out, seed=rng.randint(0, 999))

    def rand_bilinear():
        h, w = rng.randint(1, 9), rng.choice([2, 4, 6, 8, 5, 7])
        out = (2 * h, 2 * w) if rng.random() < 0.5 else (rng.randint(1, 20), rng.choice([4, 8, 12, 5, 9]))
        return Bilinear(cuda, rng.randint(1, 3), rng.randint(1, 4), h, w, out, align=rng.random() < 0.5, seed=rng.randint(0, 999))

    def rand_hist():
        nbins, lo, hi = rng.choice([(1024, 0.0, 1.0), (16, 0.0, 1.0), (100, -1.0, 2.0), (7, 0.0, 3.0)])
        return Histc(cuda, rng.choice([1, 63, 1000, 40001]), nbins, lo, hi, seed=rng.randint(0, 999))

    makers = {"im2col_kernel": rand_im2col, "MaxPoolForward": rand_pool, "batch_norm_collect_statistics_kernel": rand_bn,
              "upsample_nearest2d_out_frame": rand_up, "upsample_bilinear2d_out_frame": rand_bilinear, "kernelHistogram1D": rand_hist}
    sync_kernels = {"batch_norm_collect_statistics_kernel", "kernelHistogram1D"}
    pairs = [(i, k1, k2) for i, (_, k1, k2) in enumerate(cfg.fusions()) if k1 in makers and k2 in makers]
    assert len(pairs) == 15
    launched = 0
    for case in range(120):
        i, k1, k2 = rng.choice(pairs)
        a, b = makers[k1](), makers[k2]()
        plan = cfg.plan(i, rng.choice(["hfuse", "hfuse", "hfuse_lb", "vfuse"]))
        label = f"case {case}: {k1} + {k2}"
        if not plan.name.count("vfuse"):
            y1 = cfg.kernel(k1).block_dim.y
            y2 = cfg.kernel(k2).block_dim.y
            t1 = 64 * rng.randint(1, 8)
            t2 = 64 * rng.randint(1, (1024 - t1) // 64)
            if t1 % y1 == 0 and t2 % y2 == 0 and rng.random() < 0.8:
                plan.set_block(t1, t2)
                label += f" block {t1}+{t2}"
            plan.set_lending(rng.random() < 0.5)
            modes = [None, L.HF_BARRIER_BLOCKIDX]
            if k1 in sync_kernels and k2 in sync_kernels:
                modes.append(L.HF_BARRIER_MATCHED)
            mode = rng.choice(modes)
            if mode is not None:
                plan.set_barrier_mode(mode)
                label += f" mode {mode}"
            if rng.random() < 0.3:
                g = (rng.randint(1, 40), rng.randint(1, 40))
                plan.set_grids(*g)
                label += f" grids {g}"
        plan.launch(a.args, b.args, grid_blocks=rng.choice([0, 0, 0, 3, 17]))
        sync()
        try:
            a.check()
            b.check()
        except AssertionError as e:
            raise AssertionError(f"{label}: {e}") from e
        launched += 1
    assert launched == 120
