"""Pins of the fusion model: hand-worked numbers from the reference's own YAML
tables (configs/ml_kernels.yaml, configs/crypto_kernels.yaml) pushed through the
rules of include/KernelFusion.h:45-80, main.cpp:215-227, KernelPrinter.cpp:42-66
and ThreadInfoRewriter.cpp:38-58 -- worked by hand here, not by calling the code
under test twice."""
import itertools

import pytest

from oracle import oracle as O

# rows of configs/ml_kernels.yaml / crypto_kernels.yaml: (BlockDim, Reg, ExecTime)
IM2COL = ((512, 1, 1), 49, 31.0)
MAXPOOL = ((256, 1, 1), 24, 95.0)
UPSAMPLE = ((512, 1, 1), 43, 77.0)
HIST = ((512, 1, 1), 32, 1.0)
BN = ((32, 16, 1), 24, 52.0)
ETHASH = ((128, 1, 1), 130, -1.0)
SIA = ((128, 1, 1), 64, -1.0)


def test_context_exectime_resplit_granule_32():
    # 31/(31+95) * 768 / 32 = 5.904 -> 5 * 32 = 160 threads; MaxPool takes 608
    p = O.context([IM2COL, MAXPOOL], imbalanced=True)
    assert (p.lo[0], p.hi[0], p.lo[1], p.hi[1]) == (0, 160, 160, 768)
    assert p.block_dim[0].x == 160 and p.block_dim[1].x == 608
    # upsample 77 : bn 52 over 1024 threads: int(77/129*32) = 19 -> 608; bn rest 416 -> X = 416/16 = 26
    p = O.context([UPSAMPLE, BN], imbalanced=True)
    assert (p.hi[0], p.hi[1]) == (608, 1024)
    assert (p.block_dim[1].x, p.block_dim[1].y) == (26, 16)
    # histogram's ExecTime 1 against 95 leaves it no thread at all: int(1/96*24) = 0; the printer
    # would then divide by a block size of zero (KernelPrinter.cpp:49), the oracle refuses instead
    with pytest.raises(ValueError):
        O.context([HIST, MAXPOOL], imbalanced=True)


def test_context_balanced_and_baseline_bounds():
    p = O.context([IM2COL, MAXPOOL], imbalanced=False)
    assert (p.lo[0], p.hi[0], p.lo[1], p.hi[1]) == (0, 512, 512, 768) and p.launch_threads == 768
    p = O.context([IM2COL, MAXPOOL], base_line=True, imbalanced=False)
    assert (p.lo[0], p.hi[0], p.lo[1], p.hi[1]) == (0, 512, 0, 256) and p.launch_threads == 512


def test_launch_bounds_of_the_printer():
    # 65536/49/512 = 2, 65536/24/256 = 10, cap 2048/768 = 2
    p = O.context([IM2COL, MAXPOOL], launch_bound=True, imbalanced=False)
    assert (p.launch_threads, p.launch_blocks) == (768, 2)
    # ethash 65536/130/128 = 3, sia 65536/64/128 = 8, cap 2048/256 = 8
    p = O.context([ETHASH, SIA], launch_bound=True, imbalanced=False)
    assert (p.launch_threads, p.launch_blocks) == (256, 3)
    p = O.context([ETHASH, SIA], launch_bound=False, imbalanced=False)
    assert p.launch_blocks == 0


def test_split_enumeration_of_the_driver():
    # Split = 128, 256, ... < d1 + d2; the first kernel gets exactly Split threads
    assert O.enumerate_splits([IM2COL, MAXPOOL]) == [128, 256, 384, 512, 640]
    assert O.enumerate_splits([UPSAMPLE, BN]) == [128, 256, 384, 512, 640, 768, 896]
    assert O.enumerate_splits([ETHASH, SIA]) == [128]
    assert O.enumerate_splits([IM2COL, MAXPOOL], granule=64) == [128, 256, 384, 512, 640]


def test_remap_is_the_documented_formula_and_a_bijection():
    # bn half of upsample+bn at the table split: threads 512..1023 as a (32,16) block
    assert O.remap_tid(512, 512, (32, 16, 1)) == (0, 0, 0)
    assert O.remap_tid(512 + 33, 512, (32, 16, 1)) == (1, 1, 0)
    assert O.remap_tid(1023, 512, (32, 16, 1)) == (31, 15, 0)
    assert O.remap_tid(1 + 4 * 1 + 4 * 2 * 1, 0, (4, 2, 3)) == (1, 1, 1)
    for dim, lo in (((32, 16, 1), 512), ((64, 8, 1), 0), ((4, 2, 3), 128)):
        n = dim[0] * dim[1] * dim[2]
        seen = {O.remap_tid(lo + t, lo, dim) for t in range(n)}
        assert seen == set(itertools.product(range(dim[0]), range(dim[1]), range(dim[2])))


def test_context_of_three_kernels_hand_worked():
    """orc_context_n against numbers worked by hand through include/KernelFusion.h:45-80 and
    lib/KernelFuser/KernelPrinter.cpp:46-66 (32-thread granule, 64 K registers, 2048 threads, as the reference)."""
    # configs/im2col_maxpool_norm.yaml: 512x1, 256x1, 32x8 -- plain concatenation
    rows = [((512, 1, 1), 32, -1.0), ((256, 1, 1), 32, -1.0), ((32, 8, 1), 32, -1.0)]
    p = O.context_n(rows, imbalanced=False, launch_bound=True)
    assert list(p.lo)[:3] == [0, 512, 768] and list(p.hi)[:3] == [512, 768, 1024]
    assert p.launch_threads == 1024
    # min(65536/32/512 = 4, 65536/32/256 = 8, 8, 2048/1024 = 2) = 2
    assert p.launch_blocks == 2
    v = O.context_n(rows, base_line=True, imbalanced=False)
    assert list(v.lo)[:3] == [0, 0, 0] and list(v.hi)[:3] == [512, 256, 256] and v.launch_threads == 512 and v.launch_blocks == 0
    # ExecTimes 1 : 2 : 1 over 1024 threads: int(0.25 * 1024 / 32) * 32 = 256, int(0.5 * 32) * 32 = 512, rest 256
    timed = [((512, 1, 1), 32, 10.0), ((256, 1, 1), 32, 20.0), ((32, 8, 1), 32, 10.0)]
    q = O.context_n(timed, imbalanced=True)
    assert [q.hi[i] - q.lo[i] for i in range(3)] == [256, 512, 256]
    assert (q.block_dim[2].x, q.block_dim[2].y) == (32, 8) and q.block_dim[1].x == 512
    # the driver's split loop on three kernels (main.cpp:219-225): Split 128 of 768 for the first two, the third
    # keeps ExecTime -1: total time 767; int(128/767 * 32) = 5 -> 160, int(640/767 * 32) = 26 -> 832, rest 1024 - 992 = 32
    loop = [((512, 1, 1), 32, 128.0), ((256, 1, 1), 32, 640.0), ((32, 8, 1), 32, -1.0)]
    r = O.context_n(loop, imbalanced=True)
    assert [r.hi[i] - r.lo[i] for i in range(3)] == [160, 832, 32]
    # a pair through the n-kernel routine equals the two-kernel routine
    pair = [((512, 1, 1), 49, 31.0), ((256, 1, 1), 24, 95.0)]
    a, b = O.context_n(pair, launch_bound=True), O.context(pair, launch_bound=True)
    assert list(a.hi)[:2] == list(b.hi) and a.launch_blocks == b.launch_blocks and a.launch_threads == b.launch_threads
