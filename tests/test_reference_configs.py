"""Every configuration file the reference ships (`configs/*.yaml`) goes through the loader as it is.

The files are the reference's data, read in place when its tree is present (they are not copied
here); without the tree the test is skipped.  Pair files must plan under the name the reference's
printer gives the fused kernel (lib/KernelFuser/KernelPrinter.cpp:67-70); the three files that fuse
three kernels must load and be refused only when a plan is asked for."""
import glob
import os

import pytest

import hfuse_amd
from hfuse_amd import _lib as L
from hfuse_amd.launcher import Config

REF = "/root/reference/configs"
pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not on this machine")

LISTS = {"ml_fusion.yaml": ("ml_kernels.yaml", 10), "crypto_fusion.yaml": ("crypto_kernels.yaml", 6)}
TABLES = {t for t, _ in LISTS.values()}
MANY = {"crypt_four.yaml": 3, "im2col_maxpool_norm.yaml": 3, "maxpool_summary_norm.yaml": 3}


def test_fusion_lists_with_their_kernel_tables():
    for fusion, (table, n) in LISTS.items():
        cfg = Config.from_files(os.path.join(REF, fusion), os.path.join(REF, table))
        assert cfg.num_fusions == n
        for i, (file, k1, k2) in enumerate(cfg.fusions()):
            for preset in ("hfuse", "hfuse_lb", "vfuse", "vfuse_lb"):
                part = cfg.plan(i, preset, 0).partition
                assert part.name.decode() == f"{k1}_{k2}_fused_kernel_{preset}_idx_0"
            assert cfg.num_splits(i) >= 1


def test_per_pair_tables():
    seen = 0
    for path in sorted(glob.glob(os.path.join(REF, "*.yaml"))):
        name = os.path.basename(path)
        if name in LISTS or name in TABLES or name in MANY or name == "test.yaml":
            continue
        cfg = Config.from_files(None, path)            # the older form: a bare list of kernel rows, fused in order
        assert cfg.num_fusions == 1 and cfg.num_kernels == 2, name
        _, k1, k2 = cfg.fusion(0)
        part = cfg.plan(0, "hfuse", 0).partition
        assert part.name.decode() == f"{k1}_{k2}_fused_kernel_hfuse_idx_0"
        assert part.hi[0] - part.lo[0] == 128 and part.hi[1] == part.launch_threads   # split idx 0 = 128 threads
        seen += 1
    assert seen == 16


def test_lists_of_three_kernels_load_and_plan():
    """The reference's three-kernel lists: the Context's partition among three at the table's block shapes."""
    want = {"crypt_four.yaml": [128, 256, 384], "im2col_maxpool_norm.yaml": [512, 768, 1024]}
    for name, n in MANY.items():
        cfg = Config.from_files(None, os.path.join(REF, name))
        assert cfg.num_fusions == 1 and len(cfg.fusion_kernels(0)) == n
        if n != 3:
            continue
        v = cfg.plan(0, "vfuse").partition_n
        assert v.n == 3 and list(v.lo)[:3] == [0, 0, 0]
        if name in want:
            part = cfg.plan(0).partition_n
            assert list(part.hi)[:3] == want[name] and part.launch_threads == want[name][2]
            assert part.name.decode() == "_".join(cfg.fusion_kernels(0)) + "_fused_kernel_hfuse_table"
        else:   # maxpool_summary_norm.yaml: 256 + 512 + 512 threads do not fit one workgroup
            with pytest.raises(hfuse_amd.HfuseError) as e:
                cfg.plan(0)
            assert e.value.code == L.HF_EINVAL and "exceeds 1024" in e.value.message


def test_the_toy_file_names_kernels_this_library_does_not_have():
    cfg = Config.from_files(None, os.path.join(REF, "test.yaml"))
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(0)
    assert e.value.code == L.HF_ENOTFOUND
