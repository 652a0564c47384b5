"""Host logic of the library (no GPU): YAML schemas, plans, partition parity with
the oracle, and the error behaviour at the C-ABI."""
import ctypes as C
import re

import os

import pytest

import hfuse_amd
from hfuse_amd import _lib as L
from hfuse_amd.launcher import Config
from oracle import oracle as O

KERNELS_MAP = """
im2col_kernel:
  KernelName: im2col_kernel
  HasBarriers: false
  BlockDim:
    X: 512
    Y: 1
    Z: 1
  Reg: 49
  ExecTime: 31
MaxPoolForward:
  KernelName: MaxPoolForward   # trailing comment
  HasBarriers: false
  BlockDim:
    X: 256
    Y: 1
    Z: 1
  Reg: 24
  ExecTime: 95
batch_norm_collect_statistics_kernel:
  KernelName: batch_norm_collect_statistics_kernel
  HasBarriers: true
  BlockDim:
    X: 32
    Y: 16
    Z: 1
  Reg: 24
  ExecTime: 52
"""

FUSION = """
- File: Im2ColMaxPool.cu
  Kernels:
   - im2col_kernel
   - MaxPoolForward
- File: MaxPoolBatchNorm.cu
  Kernels:
  - MaxPoolForward
  - batch_norm_collect_statistics_kernel
"""

# the older per-pair form: a bare list of rows, Reg optional
LEGACY = """
- KernelName: im2col_kernel
  HasBarriers: false
  BlockDim:
    X: 512
    Y: 1
    Z: 1
- KernelName: MaxPoolForward
  HasBarriers: false
  BlockDim:
    X: 256
    Y: 1
    Z: 1
  Reg: 24
"""


def test_parse_map_form_and_fusion_list():
    cfg = Config(FUSION, KERNELS_MAP)
    assert cfg.num_kernels == 3 and cfg.num_fusions == 2
    assert cfg.fusion(0) == ("Im2ColMaxPool.cu", "im2col_kernel", "MaxPoolForward")
    assert cfg.fusion(1) == ("MaxPoolBatchNorm.cu", "MaxPoolForward", "batch_norm_collect_statistics_kernel")
    k = cfg.kernel("batch_norm_collect_statistics_kernel")
    assert (k.block_dim.x, k.block_dim.y, k.block_dim.z) == (32, 16, 1)
    assert k.reg == 24 and k.exec_time == 52.0 and k.has_barriers == 1
    assert cfg.kernel("MaxPoolForward").kernel_name == b"MaxPoolForward"


def test_parse_legacy_list_form():
    cfg = Config(None, LEGACY)
    assert cfg.num_fusions == 1
    assert cfg.fusion(0)[1:] == ("im2col_kernel", "MaxPoolForward")
    assert cfg.kernel("im2col_kernel").reg == 0 and cfg.kernel("im2col_kernel").exec_time == -1.0


def test_shipped_config_lists_the_five_benchmarked_pairs_first(cfg):
    pairs = [f[1:] for f in cfg.fusions()[:5]]
    assert pairs == [("im2col_kernel", "MaxPoolForward"),
                     ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame"),
                     ("kernelHistogram1D", "MaxPoolForward"),
                     ("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash"),
                     ("ethash_search", "sia_blake2b_gpu_hash")]


@pytest.mark.parametrize("bad,needle", [
    ("im2col_kernel:\n  HasBarriers: false\n  BlockDim: \n    X: 1\n    Y: 1\n    Z: 1\n  Reg: 1\n", "KernelName"),
    ("k:\n  KernelName: k\n  BlockDim:\n    X: 1\n    Y: 1\n    Z: 1\n  Reg: 1\n", "HasBarriers"),
    ("k:\n  KernelName: k\n  HasBarriers: false\n  Reg: 1\n", "BlockDim"),
    ("k:\n  KernelName: k\n  HasBarriers: false\n  BlockDim:\n    X: 1\n    Y: 1\n  Reg: 1\n", "BlockDim"),
    ("k:\n  KernelName: k\n  HasBarriers: false\n  BlockDim:\n    X: 1\n    Y: 1\n    Z: 1\n", "Reg"),
    ("k:\n  KernelName: k\n  HasBarriers: maybe\n  BlockDim:\n    X: 1\n    Y: 1\n    Z: 1\n  Reg: 1\n", "HasBarriers"),
    ("k:\n  KernelName: k\n  HasBarriers: false\n  BlockDim:\n    X: -4\n    Y: 1\n    Z: 1\n  Reg: 1\n", "BlockDim"),
    ("k:\n  KernelName: k\n  HasBarriers: false\n  BlockDim:\n    X: 1\n    Y: 1\n    Z: 1\n  Reg: 1\n  Bogus: 2\n", "Bogus"),
    ("just a scalar", "expected"),
    ("k:\n\tKernelName: k\n", "tab"),
    ("", "expected"),
])
def test_kernel_table_schema_errors(bad, needle):
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config("- File: f\n  Kernels:\n    - k\n    - k\n", bad)
    assert e.value.code == L.HF_EPARSE and needle in e.value.message


def test_fusion_list_errors():
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config("- File: f\n  Kernels:\n    - im2col_kernel\n    - nope\n", KERNELS_MAP)
    assert e.value.code == L.HF_EPARSE and "nope" in e.value.message
    # the schema allows any number of kernels per entry (the reference's crypt_four.yaml names three):
    # such a list loads; plans exist for entries of two and of three kernels
    cfg = Config("- File: one\n  Kernels:\n    - im2col_kernel\n"
                 "- File: three\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n    - im2col_kernel\n"
                 "- File: two\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n", KERNELS_MAP)
    assert cfg.num_fusions == 3
    assert cfg.fusion(0) == ("one", "im2col_kernel", "")
    assert cfg.fusion_kernels(1) == ["im2col_kernel", "MaxPoolForward", "im2col_kernel"]
    assert cfg.find_fusion("im2col_kernel", "MaxPoolForward") == 2      # the triple is not mistaken for the pair
    assert cfg.find_fusion_n("im2col_kernel", "MaxPoolForward", "im2col_kernel") == 1
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(0)
    assert e.value.code == L.HF_EUNSUPPORTED and "two or three" in e.value.message
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.num_splits(0)
    assert e.value.code == L.HF_EUNSUPPORTED
    with pytest.raises(hfuse_amd.HfuseError) as e:                      # three kernels that are none of the built lists:
        cfg.plan(1)                                                     # said when the plan is made, not at the launch
    assert e.value.code == L.HF_EUNSUPPORTED and "in any order" in e.value.message
    too_wide = Config("- File: three\n  Kernels: [im2col_kernel, MaxPoolForward, batch_norm_collect_statistics_kernel]\n",
                      KERNELS_MAP)
    with pytest.raises(hfuse_amd.HfuseError) as e:                      # 512 + 256 + 512 threads
        too_wide.plan(0)
    assert e.value.code == L.HF_EINVAL and "exceeds 1024" in e.value.message
    assert cfg.num_splits(1) == 5                                        # the loop varies the first two: 128 .. 640 < 768
    cfg.plan(2)
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config("- File: f\n  Kernels: []\n", KERNELS_MAP)
    assert e.value.code == L.HF_EPARSE
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config("- Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n", KERNELS_MAP)
    assert "File" in e.value.message
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config.from_files("/nonexistent/fusion.yaml", "/nonexistent/kernels.yaml")
    assert e.value.code == L.HF_EIO and "failed to read configs" in e.value.message


def _rows(cfg, i):
    _, k1, k2 = cfg.fusion(i)
    out = []
    for k in (k1, k2):
        r = cfg.kernel(k)
        out.append(((r.block_dim.x, r.block_dim.y, r.block_dim.z), r.reg, r.exec_time))
    return out


def test_partition_matches_oracle_for_every_shipped_pair_and_split(cfg):
    """Product partition == oracle Context with the wavefront granule and gfx950 register file."""
    checked = 0
    for i in range(cfg.num_fusions):
        rows = _rows(cfg, i)
        total = sum(r[0][0] * r[0][1] * r[0][2] for r in rows)
        assert cfg.num_splits(i) == len(O.enumerate_splits(rows, granule=64))
        for idx in range(cfg.num_splits(i)):
            split = 128 * (idx + 1)
            ex = [(rows[0][0], rows[0][1], float(split)), (rows[1][0], rows[1][1], float(total - split))]
            for preset, lb in (("hfuse", False), ("hfuse_lb", True)):
                want = O.context(ex, launch_bound=lb, imbalanced=True, granule=64, reg_file=4 * 512 * 64,
                                 max_threads=2048)
                try:
                    plan = cfg.plan(i, preset, idx)
                except hfuse_amd.HfuseError as e:
                    # legal in the reference's arithmetic, refused here: part not a multiple of 64 / Y
                    assert e.code == L.HF_EINVAL
                    continue
                got = plan.partition
                assert list(got.lo) == list(want.lo) and list(got.hi) == list(want.hi)
                for h in range(2):
                    assert (got.block_dim[h].x, got.block_dim[h].y) == (want.block_dim[h].x, want.block_dim[h].y)
                assert got.launch_threads == want.launch_threads and got.launch_blocks == want.launch_blocks
                assert got.name.decode().endswith(f"_fused_kernel_{preset}_idx_{idx}")
                checked += 1
    assert checked > 40


def test_fused_name_and_presets():
    cfg = Config(FUSION, KERNELS_MAP)
    p = cfg.plan(0, "hfuse", 1)
    assert p.name == "im2col_kernel_MaxPoolForward_fused_kernel_hfuse_idx_1"
    assert list(p.partition.hi) == [256, 768]
    v = cfg.plan(0, "vfuse_lb", 0).partition
    assert v.name == b"im2col_kernel_MaxPoolForward_fused_kernel_vfuse_lb_idx_0"
    assert (list(v.lo), list(v.hi), v.launch_threads) == ([0, 0], [512, 256], 512)
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(0, "hfuse_bar_sync", 0)
    assert e.value.code == L.HF_ENOTFOUND
    # ExecTime-proportional split (KernelFusion.h:63-72) at the wavefront granule:
    # int(31/126 * 768 / 64) * 64 = 128
    assert list(cfg.plan(0, "hfuse", L.HF_SPLIT_EXECTIME).partition.hi) == [128, 768]


def test_split_rules():
    cfg = Config(FUSION, KERNELS_MAP)
    with pytest.raises(hfuse_amd.HfuseError):
        cfg.plan(0, "hfuse", 5)  # 768 threads: indices 0..4 only
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(0, "hfuse", L.HF_SPLIT_TABLE, 100)
    assert "multiple" in e.value.message
    with pytest.raises(hfuse_amd.HfuseError):
        cfg.plan(0, "hfuse", L.HF_SPLIT_TABLE, 768)  # nothing left for kernel 2
    p = cfg.plan(1, "hfuse", L.HF_SPLIT_TABLE, 256).partition  # bn keeps Y = 16 -> X = 32
    assert (p.block_dim[1].x, p.block_dim[1].y, p.hi[1]) == (32, 16, 768)
    p = cfg.plan(1, "hfuse", L.HF_SPLIT_TABLE, 448).partition  # 320 threads left = 20 x 16, five waves
    assert (p.block_dim[1].x, p.block_dim[1].y) == (20, 16)
    big = KERNELS_MAP.replace("X: 512", "X: 1024")
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config(FUSION, big).plan(0, "hfuse")
    assert "1024" in e.value.message


def test_tuned_split_and_block_keys_of_the_fusion_list():
    """`Split` / `Threads` (beyond the reference's schema) give a pair its default fused block."""
    fusion = ("- File: a\n  Split: 128\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n"
              "- File: b\n  Split: 256\n  Threads: 512\n  Kernels:\n    - MaxPoolForward\n"
              "    - batch_norm_collect_statistics_kernel\n")
    cfg = Config(fusion, KERNELS_MAP)
    a = cfg.plan(0).partition
    assert (list(a.lo), list(a.hi)) == ([0, 128], [128, 768])        # re-split of the table's 512 + 256
    b = cfg.plan(1).partition
    assert (list(b.lo), list(b.hi), b.launch_threads) == ([0, 256], [256, 512], 512)
    assert (b.block_dim[1].x, b.block_dim[1].y) == (16, 16)           # bn keeps Y, X = threads / Y
    assert b.name == b"MaxPoolForward_batch_norm_collect_statistics_kernel_fused_kernel_hfuse_block_256_256"
    # an explicit split index still follows the reference's enumeration over the table's block
    assert list(cfg.plan(1, "hfuse", 0).partition.hi) == [128, 768]
    for bad in ("  Split: 100\n", "  Split: 0\n", "  Split: 128\n  Threads: 128\n", "  Threads: 512\n",
                "  Split: 128\n  Threads: 2048\n", "  Bogus: 1\n"):
        with pytest.raises(hfuse_amd.HfuseError) as e:
            Config("- File: a\n" + bad + "  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n", KERNELS_MAP)
        assert e.value.code == L.HF_EPARSE


def test_set_block_rules():
    cfg = Config(FUSION, KERNELS_MAP)
    plan = cfg.plan(1)  # MaxPool (256) + bn (32,16)
    plan.set_block(128, 256)
    p = plan.partition
    assert (list(p.hi), p.block_dim[1].x, p.block_dim[1].y, p.launch_threads) == ([128, 384], 16, 16, 384)
    for bad in ((100, 256), (0, 256), (128, 0), (512, 768), (128, 64 * 3 + 8)):
        with pytest.raises(hfuse_amd.HfuseError):
            plan.set_block(*bad)
    # under a vertical preset both bodies start at thread 0 (KernelFusion.h:76-78): the two counts are the threads
    # that run each body, the block is the larger of them
    v = cfg.plan(1, "vfuse")
    v.set_block(128, 512)
    q = v.partition
    assert (list(q.lo), list(q.hi), q.launch_threads) == ([0, 0], [128, 512], 512)
    assert q.name.decode().endswith("_fused_kernel_vfuse_block_128_512")
    for bad in ((100, 256), (128, 1088)):
        with pytest.raises(hfuse_amd.HfuseError):
            v.set_block(*bad)
    plan.set_grids(3, 5)
    plan.set_lending(False)
    with pytest.raises(hfuse_amd.HfuseError):
        plan.set_grids(-1, 0)


def test_local_index_follows_the_remap(cfg):
    plan = cfg.plan(cfg.find_fusion("upsample_nearest2d_out_frame", "batch_norm_collect_statistics_kernel"))
    part = plan.partition
    dim = (part.block_dim[1].x, part.block_dim[1].y, part.block_dim[1].z)
    for tid in (part.lo[1], part.lo[1] + 65, part.hi[1] - 1):
        assert plan.local_index(1, tid) == O.remap_tid(tid, part.lo[1], dim)
    with pytest.raises(hfuse_amd.HfuseError):
        plan.local_index(1, part.lo[1] - 1)


def test_barrier_policy(cfg):
    assert cfg.plan(0).partition.barrier_mode == L.HF_BARRIER_NONE
    # the policy of the library, whatever mode the shipped list tunes this pair to: an explicit split takes no tuned keys
    bn_up = cfg.plan(1, "hfuse", 0)
    assert bn_up.partition.barrier_mode == L.HF_BARRIER_SUBSET
    with pytest.raises(hfuse_amd.HfuseError):
        bn_up.set_barrier_mode(L.HF_BARRIER_MATCHED)  # upsample never synchronises
    with pytest.raises(hfuse_amd.HfuseError):
        bn_up.set_barrier_mode(L.HF_BARRIER_NONE)
    bn_up.set_barrier_mode(L.HF_BARRIER_BLOCKIDX)
    both = cfg.plan(cfg.find_fusion("kernelHistogram1D", "batch_norm_collect_statistics_kernel"))
    both.set_barrier_mode(L.HF_BARRIER_MATCHED)
    assert both.partition.barrier_mode == L.HF_BARRIER_MATCHED


def test_unknown_kernels_and_mixed_pairs():
    table = KERNELS_MAP + """
foo:
  KernelName: foo
  HasBarriers: false
  BlockDim:
    X: 256
    Y: 1
    Z: 1
  Reg: 8
sia_blake2b_gpu_hash:
  KernelName: sia_blake2b_gpu_hash
  HasBarriers: false
  BlockDim:
    X: 128
    Y: 1
    Z: 1
  Reg: 64
"""
    fusion = ("- File: a\n  Kernels:\n    - foo\n    - MaxPoolForward\n"
              "- File: b\n  Kernels:\n    - MaxPoolForward\n    - sia_blake2b_gpu_hash\n")
    cfg = Config(fusion, table)
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(0)
    assert e.value.code == L.HF_ENOTFOUND and "foo" in e.value.message
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(1)
    assert e.value.code == L.HF_EUNSUPPORTED


# The reference's own two ML configuration files, restated in its schema (same kernel names,
# block shapes, Reg and ExecTime as configs/ml_kernels.yaml; same ten pairs as configs/ml_fusion.yaml).
REFERENCE_ML_KERNELS = """
upsample_bilinear2d_out_frame:
  KernelName: upsample_bilinear2d_out_frame
  HasBarriers: false
  BlockDim:
    X: 512
    Y: 1
    Z: 1
  Reg: 43
  ExecTime: 77
kernelHistogram1D:
  KernelName: kernelHistogram1D
  HasBarriers: false
  BlockDim:
    X: 512
    Y: 1
    Z: 1
  Reg: 32
  ExecTime: 1
batch_norm_collect_statistics_kernel:
  KernelName: batch_norm_collect_statistics_kernel
  HasBarriers: false
  BlockDim:
    X: 32
    Y: 16
    Z: 1
  Reg: 24
  ExecTime: 52
im2col_kernel:
  KernelName: im2col_kernel
  HasBarriers: false
  BlockDim:
    X: 512
    Y: 1
    Z: 1
  Reg: 49
  ExecTime: 31
MaxPoolForward:
  KernelName: MaxPoolForward
  HasBarriers: false
  BlockDim:
    X: 256
    Y: 1
    Z: 1
  Reg: 24
  ExecTime: 95
"""
REFERENCE_ML_PAIRS = [
    ("im2col_kernel", "MaxPoolForward"), ("im2col_kernel", "batch_norm_collect_statistics_kernel"),
    ("im2col_kernel", "kernelHistogram1D"), ("im2col_kernel", "upsample_bilinear2d_out_frame"),
    ("MaxPoolForward", "batch_norm_collect_statistics_kernel"), ("MaxPoolForward", "upsample_bilinear2d_out_frame"),
    ("kernelHistogram1D", "MaxPoolForward"), ("kernelHistogram1D", "upsample_bilinear2d_out_frame"),
    ("upsample_bilinear2d_out_frame", "batch_norm_collect_statistics_kernel"),
    ("kernelHistogram1D", "batch_norm_collect_statistics_kernel"),
]
REFERENCE_ML_FUSION = "".join(f"- File: f{i}.cu\n  Kernels:\n   - {a}\n   - {b}\n" for i, (a, b) in enumerate(REFERENCE_ML_PAIRS))


def test_reference_ml_configuration_plans_every_pair():
    """All ten pairs of the reference's ML lists get a plan (bilinear upsampling included)."""
    cfg = Config(REFERENCE_ML_FUSION, REFERENCE_ML_KERNELS)
    assert cfg.num_fusions == 10
    for i, (a, b) in enumerate(REFERENCE_ML_PAIRS):
        part = cfg.plan(i).partition
        assert part.name.decode() == f"{a}_{b}_fused_kernel_hfuse_table"
        assert part.launch_threads in (768, 1024)
        for idx in range(cfg.num_splits(i)):
            assert cfg.plan(i, "hfuse_lb", idx).partition.hi[0] == 128 * (idx + 1)


def test_launch_argument_errors_never_reach_the_gpu(cfg):
    """Null pointers and inconsistent shapes are refused on the host."""
    lib = L.lib()
    plan = cfg.plan(0)
    a, b = L.Im2colArgs(), L.MaxPoolArgs()
    assert lib.hf_launch_fused(plan._h, C.byref(a), C.byref(b), 0, None) == L.HF_EINVAL
    assert b"null data pointer" in lib.hf_last_error()
    assert lib.hf_launch_fused(plan._h, None, C.byref(b), 0, None) == L.HF_EINVAL
    assert lib.hf_launch_native(b"no_such_kernel", C.byref(a), 0, 0, None) == L.HF_ENOTFOUND
    assert lib.hf_launch_native(None, C.byref(a), 0, 0, None) == L.HF_EINVAL
    a.data_im = a.data_col = 256
    a.n, a.height, a.width, a.kernel_h, a.kernel_w = 64, 8, 8, 3, 3
    a.stride_h = a.stride_w = a.dilation_h = a.dilation_w = 1
    a.pad_h = a.pad_w = 1
    a.height_col, a.width_col = 8, 7  # does not follow from the geometry
    assert lib.hf_launch_native(b"im2col_kernel", C.byref(a), 0, 0, None) == L.HF_EINVAL
    assert b"height_col" in lib.hf_last_error()
    e = L.EthashArgs()
    e.g_output = 256
    assert lib.hf_launch_native(b"ethash_search", C.byref(e), 0, 0, None) == L.HF_EINVAL
    assert b"hf_ethash_set_constants" in lib.hf_last_error()
    h = L.HistcArgs()
    h.a.data = h.b.data = 256
    h.a.dims = h.b.dims = 1
    h.nbins, h.minvalue, h.maxvalue = 8, 1.0, 0.0
    assert lib.hf_launch_native(b"kernelHistogram1D", C.byref(h), 0, 0, None) == L.HF_EINVAL
    assert b"max must be larger than min" in lib.hf_last_error()
    v = cfg.plan(0, "vfuse")
    assert lib.hf_launch_fused(v._h, C.byref(a), C.byref(b), 0, None) in (L.HF_EINVAL, L.HF_EUNSUPPORTED)
    # extents whose product wraps to zero used to divide by zero; every extent is bounded now
    a.height_col = a.width_col = 1 << 32
    assert lib.hf_launch_native(b"im2col_kernel", C.byref(a), 0, 0, None) == L.HF_EINVAL
    assert b"oversized geometry" in lib.hf_last_error()
    # a grid whose thread count does not fit the bodies' 32-bit work-item counters
    a.height_col, a.width_col = 8, 8
    assert lib.hf_launch_native(b"im2col_kernel", C.byref(a), 1 << 23, 1024, None) == L.HF_EINVAL
    assert b"32 bits" in lib.hf_last_error()
    b.bottom_data = b.top_data = b.top_mask = 256
    b.nthreads, b.num, b.channels, b.height, b.width, b.pooled_height, b.pooled_width = 16, 1, 1, 8, 8, 4, 4
    b.kernel_h = b.kernel_w = b.stride_h = b.stride_w = 2
    b.dilation_h = b.dilation_w = 1
    assert lib.hf_launch_fused(plan._h, C.byref(a), C.byref(b), 1 << 23, None) == L.HF_EINVAL
    assert b"32 bits" in lib.hf_last_error()


def test_counter_wrap_is_refused_on_the_host(cfg):
    """A caller grid large enough that a 32-bit work-item counter would wrap (and never end its loop)
    is refused; the searches count in 64 bits, so a full-range scan (threads = 2^32 - 1) passes the
    validators and only fails for want of a device."""
    lib = L.lib()
    up = L.UpsampleNearestArgs()
    up.idata = up.odata = 256
    up.nc, up.height1, up.width1, up.height2, up.width2 = 1 << 11, 512, 512, 1024, 1024  # 2^28 work items in the exact-2x path
    up.height_scale = up.width_scale = 0.5
    # two items per trip: 2^28 + 2 * grid * block must stay within 2^32
    assert lib.hf_launch_native(b"upsample_nearest2d_out_frame", C.byref(up), 1 << 22, 512, None) == L.HF_EINVAL
    assert b"32 bits" in lib.hf_last_error()
    ok = lib.hf_launch_native(b"upsample_nearest2d_out_frame", C.byref(up), 1 << 20, 512, None)
    assert ok in (L.HF_OK, L.HF_EHIP), lib.hf_last_error()
    hdr = bytes(range(80))
    assert lib.hf_sha256d_set_block(hdr, 1, None) == 0 and lib.hf_sia_blake2b_set_block(hdr, None) == 0
    sh = L.Sha256dArgs()
    sh.threads, sh.start_nonce, sh.res_nonces = 0xFFFFFFFF, 0, 256
    b2 = L.Blake2bArgs()
    b2.threads, b2.start_nonce, b2.res_nonce = 0xFFFFFFFF, 0, 256
    import torch
    if not torch.cuda.is_available():   # with a device these would launch on made-up pointers
        assert lib.hf_launch_native(b"sha256d_gpu_hash_shared", C.byref(sh), 0, 0, None) in (L.HF_OK, L.HF_EHIP)
        assert lib.hf_launch_native(b"sia_blake2b_gpu_hash", C.byref(b2), 0, 0, None) in (L.HF_OK, L.HF_EHIP)


def test_vertical_presets_need_whole_wavefronts():
    """A BlockDim that is not a multiple of 64 threads is refused under vfuse / vfuse_lb as under hfuse:
    the vertical kernel runs whole wavefronts of each body and would leave the ragged lanes' items undone."""
    table = KERNELS_MAP.replace("X: 512", "X: 96", 1)
    c = Config(FUSION, table)
    for preset in ("vfuse", "vfuse_lb", "hfuse"):
        with pytest.raises(hfuse_amd.HfuseError) as e:
            c.plan(0, preset)
        assert e.value.code == L.HF_EINVAL and "wavefront" in e.value.message, preset


def test_bilinear_scales_are_validated():
    """Scales that would send the unclamped source index outside the input (too large, inf, NaN) are refused."""
    lib = L.lib()
    def args(rh, rw, align=0):
        bl = L.UpsampleBilinearArgs()
        bl.n, bl.rheight, bl.rwidth, bl.align_corners = 256, rh, rw, align
        bl.idata.data = bl.odata.data = 256
        bl.idata.sizes[:] = [2, 3, 8, 8]; bl.idata.strides[:] = [192, 64, 8, 1]
        bl.odata.sizes[:] = [2, 3, 16, 16]; bl.odata.strides[:] = [768, 256, 16, 1]
        return bl
    for rh, rw, align in ((float("inf"), 0.5, 0), (0.5, float("inf"), 0), (float("nan"), 0.5, 0), (0.6, 0.5, 0),
                          (0.5, 0.6, 0), (0.5, 8.0 / 15.0 + 1e-3, 1), (1e30, 0.5, 1), (-0.5, 0.5, 0)):
        a = args(rh, rw, align)
        assert lib.hf_launch_native(b"upsample_bilinear2d_out_frame", C.byref(a), 0, 0, None) == L.HF_EINVAL, (rh, rw, align)
    import torch
    if not torch.cuda.is_available():
        for rh, rw, align in ((0.5, 0.5, 0), (7.0 / 15.0, 7.0 / 15.0, 1), (0.25, 0.5, 0), (0.0, 0.0, 1)):
            a = args(rh, rw, align)
            assert lib.hf_launch_native(b"upsample_bilinear2d_out_frame", C.byref(a), 0, 0, None) in (L.HF_OK, L.HF_EHIP), \
                (rh, rw, align, lib.hf_last_error())


def test_constants_objects_are_independent_of_the_process_wide_set(cfg):
    """hf_constants: a caller-owned set; a plan bound to it, or hf_launch_native_with, does not look at the
    process-wide set at all (here the process-wide Ethash constants are unset in a fresh library state
    only if no other test set them, so the check goes through an unset *caller-owned* set instead)."""
    lib = L.lib()
    from hfuse_amd import launcher as H
    empty, full = H.Constants(), H.Constants()
    hdr = bytes(range(80))
    full.set_sha256d(hdr, 1).set_sia_blake2b(hdr)
    sh = L.Sha256dArgs()
    sh.threads, sh.start_nonce, sh.res_nonces = 0, 0, 256     # zero nonces: validated, nothing launched
    assert lib.hf_sha256d_set_block(hdr, 1, None) == 0         # process-wide set has it ...
    assert lib.hf_launch_native_with(b"sha256d_gpu_hash_shared", C.byref(sh), empty._h, 0, 0, None) == L.HF_EINVAL
    assert b"hf_sha256d_set_block" in lib.hf_last_error()      # ... the empty caller-owned set does not
    assert lib.hf_launch_native_with(b"sha256d_gpu_hash_shared", C.byref(sh), full._h, 0, 0, None) == L.HF_OK
    assert lib.hf_launch_native_with(b"sha256d_gpu_hash_shared", C.byref(sh), None, 0, 0, None) == L.HF_EINVAL
    i = cfg.find_fusion("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash")
    plan = cfg.plan(i)
    b2 = L.Blake2bArgs()
    b2.threads, b2.start_nonce, b2.res_nonce = 0, 0, 256
    plan.bind_constants(empty)
    assert lib.hf_launch_fused(plan._h, C.byref(sh), C.byref(b2), 0, None) == L.HF_EINVAL
    plan.bind_constants(None)                                  # back to the process-wide set
    assert lib.hf_sia_blake2b_set_block(hdr, None) == 0
    import torch
    if not torch.cuda.is_available():
        assert lib.hf_launch_fused(plan._h, C.byref(sh), C.byref(b2), 0, None) in (L.HF_OK, L.HF_EHIP)
    with pytest.raises(hfuse_amd.HfuseError):
        H.Constants().set_ethash(type("T", (), {"data_ptr": lambda self: 8})(), 4, bytes(32), 1)  # misaligned DAG


def test_launch_bound_formula_and_built_variants():
    """The register-cap axis: the occupancy formula of the reference's printer (KernelPrinter.cpp:44-66) with
    this part's constants (128 K registers, 2048 threads a CU), hand-worked for the five benchmarked pairs at fixed
    block shapes, and the build each request resolves to.  B blocks of T threads are B * T / 64 waves on four SIMDs:
    the bound is rounded up, so that all of them fit.
      im2col(Reg 42, 256 thr) + max-pool(32, 448): min(131072/42/256 = 12, 131072/32/448 = 9, 2048/704 = 2) = 2 blocks
        of 704 threads = 22 waves = 5.5 -> 6 waves per SIMD;
      bn(23, 128) + upsample(22, 128): min(44, 46, 8) = 8 blocks of 256 = 32 waves -> 8;
      histogram(19, 768) + max-pool(32, 128): min(8, 32, 2) = 2 of 896 = 28 waves -> 7;
      SHA-256d(70, 128) + Blake2b(76, 128): min(14, 13, 8) = 8 of 256 -> 8;
      Ethash(116, 128) + Blake2b(76, 64): min(8, 26, 10) = 8 of 192 = 24 waves -> 6;
      max-pool(32, 64) + bn(23, 128): min(64, 44, 10) = 10 of 192 = 30 waves = 7.5 -> 8."""
    kernels = open(os.path.join(hfuse_amd.CONFIG_DIR, "gfx950_kernels.yaml")).read()
    shapes = [("im2col_kernel", "MaxPoolForward", 256, 448, 6),
              ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame", 128, 128, 8),
              ("kernelHistogram1D", "MaxPoolForward", 768, 128, 7),
              ("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash", 128, 128, 8),
              ("ethash_search", "sia_blake2b_gpu_hash", 128, 64, 6),
              ("MaxPoolForward", "batch_norm_collect_statistics_kernel", 64, 128, 8)]
    text = "".join(f"- File: f{n}\n  Kernels: [{a}, {b}]\n  Split: {t1}\n  Threads: {t1 + t2}\n" for n, (a, b, t1, t2, _) in enumerate(shapes))
    cfg = Config(text, kernels)
    for i, (_, _, t1, t2, w) in enumerate(shapes):
        plain, lb = cfg.plan(i), cfg.plan(i, "hfuse_lb")
        assert plain.launch_waves == (w, 0), (i, plain.launch_waves)      # the plain preset runs the plain build
        assert lb.launch_waves == (w, w), (i, lb.launch_waves)            # the _lb preset the build bounded at the formula's value
        blocks, threads = lb.partition.launch_blocks, lb.partition.launch_threads
        assert threads == t1 + t2 and -(-blocks * (threads // 64) // 4) == w
        plain.set_launch_bound(True)
        assert plain.launch_waves == (w, w)
        plain.set_launch_waves(8)
        assert plain.launch_waves == (w, 8)
        with pytest.raises(hfuse_amd.HfuseError):
            plain.set_launch_waves(9)
        if i < 5:
            # the five benchmarked pairs are built at 5, 6, 7 and 8 waves per SIMD: any request gets the smallest
            # build that is not below it (up to four the plain build's launch bound already holds)
            for ask, got in ((7, 7), (6, 6), (5, 5), (3, 5), (1, 5)):
                plain.set_launch_waves(ask)
                assert plain.launch_waves == (w, got), (i, ask, plain.launch_waves)
            # ... so another block shape of the pair runs the build at its own formula value
            other = cfg.plan(i, "hfuse_lb")
            other.set_block(64, 64)
            f, b = other.launch_waves
            assert f == b and 5 <= f <= 8
        else:
            plain.set_launch_waves(3)                                     # every other pair: the 8-wave build
            assert plain.launch_waves == (w, 8)
        plain.set_launch_waves(0)
        plain.set_launch_bound(False)
        assert plain.launch_waves == (w, 0)
        plain.set_barrier_mode(L.HF_BARRIER_BLOCKIDX)
        plain.set_launch_bound(True)
        assert plain.launch_waves[1] == 0                                 # the block-index partition has no bounded build
    # three more pairs of the shipped list have a second build, at the formula's value of these block shapes --
    # im2col(42, 256) + upsample(22, 512): min(12, 11, 2) = 2 blocks of 768 threads = 6 waves per SIMD;
    # im2col(42, 256) + histogram(19, 640): min(12, 10, 2) = 2 of 896 = 7; im2col + bilinear upsampling (32, 512): 6
    shipped = hfuse_amd.default_config()
    for k1, k2, block, w in (("im2col_kernel", "upsample_nearest2d_out_frame", (256, 512), 6),
                             ("im2col_kernel", "kernelHistogram1D", (256, 640), 7),
                             ("im2col_kernel", "upsample_bilinear2d_out_frame", (256, 512), 6)):
        p = shipped.plan(shipped.find_fusion(k1, k2), "hfuse_lb")
        p.set_block(*block)              # whatever shape the list is tuned to today
        assert p.launch_waves == (w, w), (k1, k2, p.launch_waves)
        p.set_launch_waves(8)
        assert p.launch_waves == (w, 8)


TRIPLE_TABLE = """
a:
  KernelName: im2col_kernel
  HasBarriers: false
  BlockDim: {bd0}
  Reg: 42
  ExecTime: {e0}
b:
  KernelName: MaxPoolForward
  HasBarriers: false
  BlockDim: {bd1}
  Reg: 32
  ExecTime: {e1}
c:
  KernelName: batch_norm_collect_statistics_kernel
  HasBarriers: true
  BlockDim: {bd2}
  Reg: 23
{e2}"""


def _triple_cfg(dims, times):
    def bd(d):
        return "\n    X: %d\n    Y: %d\n    Z: 1" % d
    e2 = "  ExecTime: %s\n" % times[2] if times[2] is not None else ""
    return Config("- File: t\n  Kernels:\n    - a\n    - b\n    - c\n",
                  TRIPLE_TABLE.format(bd0=bd(dims[0]), bd1=bd(dims[1]), bd2=bd(dims[2]), e0=times[0], e1=times[1], e2=e2))


def test_three_kernel_partition_matches_oracle():
    """Plans of three-kernel entries against the oracle's Context of three (64-lane granule, this part's
    register file): table split, every index of the driver's split loop, the ExecTime split, the vertical
    presets, the launch-bound hint, the local index remap; refusals are parts that are empty, ragged or do
    not divide by BlockDim.Y, and blocks beyond 1024 threads."""
    import random
    rng = random.Random(31337)
    regs = (42, 32, 23)
    checked = refused = 0
    for case in range(120):
        dims = []
        for y in (1, 1, rng.choice([1, 4, 8])):
            t = rng.choice([64, 128, 192, 256, 320, 512])
            dims.append((t // y, y))
        times = [rng.choice([5.0, 17.0, 31.0, 95.0]) for _ in range(3)]
        no_e2 = rng.random() < 0.3
        cfg = _triple_cfg(dims, times[:2] + [None if no_e2 else times[2]])
        total = sum(x * y for x, y in dims)
        d01 = dims[0][0] * dims[0][1] + dims[1][0] * dims[1][1]

        def rows(e):
            return [((dims[i][0], dims[i][1], 1), regs[i], e[i]) for i in range(3)]
        variants = [(L.HF_SPLIT_TABLE, rows(times), False)]
        for idx in range(cfg.num_splits(0)):
            variants.append((idx, rows([128.0 * (idx + 1), d01 - 128.0 * (idx + 1), -1.0 if no_e2 else times[2]]), True))
        assert cfg.num_splits(0) == len(range(128, d01, 128))
        if not no_e2:
            variants.append((L.HF_SPLIT_EXECTIME, rows(times), True))
        for idx, ex, imb in variants:
            for preset, lb in (("hfuse", False), ("hfuse_lb", True)):
                try:
                    want = O.context_n(ex, launch_bound=lb, imbalanced=imb, granule=64, reg_file=4 * 512 * 64, max_threads=2048)
                except ValueError:
                    want = None
                try:
                    plan = cfg.plan(0, preset, idx)
                except hfuse_amd.HfuseError as e:
                    assert e.code == L.HF_EINVAL
                    refused += 1
                    if want is not None:
                        parts = [want.hi[h] - want.lo[h] for h in range(3)]
                        assert sum(parts) > 1024 or any(p == 0 or p > 1 << 20 or p % 64 or p % dims[h][1] for h, p in enumerate(parts)), (dims, idx, parts)
                    continue
                got = plan.partition_n
                assert want is not None and got.n == 3 and plan.num_kernels == 3
                assert list(got.lo)[:3] == list(want.lo)[:3] and list(got.hi)[:3] == list(want.hi)[:3], (dims, idx)
                for h in range(3):
                    assert (got.block_dim[h].x, got.block_dim[h].y) == (want.block_dim[h].x, want.block_dim[h].y)
                    tid = rng.randrange(got.lo[h], got.hi[h])
                    assert plan.local_index(h, tid) == O.remap_tid(tid, got.lo[h], (got.block_dim[h].x, got.block_dim[h].y, 1))
                assert got.launch_threads == want.launch_threads and got.launch_blocks == want.launch_blocks
                checked += 1
        for preset, lb in (("vfuse", False), ("vfuse_lb", True)):
            want = O.context_n(rows(times), base_line=True, launch_bound=lb, imbalanced=False, granule=64,
                               reg_file=4 * 512 * 64, max_threads=2048)
            got = cfg.plan(0, preset, 0).partition_n
            assert list(got.lo)[:3] == [0, 0, 0] and list(got.hi)[:3] == list(want.hi)[:3]
            assert got.launch_threads == want.launch_threads and got.launch_blocks == want.launch_blocks
            checked += 1
    assert checked > 300 and refused > 20


def test_three_kernel_plans_refuse_the_calls_that_shape_a_pair():
    cfg = _triple_cfg([(256, 1), (256, 1), (32, 8)], [1.0, 1.0, 1.0])
    plan = cfg.plan(0)
    lib = L.lib()
    assert plan.partition_n.name.decode() == "im2col_kernel_MaxPoolForward_batch_norm_collect_statistics_kernel_fused_kernel_hfuse_table"
    for call in (lambda: plan.set_block(128, 128), lambda: plan.set_grids(1, 1), lambda: plan.set_lending(True),
                 lambda: plan.set_barrier_mode(L.HF_BARRIER_BLOCKIDX), lambda: plan.set_launch_bound(True),
                 lambda: plan.set_launch_waves(8), lambda: plan.partition, lambda: plan.local_index(3, 0)):
        with pytest.raises(hfuse_amd.HfuseError) as e:
            call()
        assert e.value.code == L.HF_EINVAL
    a = L.Im2colArgs()
    assert lib.hf_launch_fused(plan._h, C.byref(a), C.byref(a), 0, None) == L.HF_EINVAL
    ptrs = (C.c_void_p * 3)(C.addressof(a), C.addressof(a), C.addressof(a))
    assert lib.hf_launch_fused_n(plan._h, ptrs, 2, 0, None) == L.HF_EINVAL         # three lists for three kernels
    assert lib.hf_launch_fused_n(plan._h, ptrs, 3, 0, None) == L.HF_EINVAL         # null data pointers: refused on the host
    assert b"null data pointer" in lib.hf_last_error()
    with pytest.raises(hfuse_amd.HfuseError):
        cfg.plan(0, "hfuse", L.HF_SPLIT_TABLE, 128)                                 # split_threads shapes a pair
    plan.set_block_n(128, 512, 256)
    q = plan.partition_n
    assert list(q.hi)[:3] == [128, 640, 896] and q.name.decode().endswith("_hfuse_block_128_512_256")
    assert (q.block_dim[2].x, q.block_dim[2].y) == (32, 8)
    for bad in ((128, 512), (128, 512, 100), (512, 512, 512), (64, 64, 68), (0, 64, 64)):
        with pytest.raises(hfuse_amd.HfuseError):
            plan.set_block_n(*bad)
    # the keys that tune a pair do not apply to a three-kernel entry
    keyed = Config("- File: t\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n    - batch_norm_collect_statistics_kernel\n  Split: 128\n",
                   KERNELS_MAP.replace("X: 512", "X: 256", 1))
    with pytest.raises(hfuse_amd.HfuseError) as e:
        keyed.plan(0)
    assert e.value.code == L.HF_EINVAL and "Blocks" in e.value.message
    # a pair through the n-kernel calls
    pair = Config(FUSION, KERNELS_MAP).plan(0)
    pair.set_block_n(128, 256)
    assert list(pair.partition_n.hi)[:2] == [128, 384] and pair.partition_n.n == 2
    # the shipped three-kernel list and its Blocks key
    t = hfuse_amd.triples_config()
    assert [list(t.plan(i).partition_n.hi)[:3] for i in range(3)] == [[64, 192, 256], [256, 640, 768], [512, 768, 1024]]
    with pytest.raises(hfuse_amd.HfuseError) as e:   # one thread count per kernel
        Config("- File: t\n  Kernels:\n    - a\n    - b\n  Blocks:\n    - 64\n    - 64\n    - 64\n", KERNELS_MAP.replace("im2col_kernel:", "a:").replace("MaxPoolForward:", "b:"))
    assert e.value.code == L.HF_EPARSE and "Blocks" in e.value.message


def test_shipped_preset_and_its_keys():
    """`Preset:` names the preset an entry ships with (one of the driver's four, main.cpp:182-193); "shipped" asks for
    it.  Under a vertical preset `Blocks:` gives the threads that run each body and `Grids:` the workgroups each
    body strides over; a plan of any other preset ignores both."""
    text = ("- File: a\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n  Split: 256\n  Threads: 704\n"
            "  Preset: vfuse\n  Blocks:\n    - 768\n    - 1024\n  Grids:\n    - 256\n    - 512\n"
            "- File: b\n  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n  Split: 256\n  Threads: 704\n")
    cfg = Config(text, KERNELS_MAP)
    v = cfg.plan(0, "shipped").partition
    assert v.name.decode() == "im2col_kernel_MaxPoolForward_fused_kernel_vfuse_block_768_1024"
    assert (list(v.lo), list(v.hi), v.launch_threads) == ([0, 0], [768, 1024], 1024)
    h = cfg.plan(0, "hfuse").partition                      # the thread partition keeps its own tuned shape
    assert (list(h.hi), h.launch_threads) == ([256, 704], 704)
    assert cfg.plan(0, "vfuse", 0).partition.launch_threads == 512   # an explicit variant: the table's BlockDims
    s = cfg.plan(1, "shipped").partition                    # no Preset key: the thread partition
    assert s.name.decode().startswith("im2col_kernel_MaxPoolForward_fused_kernel_hfuse") and list(s.hi) == [256, 704]
    for bad in ("  Preset: fast\n", "  Grids:\n    - 1\n", "  Grids: 5\n", "  Blocks:\n    - 100\n    - 64\n"):
        with pytest.raises(hfuse_amd.HfuseError) as e:
            Config("- File: a\n" + bad + "  Kernels:\n    - im2col_kernel\n    - MaxPoolForward\n", KERNELS_MAP)
        assert e.value.code == L.HF_EPARSE
    with pytest.raises(hfuse_amd.HfuseError) as e:
        cfg.plan(0, "fastest")
    assert e.value.code == L.HF_ENOTFOUND


def test_header_symbols_are_all_exported():
    """Every function include/hfuse_gfx950.h declares is exported by the built library."""
    import os
    hdr = open(os.path.join(os.path.dirname(hfuse_amd.__file__), "..", "include", "hfuse_gfx950.h")).read()
    declared = set(re.findall(r"HF_API\s+[\w\s\*]+?\b(hf_\w+)\s*\(", hdr))
    assert len(declared) >= 20
    assert declared == set(L.PROTOTYPES), declared ^ set(L.PROTOTYPES)
    lib = L.lib()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.hf_version() == L.ABI_VERSION == 300   # _lib.lib() refuses any other build


def test_deep_nesting_is_refused_not_followed():
    """A file nested thousands of levels deep must come back as a parse error (bounded recursion)."""
    deep = "".join(" " * i + f"k{i}:\n" for i in range(5000)) + " " * 5000 + "v: 1\n"
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config(None, deep)
    assert e.value.code == L.HF_EPARSE and "nesting" in e.value.message
    seqs = "".join(" " * i + "-\n" for i in range(5000)) + " " * 5000 + "- x\n"
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config(seqs, KERNELS_MAP)
    assert e.value.code == L.HF_EPARSE


def test_partition_matches_oracle_on_random_kernel_tables():
    """Seeded random tables (block shapes, Reg, ExecTime), every preset, every split of the
    enumeration plus the ExecTime split: the library's partition, block shapes, launch threads,
    launch-bounds hint and index remap equal the oracle's Context wherever the library accepts
    the variant, and what it refuses is a part that is empty or not a multiple of 64 / BlockDim.Y."""
    import random
    rng = random.Random(20240607)
    checked = refused = 0
    for case in range(300):
        rows = []
        for _ in range(2):
            y = rng.choice([1, 1, 1, 2, 4, 8, 16])
            x = rng.choice([32, 64, 128, 192, 256, 320, 512, 768, 1024]) // y
            if x == 0 or x * y > 1024:
                x, y = 64, 1
            rows.append(((x, y, 1), rng.choice([8, 16, 24, 32, 49, 64, 128, 255]), rng.choice([-1.0, 1.0, 17.0, 52.5, 95.0])))
        total = sum(r[0][0] * r[0][1] for r in rows)
        if total > 1024:
            continue
        names = ("im2col_kernel", "MaxPoolForward")   # any two built kernels: only the table's numbers matter here
        table = "".join(f"k{i}:\n  KernelName: {names[i]}\n  HasBarriers: false\n  BlockDim:\n    X: {r[0][0]}\n    Y: {r[0][1]}\n    Z: 1\n"
                        f"  Reg: {r[1]}\n" + (f"  ExecTime: {r[2]}\n" if r[2] > 0 else "") for i, r in enumerate(rows))
        cfg = Config("- File: f\n  Kernels:\n    - k0\n    - k1\n", table)
        assert cfg.num_splits(0) == len(O.enumerate_splits(rows, granule=64))
        variants = [(idx, [(rows[0][0], rows[0][1], float(128 * (idx + 1))), (rows[1][0], rows[1][1], float(total - 128 * (idx + 1)))])
                    for idx in range(cfg.num_splits(0))]
        if rows[0][2] > 0 and rows[1][2] > 0:
            variants.append((L.HF_SPLIT_EXECTIME, rows))
        for idx, ex in variants:
            for preset, lb in (("hfuse", False), ("hfuse_lb", True)):
                try:
                    want = O.context(ex, launch_bound=lb, imbalanced=True, granule=64, reg_file=4 * 512 * 64, max_threads=2048)
                except ValueError:
                    want = None
                try:
                    got = cfg.plan(0, preset, idx).partition
                except hfuse_amd.HfuseError as e:
                    assert e.code == L.HF_EINVAL
                    refused += 1
                    if want is not None:   # the reference's arithmetic allows it; here a part must be whole wavefronts / rows
                        parts = [want.hi[h] - want.lo[h] for h in range(2)]
                        assert any(p == 0 or p % 64 or p % rows[h][0][1] for h, p in enumerate(parts)), (rows, idx, parts)
                    continue
                assert want is not None, (rows, idx)
                assert list(got.lo) == list(want.lo) and list(got.hi) == list(want.hi), (rows, idx)
                for h in range(2):
                    assert (got.block_dim[h].x, got.block_dim[h].y) == (want.block_dim[h].x, want.block_dim[h].y)
                assert got.launch_threads == want.launch_threads and got.launch_blocks == want.launch_blocks
                checked += 1
        for preset, lb in (("vfuse", False), ("vfuse_lb", True)):
            want = O.context(rows, base_line=True, launch_bound=lb, imbalanced=False, granule=64, reg_file=4 * 512 * 64, max_threads=2048)
            try:
                got = cfg.plan(0, preset, 0).partition
            except hfuse_amd.HfuseError as e:   # the vertical kernel runs whole wavefronts of each body too
                assert e.code == L.HF_EINVAL and any((r[0][0] * r[0][1]) % 64 for r in rows), rows
                refused += 1
                continue
            assert not any((r[0][0] * r[0][1]) % 64 for r in rows), rows
            assert list(got.lo) == [0, 0] == list(want.lo) and list(got.hi) == list(want.hi)
            assert got.launch_threads == want.launch_threads and got.launch_blocks == want.launch_blocks
            checked += 1
    assert checked > 800 and refused > 10


def test_native_threads_key():
    """`NativeThreads` (not in the reference's schema) names the block of the unfused launch; BlockDim stays
    the basis of the split enumeration."""
    row = "k:\n  KernelName: kernelHistogram1D\n  HasBarriers: true\n  BlockDim:\n    X: 512\n    Y: 1\n    Z: 1\n  Reg: 19\n"
    fusion = "- File: f\n  Kernels:\n    - k\n    - k\n"
    cfg = Config(fusion, row + "  NativeThreads: 768\n")
    info = cfg.kernel("k")
    assert info.native_threads == 768 and info.block_dim.x == 512
    assert Config(fusion, row).kernel("k").native_threads == 512
    assert cfg.num_splits(0) == 7                       # 128 * (n + 1) < 512 + 512, whatever the native block
    for bad in ("0", "100", "2048", "many"):
        with pytest.raises(hfuse_amd.HfuseError) as e:
            Config(fusion, row + f"  NativeThreads: {bad}\n")
        assert e.value.code == L.HF_EPARSE and "NativeThreads" in e.value.message
    assert hfuse_amd.default_config().kernel("kernelHistogram1D").native_threads == 768
