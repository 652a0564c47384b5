"""The C command-line enumerator against the Python mirror of the same C-ABI calls."""
import os
import subprocess

import pytest

import hfuse_amd
from hfuse_amd import _lib as L
from hfuse_amd import launcher as H

PKG = os.path.dirname(os.path.abspath(hfuse_amd.__file__))
TOOL = os.path.join(PKG, "hfuse-plan")
FUSION = os.path.join(PKG, "configs", "gfx950_fusion.yaml")
KERNELS = os.path.join(PKG, "configs", "gfx950_kernels.yaml")
BARRIER = {L.HF_BARRIER_NONE: "none", L.HF_BARRIER_MATCHED: "matched", L.HF_BARRIER_SUBSET: "subset",
           L.HF_BARRIER_BLOCKIDX: "blockidx"}


@pytest.fixture(scope="module")
def tool():
    if not os.path.exists(TOOL):
        subprocess.check_call(["make", "-C", os.path.join(PKG, "csrc"), "../hfuse-plan"])
    return TOOL


def test_enumeration_matches_the_library(tool):
    out = subprocess.run([tool, FUSION, KERNELS], capture_output=True, text=True, check=True).stdout.splitlines()
    assert out[0].startswith("# file\tname\tpreset")
    rows = [ln.split("\t") for ln in out[1:] if not ln.startswith("#")]
    cfg = H.Config.from_files(FUSION, KERNELS)
    want = []
    for i, (file, k1, k2) in enumerate(cfg.fusions()):
        for preset in ("vfuse_lb", "vfuse", "hfuse", "hfuse_lb"):
            idxs = range(cfg.num_splits(i)) if preset.startswith("hfuse") else [0]
            for idx in idxs:
                p = cfg.plan(i, preset, idx).partition
                want.append([file, p.name.decode(), preset, str(idx), f"[{p.lo[0]},{p.hi[0]})", f"[{p.lo[1]},{p.hi[1]})",
                             "x".join(str(v) for v in (p.block_dim[0].x, p.block_dim[0].y, p.block_dim[0].z)),
                             "x".join(str(v) for v in (p.block_dim[1].x, p.block_dim[1].y, p.block_dim[1].z)),
                             str(p.launch_threads), str(p.launch_blocks), BARRIER[p.barrier_mode]])
    assert rows == want
    # the reference's naming: <K1>_<K2>_fused_kernel_<preset>_idx_<n> (KernelPrinter.cpp:67-70)
    assert all(r[1] == f"{r[1].split('_fused_kernel_')[0]}_fused_kernel_{r[2]}_idx_{r[3]}" for r in rows)


def test_three_kernel_entries(tool):
    """The shipped three-kernel list: every preset and split the driver's loop would print, three bounds a line."""
    triples = os.path.join(PKG, "configs", "gfx950_triples.yaml")
    out = subprocess.run([tool, triples, KERNELS], capture_output=True, text=True).stdout.splitlines()
    rows = [ln.split("\t") for ln in out if not ln.startswith("#")]
    cfg = H.Config.from_files(triples, KERNELS)
    seen = 0
    for i in range(cfg.num_fusions):
        file = cfg.fusion(i)[0]
        for preset in ("vfuse_lb", "vfuse", "hfuse", "hfuse_lb"):
            idxs = range(cfg.num_splits(i)) if preset.startswith("hfuse") else [0]
            for idx in idxs:
                try:
                    p = cfg.plan(i, preset, idx).partition_n
                except hfuse_amd.HfuseError:
                    continue      # printed as a comment line, as the reference prints the problem and goes on
                want = [file, p.name.decode(), preset, str(idx)] + [f"[{p.lo[k]},{p.hi[k]})" for k in range(3)] + \
                       ["x".join(str(v) for v in (p.block_dim[k].x, p.block_dim[k].y, p.block_dim[k].z)) for k in range(3)] + \
                       [str(p.launch_threads), str(p.launch_blocks), BARRIER[p.barrier_mode]]
                assert want in rows, want
                seen += 1
    assert seen >= 6 and len(rows) == seen


def test_per_pair_table_and_errors(tool, tmp_path):
    table = tmp_path / "pair.yaml"
    table.write_text("- KernelName: im2col_kernel\n  HasBarriers: false\n  BlockDim:\n    X: 512\n    Y: 1\n    Z: 1\n"
                     "- KernelName: MaxPoolForward\n  HasBarriers: false\n  BlockDim:\n    X: 256\n    Y: 1\n    Z: 1\n")
    out = subprocess.run([tool, "-", str(table)], capture_output=True, text=True, check=True).stdout
    assert "im2col_kernel_MaxPoolForward_fused_kernel_hfuse_idx_1\thfuse\t1\t[0,256)\t[256,768)" in out
    bad = subprocess.run([tool, FUSION, str(tmp_path / "missing.yaml")], capture_output=True, text=True)
    assert bad.returncode == 1 and "missing.yaml" in bad.stderr
    assert subprocess.run([tool], capture_output=True).returncode == 2
