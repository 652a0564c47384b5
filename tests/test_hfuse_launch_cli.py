"""The C++ host program over the C-ABI: for every shipped pair it must report that the fused
launch wrote the same bytes as the two native launches (small shapes; full shapes for two pairs)."""
import os
import subprocess

import pytest

import hfuse_amd

pytestmark = pytest.mark.gpu
PKG = os.path.dirname(os.path.abspath(hfuse_amd.__file__))
TOOL = os.path.join(PKG, "hfuse-launch")
FUSION = os.path.join(PKG, "configs", "gfx950_fusion.yaml")
KERNELS = os.path.join(PKG, "configs", "gfx950_kernels.yaml")


def run(*extra):
    assert os.path.exists(TOOL), "build the library first (make -C hfuse_amd/csrc)"
    return subprocess.run([TOOL, FUSION, KERNELS, *extra], capture_output=True, text=True, timeout=300)


def test_every_shipped_pair_small(cuda):
    cfg = hfuse_amd.default_config()
    for i, (file, k1, k2) in enumerate(cfg.fusions()):
        # the benchmarked pairs also under the vertical and the register-bounded presets
        for extra in ((), ("--preset", "vfuse"), ("--preset", "hfuse_lb"), ("--preset", "vfuse_lb")) if i < 5 else ((),):
            r = run(str(i), "--small", "--iters", "3", *extra)
            assert r.returncode == 0, (file, r.stdout, r.stderr)
            assert f"fused == native: {k1} yes, {k2} yes" in r.stdout
            assert "speedup of the fused kernel over back to back" in r.stdout


@pytest.mark.parametrize("pair", ["NormalizationUpSample", "SummaryMaxpool"])
def test_benchmark_shapes(cuda, pair):
    r = run(pair, "--iters", "10")
    assert r.returncode == 0, (r.stdout, r.stderr)
    assert r.stdout.count(" yes") == 2


def test_all_pairs_in_one_run(cuda):
    r = run("all", "--small", "--iters", "2")
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr)
    cfg = hfuse_amd.default_config()
    assert r.stdout.count("fused == native:") == cfg.num_fusions
    assert " NO" not in r.stdout and "fused over back to back" in r.stdout


def test_three_kernel_list_small(cuda):
    cfg = hfuse_amd.triples_config()
    triples = os.path.join(PKG, "configs", "gfx950_triples.yaml")
    assert os.path.exists(TOOL), "build the library first (make -C hfuse_amd/csrc)"
    r = subprocess.run([TOOL, triples, KERNELS, "all", "--small", "--iters", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr)
    assert r.stdout.count("fused == native:") == 3 * cfg.num_fusions
    assert " NO" not in r.stdout and "three native launches back to back" in r.stdout


def test_errors(cuda):
    assert run("NoSuchPair").returncode == 1
    assert run("0", "--preset", "hfuse_bar_sync").returncode == 1
    assert subprocess.run([TOOL], capture_output=True).returncode == 2
