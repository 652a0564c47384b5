"""Seeded mutation test of the YAML reader and the partition model under ASan + UBSan (host code only)."""
import os
import subprocess

import pytest

import hfuse_amd
from hfuse_amd import _lib as L
from hfuse_amd.launcher import Config

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(os.path.abspath(hfuse_amd.__file__))
CSRC = os.path.join(PKG, "csrc")


@pytest.fixture(scope="module")
def fuzzer(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("fuzz") / "host_fuzz")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
                           "-fno-sanitize-recover=undefined", "-static-libasan", "-static-libubsan", "-I", os.path.join(HERE, "..", "include"),
                           os.path.join(HERE, "host_fuzz.cpp"), os.path.join(CSRC, "fusion_model.cpp"),
                           os.path.join(CSRC, "yaml_lite.cpp"), "-o", exe])
    return exe


@pytest.mark.parametrize("fusion", ["gfx950_fusion.yaml", "gfx950_triples.yaml"])
@pytest.mark.parametrize("maxmut", [1, 6])
def test_mutated_configs_never_crash_the_host_model(fuzzer, maxmut, fusion):
    env = dict(os.environ, MAXMUT=str(maxmut))
    r = subprocess.run([fuzzer, os.path.join(PKG, "configs", fusion),
                        os.path.join(PKG, "configs", "gfx950_kernels.yaml"), "12000"],
                       capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    ok, bad = (int(x) for x in r.stdout.split()[1::2])
    assert ok > 200 and bad > 200   # both sides of the parser are exercised


@pytest.mark.parametrize("dim", ["X: 0", "Y: 0", "X: 2048", "X: 64\n    Y: 64"])
def test_block_dim_must_be_launchable(dim):
    """A zero or oversized BlockDim used to reach a division in the launch-bounds formula."""
    body = dim if "Y:" in dim and "X:" in dim else (dim + "\n    Y: 1" if dim.startswith("X") else "X: 64\n    " + dim)
    table = f"k:\n  KernelName: im2col_kernel\n  HasBarriers: false\n  BlockDim:\n    {body}\n    Z: 1\n  Reg: 8\n"
    with pytest.raises(hfuse_amd.HfuseError) as e:
        Config("- File: a\n  Kernels:\n    - k\n    - k\n", table)
    assert e.value.code == L.HF_EPARSE and "BlockDim" in e.value.message


def test_allocation_failures_come_back_as_error_codes(tmp_path):
    """Every host allocation of config loading and plan creation fails once (injected through a
    replaced `operator new`): the C-ABI answers HF_ENOMEM, no exception crosses the boundary."""
    exe = str(tmp_path / "alloc_fault")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-I", os.path.join(HERE, "..", "include"),
                           os.path.join(HERE, "alloc_fault.cpp"), "-L", PKG, "-lhfuse_gfx950",
                           "-Wl,-rpath," + PKG, "-o", exe])
    r = subprocess.run([exe, os.path.join(PKG, "configs", "gfx950_fusion.yaml"),
                        os.path.join(PKG, "configs", "gfx950_kernels.yaml")],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout + r.stderr)[-2000:]
    words = r.stdout.split()
    assert int(words[1]) > 100 and int(words[3]) >= 1   # that many distinct allocations were failed
