"""What the compiler made of every kernel in the built library, read from its code objects.

A kernel body that is not inlined into the fused kernel becomes a call: the kernel then carries a
private stack per lane and the callee's worst-case register count, which costs the fused
histogram pairs a factor of three on the GPU while every result stays right.  These checks see
that at build time, on the CPU.
"""
import re

import pytest

from hfuse_amd import _lib
from hfuse_amd.codeobj import kernel_resources, offload_bundles, short_name

# The launch-bound presets' builds are compiled for 8 waves per SIMD and may spill: that is their point.
def bounded(r):
    return "_lb<" in short_name(r.name)


TENSOR = ("Im2col", "MaxPool", "BnStats", "UpsampleNearest", "UpsampleBilinear", "Histc")
SEARCH = ("Sha256d", "Blake2b", "Ethash")


@pytest.fixture(scope="module")
def rows():
    r = kernel_resources()
    assert r, "no gfx950 kernels found in " + str(_lib.LIB_PATH)
    return r


def test_library_holds_gfx950_code_objects():
    blob = open(_lib.LIB_PATH, "rb").read()
    triples = [t for t, obj in offload_bundles(blob) if obj]
    assert triples and all("gfx950" in t for t in triples)


def test_every_kernel_family_is_present(rows):
    names = [short_name(r.name) for r in rows]
    for body in TENSOR + SEARCH:
        # (im2col's native kernel is the build with its residency capped)
        assert any(n.startswith(("native_kernel<" + body, "native_kernel_capped<" + body)) for n in names), body
    for kind in ("fused_kernel<", "vertical_kernel<", "blockidx_kernel<", "fused_kernel_lb<", "vertical_kernel_lb<"):
        assert sum(n.startswith(kind) for n in names) >= 20, kind


def test_no_vector_spills_and_no_dynamic_stack(rows):
    # (scalar registers may spill: they go to lanes of a vector register, not to memory)
    bad = [short_name(r.name) for r in rows if (r.vgpr_spills and not bounded(r)) or r.dynamic_stack]
    assert not bad, bad


def test_tensor_kernels_have_no_private_stack(rows):
    bad = [(short_name(r.name), r.private_bytes) for r in rows
           if r.private_bytes and not bounded(r) and not any(s in r.name for s in SEARCH)]
    assert not bad, bad


def test_search_kernels_only_carry_the_record_helper_stack(rows):
    # the rarely taken "record a hit" helper is deliberately a call; its frame is 48 bytes
    bad = [(short_name(r.name), r.private_bytes) for r in rows
           if any(s in r.name for s in SEARCH) and not bounded(r) and r.private_bytes > 64]
    assert not bad, bad


def test_fusing_never_halves_occupancy(rows):
    """A fused kernel needs about the registers of its hungrier half, not more than 1.25x."""
    native = {}
    for r in rows:
        m = re.match(r"native_kernel(?:_capped)?<(.+?), \d+(?:, \d+)?>$", short_name(r.name))
        if m:
            native[m.group(1)] = r
    checked = 0
    for r in rows:
        m = re.match(r"fused_kernel<(.+), (\d+), (true|false)>$", short_name(r.name))
        if not m:
            continue
        halves = [h for h in native if m.group(1).startswith(h + ", ") or m.group(1).endswith(", " + h)]
        if len(halves) < 1:
            continue
        need = max(native[h].vgpr for h in halves)
        assert r.vgpr <= 1.25 * need + 8, (short_name(r.name), r.vgpr, need)
        checked += 1
    assert checked >= 20


def test_bounded_builds_fit_their_waves_per_simd(rows):
    """A build bounded for W waves per SIMD holds at most 512 / W vector registers (in granules of 8):
    64 for the 8-wave build every pair has, 72 / 80 / 96 for the 7- / 6- / 5-wave builds of the benchmarked pairs."""
    lb = [r for r in rows if bounded(r)]
    assert len(lb) >= 40
    budget = {8: 64, 7: 72, 6: 80, 5: 96}
    seen = set()
    bad = []
    for r in lb:
        m = re.search(r", (\d+)>$", short_name(r.name))
        waves = int(m.group(1)) if m and "fused_kernel_lb" in short_name(r.name) else 8
        seen.add(waves)
        if r.vgpr + r.agpr > budget[waves]:
            bad.append((short_name(r.name), r.vgpr + r.agpr, waves))
    assert not bad, bad
    assert {5, 6, 7, 8} <= seen


def test_cli_prints_a_table(capsys):
    from hfuse_amd.codeobj import main

    assert main(["--match", "native_kernel"]) == 0
    out = capsys.readouterr().out
    assert "native_kernel<Histc, 1024>" in out and "waves/SIMD" in out
