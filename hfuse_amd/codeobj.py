"""Register, LDS and private-stack use of every kernel in the built library.

The library's gfx950 code objects sit in clang offload bundles inside the shared object; each
code object is an ELF whose NT_AMDGPU_METADATA note (type 32, MessagePack) lists, per kernel,
the numbers the loader uses to size a wave: `.vgpr_count`, `.agpr_count`, `.sgpr_count`,
`.group_segment_fixed_size` (static LDS), `.private_segment_fixed_size` (bytes of stack per
lane) and the spill counts.  The reference bounds registers per fused kernel from the outside
(`__launch_bounds__` it prints, lib/KernelFuser/KernelPrinter.cpp:70-80, and the register caps
its build scripts sweep); here the compiler's result is read back, so a body that stops being
inlined (a call, a private stack, occupancy halved) is seen at build time, not on the GPU.

    python -m hfuse_amd.codeobj [--lib PATH] [--match REGEX]
"""
from __future__ import annotations

import argparse
import re
import struct
import subprocess
from dataclasses import dataclass
from pathlib import Path
from typing import Iterator, List

_BUNDLE_MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"
_SHT_NOTE = 7
_NT_AMDGPU_METADATA = 32
_VGPR_FILE = 512        # gfx950: unified VGPR+AGPR file per SIMD lane
_VGPR_GRANULE = 8
_MAX_WAVES = 8          # per SIMD
_SGPR_FILE = 800        # per SIMD, allocated in granules of 16
_SGPR_GRANULE = 16


@dataclass(frozen=True)
class KernelResources:
    symbol: str
    name: str            # demangled where c++filt is present
    vgpr: int
    agpr: int
    sgpr: int
    lds_static: int
    private_bytes: int   # stack per lane; > 0 means spills, arrays in memory or a real call
    vgpr_spills: int
    sgpr_spills: int
    dynamic_stack: bool
    max_threads: int

    @property
    def waves_per_simd(self) -> int:
        """Waves of this kernel one SIMD can hold by registers alone."""
        regs = max(self.vgpr + self.agpr, 1)
        regs = (regs + _VGPR_GRANULE - 1) // _VGPR_GRANULE * _VGPR_GRANULE
        scalars = (max(self.sgpr, 1) + _SGPR_GRANULE - 1) // _SGPR_GRANULE * _SGPR_GRANULE
        return max(1, min(_MAX_WAVES, _VGPR_FILE // regs, _SGPR_FILE // scalars))


def offload_bundles(blob: bytes) -> Iterator[tuple]:
    """(target triple, code object bytes) of every entry of every bundle in `blob`."""
    pos = 0
    while True:
        at = blob.find(_BUNDLE_MAGIC, pos)
        if at < 0:
            return
        (count,) = struct.unpack_from("<Q", blob, at + len(_BUNDLE_MAGIC))
        cursor = at + len(_BUNDLE_MAGIC) + 8
        for _ in range(count):
            offset, size, triple_len = struct.unpack_from("<QQQ", blob, cursor)
            cursor += 24
            triple = blob[cursor:cursor + triple_len].decode("ascii", "replace")
            cursor += triple_len
            yield triple, blob[at + offset:at + offset + size]
        pos = at + len(_BUNDLE_MAGIC)


def _metadata_notes(elf: bytes) -> Iterator[dict]:
    import msgpack

    if elf[:4] != b"\x7fELF" or elf[4] != 2:
        raise ValueError("not a 64-bit ELF code object")
    (shoff,) = struct.unpack_from("<Q", elf, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", elf, 0x3A)
    for k in range(shnum):
        base = shoff + k * shentsize
        (sh_type,) = struct.unpack_from("<I", elf, base + 4)
        if sh_type != _SHT_NOTE:
            continue
        offset, size = struct.unpack_from("<QQ", elf, base + 0x18)
        p = offset
        while p + 12 <= offset + size:
            namesz, descsz, ntype = struct.unpack_from("<III", elf, p)
            p += 12 + ((namesz + 3) & ~3)
            desc = elf[p:p + descsz]
            p += (descsz + 3) & ~3
            if ntype == _NT_AMDGPU_METADATA:
                yield msgpack.unpackb(desc, raw=False)


def _demangle(symbols: List[str]) -> List[str]:
    try:
        out = subprocess.run(["c++filt"], input="\n".join(symbols), capture_output=True, text=True, check=True)
        names = out.stdout.splitlines()
        if len(names) == len(symbols):
            return names
    except (OSError, subprocess.CalledProcessError):
        pass
    return list(symbols)


def kernel_resources(lib_path=None, arch: str = "gfx950") -> List[KernelResources]:
    """One row per kernel of `arch` in the library (default: the in-tree build)."""
    if lib_path is None:
        from . import _lib
        lib_path = _lib.LIB_PATH
    blob = Path(lib_path).read_bytes()
    rows = []
    for triple, obj in offload_bundles(blob):
        if arch not in triple or not obj:
            continue
        for meta in _metadata_notes(obj):
            for k in meta.get("amdhsa.kernels", []):
                rows.append((k[".name"], k))
    names = _demangle([s for s, _ in rows])
    return [
        KernelResources(
            symbol=s, name=n, vgpr=k.get(".vgpr_count", 0), agpr=k.get(".agpr_count", 0),
            sgpr=k.get(".sgpr_count", 0), lds_static=k.get(".group_segment_fixed_size", 0),
            private_bytes=k.get(".private_segment_fixed_size", 0),
            vgpr_spills=k.get(".vgpr_spill_count", 0), sgpr_spills=k.get(".sgpr_spill_count", 0),
            dynamic_stack=bool(k.get(".uses_dynamic_stack", False)),
            max_threads=k.get(".max_flat_workgroup_size", 0))
        for (s, k), n in zip(rows, names)
    ]


def short_name(name: str) -> str:
    """`fused_kernel<Histc, MaxPool, 1024, false>` from the demangled signature."""
    head = name.split("(", 1)[0].replace("void ", "").replace("hfuse::", "")
    return head.replace("Body", "")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--lib", default=None, help="shared object to read (default: the in-tree build)")
    ap.add_argument("--match", default=".", help="only kernels whose short name matches this regex")
    args = ap.parse_args(argv)
    rows = [r for r in kernel_resources(args.lib) if re.search(args.match, short_name(r.name))]
    print(f"{'kernel':<64} {'vgpr':>4} {'agpr':>4} {'sgpr':>4} {'lds':>6} {'stack':>5} {'spill':>5} {'waves/SIMD':>10}")
    for r in sorted(rows, key=lambda r: short_name(r.name)):
        print(f"{short_name(r.name):<64} {r.vgpr:>4} {r.agpr:>4} {r.sgpr:>4} {r.lds_static:>6} "
              f"{r.private_bytes:>5} {r.vgpr_spills + r.sgpr_spills:>5} {r.waves_per_simd:>10}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
