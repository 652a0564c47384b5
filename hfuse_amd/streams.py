"""Stream ceilings of the part, measured with the library's bare stream kernels (hf_stream_probe).

Every tensor kernel of the library is bound by HBM traffic, and what HBM delivers depends on the access
pattern: contiguous reads, contiguous writes, random 128-byte lines and a 1 : 4 read / write mix reach different
rates, all below the data sheet's 8 TB/s.  `measure()` times each pattern on rotating buffers (so that no launch
re-reads what the 256 MB memory-side cache still holds) over a few launch shapes and returns the best of each:
the rates `bench.py` judges the kernels against, taken in the same run as the kernels.

    python -m hfuse_amd.streams          # prints the table as JSON
"""
from __future__ import annotations

import ctypes as C
import json
import statistics

from . import _lib as L
from .launcher import _stream_ptr, check

MIB = 1 << 20

# launch shapes tried per pattern: (workgroups, threads)
READ_SHAPES = ((256, 256), (512, 256), (256, 512), (1024, 256), (2048, 256))
WRITE_SHAPES = ((256, 256), (512, 256), (1024, 256), (4096, 256), (16384, 256), (131072, 256))   # the last: one store a thread
LINES_SHAPES = ((8192, 128), (32768, 128), (8192, 256))
COPY_SHAPES = ((1024, 256), (4096, 256), (16384, 256), (4096, 512), (32768, 256), (16384, 512))   # the last two: one vector a thread


def _time(pattern, src, dst, nbytes, src_stride, dst_stride, nbuf, grid, block, warmup, iters, rounds=3):
    """Median over `rounds` of the microseconds per launch (events on the launch stream, launches issued from C)."""
    out = []
    for r in range(rounds):
        ms = C.c_float()
        check(L.lib().hf_time_stream_probe(pattern, C.c_void_p(src), C.c_void_p(dst), nbytes, src_stride, dst_stride, nbuf,
                                           grid, block, warmup if r == 0 else 1, iters, _stream_ptr(), C.byref(ms)))
        out.append(ms.value * 1e3 / iters)
    return statistics.median(out)


def measure(buf_mib: int = 512, nbuf: int = 8, iters: int = 16) -> dict:
    """-> {"read_gbps", "write_gbps", "read_lines_gbps", "copy_1_4_gbps", "empty_launch_us", "shapes": {...}, ...}

    `nbuf` buffers of `buf_mib` MiB in one allocation (4 GiB by default: the random lines roam over all of it)."""
    import torch
    nbytes = buf_mib * MIB
    pool = torch.ones(nbuf * nbytes // 4, dtype=torch.float32, device="cuda")
    sink = torch.zeros(4, dtype=torch.float32, device="cuda")
    base = pool.data_ptr()
    res, shapes, table = {}, {}, {}

    def best(name, rows):
        rows.sort(reverse=True)
        res[name + "_gbps"] = rows[0][0]
        shapes[name] = {"pattern": rows[0][1], "grid": rows[0][2], "block": rows[0][3]}
        table[name] = [{"pattern": p, "grid": g, "block": b, "us": round(us, 2), "gbps": round(r, 1)} for r, p, g, b, us in rows]

    rows = []
    for grid, block in READ_SHAPES:
        us = _time(L.HF_STREAM_READ, base, sink.data_ptr(), nbytes, nbytes, 0, nbuf, grid, block, 3, iters)
        rows.append((nbytes / us / 1e3, "contiguous share per workgroup", grid, block, us))
    best("read", rows)
    rows = []
    for pattern, what in ((L.HF_STREAM_WRITE, "contiguous share per workgroup"), (L.HF_STREAM_WRITE_STRIDED, "grid-stride loop"),
                          (L.HF_STREAM_WRITE_XCD, "contiguous share per workgroup, one eighth per XCD")):
        for grid, block in WRITE_SHAPES:
            us = _time(pattern, 0, base, nbytes, 0, nbytes, nbuf, grid, block, 3, iters)
            rows.append((nbytes / us / 1e3, what, grid, block, us))
    best("write", rows)
    # random lines over the whole pool; one launch reads the pool's size once
    total = nbuf * nbytes
    rows = []
    for grid, block in LINES_SHAPES:
        us = _time(L.HF_STREAM_READ_LINES, base, sink.data_ptr(), total, 0, 0, 1, grid, block, 1, 4)
        rows.append((total / us / 1e3, "random 128-byte lines", grid, block, us))
    best("read_lines", rows)
    # 1 : 4 copy: a quarter of a buffer read from the lower half of the pool, a whole buffer written in the upper half
    quarter = nbytes // 4
    rows = []
    for grid, block in COPY_SHAPES:
        us = _time(L.HF_STREAM_COPY_1_4, base, base + (nbuf // 2) * nbytes, quarter, nbytes, nbytes, nbuf // 2, grid, block, 3, iters)
        rows.append((5 * quarter / us / 1e3, "1 read : 4 writes", grid, block, us))
    best("copy_1_4", rows)
    res["empty_launch_us"] = _time(L.HF_STREAM_EMPTY, 0, 0, 0, 0, 0, 1, 1, 64, 20, 400)
    res["shapes"] = shapes
    res["table"] = table
    res["buffer_mib"], res["buffers"] = buf_mib, nbuf
    torch.cuda.synchronize()
    del pool
    torch.cuda.empty_cache()
    return res


if __name__ == "__main__":
    print(json.dumps(measure(), indent=1))
