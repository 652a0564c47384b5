"""The library's bare stream kernels (hf_stream_probe): argument checks without a GPU; on the GPU every pattern
writes / copies what it says and the measured ceilings are plausible for this part."""
import ctypes as C

import pytest

import hfuse_amd
from hfuse_amd import _lib as L
from hfuse_amd.launcher import check

PATTERNS = (L.HF_STREAM_EMPTY, L.HF_STREAM_READ, L.HF_STREAM_WRITE, L.HF_STREAM_READ_LINES, L.HF_STREAM_COPY_1_4,
            L.HF_STREAM_WRITE_STRIDED, L.HF_STREAM_WRITE_XCD)


def probe(pattern, src, dst, nbytes, grid, block):
    return L.lib().hf_stream_probe(pattern, C.c_void_p(src), C.c_void_p(dst), nbytes, grid, block, None)


def test_pattern_numbers_are_the_header_s():
    assert PATTERNS == (0, 1, 2, 3, 4, 5, 6)


@pytest.mark.parametrize("pattern,src,dst,nbytes,grid,block,needle", [
    (7, 4096, 4096, 4096, 1, 64, "pattern"),
    (-1, 4096, 4096, 4096, 1, 64, "pattern"),
    (L.HF_STREAM_READ, 0, 4096, 4096, 1, 64, "null"),
    (L.HF_STREAM_WRITE, 0, 0, 4096, 1, 64, "null"),
    (L.HF_STREAM_COPY_1_4, 4096, 0, 4096, 1, 64, "null"),
    (L.HF_STREAM_READ, 4100, 4096, 4096, 1, 64, "aligned"),
    (L.HF_STREAM_WRITE, 0, 4104, 4096, 1, 64, "aligned"),
    (L.HF_STREAM_READ, 4096, 4096, 4096, 0, 64, "grid"),
    (L.HF_STREAM_READ, 4096, 4096, 4096, 1, 96, "grid"),
    (L.HF_STREAM_READ, 4096, 4096, 4096, 1, 2048, "grid"),
    (L.HF_STREAM_WRITE_XCD, 0, 4096, 4096, 4, 64, "eight"),
    (L.HF_STREAM_READ, 4096, 4096, 0, 1, 64, "bytes"),
    (L.HF_STREAM_READ, 4096, 4096, 16 * 3 + 16, 3, 64, "bytes"),       # 64 bytes over 3 workgroups
    (L.HF_STREAM_READ_LINES, 4096, 4096, 4096, 1, 128, "bytes"),       # needs 64 * grid * block
])
def test_argument_checks_come_before_any_launch(pattern, src, dst, nbytes, grid, block, needle):
    """Refused calls return HF_EINVAL with a message and touch no memory (the pointers here are not mapped)."""
    assert probe(pattern, src, dst, nbytes, grid, block) == L.HF_EINVAL
    assert needle in L.lib().hf_last_error().decode()
    ms = C.c_float(-1.0)
    rc = L.lib().hf_time_stream_probe(pattern, C.c_void_p(src), C.c_void_p(dst), nbytes, 0, 0, 1, grid, block, 0, 1, None, C.byref(ms))
    assert rc == L.HF_EINVAL and ms.value == -1.0


def test_repetition_arguments():
    ms = C.c_float()
    lib = L.lib()
    for nbuf, warmup, iters, ss, ds in ((0, 0, 1, 0, 0), (1, -1, 1, 0, 0), (1, 0, 0, 0, 0), (1, 0, 1, 8, 0), (1, 0, 1, 0, 24)):
        rc = lib.hf_time_stream_probe(L.HF_STREAM_WRITE, None, C.c_void_p(4096), 4096, ss, ds, nbuf, 1, 64, warmup, iters, None, C.byref(ms))
        assert rc == L.HF_EINVAL, (nbuf, warmup, iters, ss, ds)
    assert lib.hf_time_stream_probe(L.HF_STREAM_EMPTY, None, None, 0, 0, 0, 1, 1, 64, 0, 1, None, None) == L.HF_EINVAL


# ------------------------------------------------------------------ on the GPU
@pytest.mark.gpu
@pytest.mark.parametrize("pattern", [L.HF_STREAM_WRITE, L.HF_STREAM_WRITE_STRIDED, L.HF_STREAM_WRITE_XCD])
@pytest.mark.parametrize("grid,block", [(8, 64), (64, 256), (1024, 1024)])
def test_write_patterns_fill_exactly_the_buffer(cuda, pattern, grid, block):
    import torch
    n4 = grid * 37 * 8                 # vectors: a multiple of the grid that is no multiple of the block
    buf = torch.full((n4 * 4 + 8,), -7.0, device=cuda)
    check(probe(pattern, 0, buf.data_ptr() + 16, n4 * 16, grid, block))
    torch.cuda.synchronize()
    got = buf.cpu()
    assert got[:4].eq(-7.0).all() and got[-4:].eq(-7.0).all()              # nothing before or after
    body = got[4:-4].view(n4, 4)
    assert body[:, 0].eq(1.0).all() and body[:, 1].eq(2.0).all() and body[:, 2].eq(3.0).all()
    lane = body[:, 3]
    assert lane.min() >= 0 and lane.max() < block and (lane == lane.round()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("grid,block,n4", [(1, 64, 5), (16, 256, 16 * (256 * 3 + 5)), (512, 512, 1 << 20)])
def test_copy_1_4_writes_four_copies(cuda, grid, block, n4):
    import torch
    g = torch.Generator().manual_seed(n4)
    src = torch.rand(n4 * 4, generator=g).to(cuda)
    dst = torch.full((4 * n4 * 4 + 4,), -1.0, device=cuda)
    check(probe(L.HF_STREAM_COPY_1_4, src.data_ptr(), dst.data_ptr(), n4 * 16, grid, block))
    torch.cuda.synchronize()
    assert dst[-4:].eq(-1.0).all()
    assert torch.equal(dst[:-4].view(4, n4 * 4), src.expand(4, -1))


@pytest.mark.gpu
def test_read_patterns_leave_memory_alone(cuda):
    import torch
    src = torch.ones(1 << 22, device=cuda)                  # 16 MiB
    sink = torch.zeros(4, device=cuda)
    for grid, block in ((256, 256), (64, 1024), (7, 64)):
        nbytes = src.numel() * 4 // (16 * grid) * 16 * grid
        check(probe(L.HF_STREAM_READ, src.data_ptr(), sink.data_ptr(), nbytes, grid, block))
    for grid, block in ((128, 128), (16, 256)):
        check(probe(L.HF_STREAM_READ_LINES, src.data_ptr(), sink.data_ptr(), 1 << 24, grid, block))
    check(probe(L.HF_STREAM_EMPTY, 0, 0, 0, 1, 64))
    torch.cuda.synchronize()
    assert sink.eq(0.0).all() and src.eq(1.0).all()


@pytest.mark.gpu
def test_measured_ceilings_are_those_of_this_part(cuda):
    """A short measurement on small buffers: every rate is a sizeable fraction of the data sheet's 8 TB/s (a pool of
    1 GiB still hits the 256 MB memory-side cache now and then, so the bound above is loose); the figures bench.py
    judges against come from the same function with its default, larger buffers."""
    from hfuse_amd import streams
    r = streams.measure(buf_mib=128, nbuf=8, iters=8)
    for key in ("read_gbps", "write_gbps", "read_lines_gbps", "copy_1_4_gbps"):
        assert 2000.0 < r[key] < 12000.0, (key, r[key])
    assert 0.2 < r["empty_launch_us"] < 20.0
    assert set(r["shapes"]) == {"read", "write", "read_lines", "copy_1_4"}
    assert r["table"]["write"][0]["gbps"] == pytest.approx(r["write_gbps"], abs=0.06)
