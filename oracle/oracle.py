"""ctypes front-end of the CPU oracle (oracle/hfuse_oracle.c).

Test infrastructure only: imported by tests/, by the smoke check and by the
cpu_baseline leg of the benchmark -- never by the hfuse_amd package.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libhfuse_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a second or two)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libhfuse_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


class Dim3(C.Structure):
    _fields_ = [("x", C.c_uint32), ("y", C.c_uint32), ("z", C.c_uint32)]


class KernelInfo(C.Structure):
    _fields_ = [("block_dim", Dim3), ("reg", C.c_uint32), ("exec_time", C.c_double)]


class Partition(C.Structure):
    _fields_ = [("lo", C.c_uint32 * 2), ("hi", C.c_uint32 * 2), ("block_dim", Dim3 * 2),
                ("launch_threads", C.c_uint32), ("launch_blocks", C.c_uint32)]


class Hit(C.Structure):
    _fields_ = [("nonce", C.c_uint64), ("digest", C.c_uint32 * 8), ("mix", C.c_uint32 * 8)]

    def digest_bytes(self) -> bytes:
        return bytes(self.digest)

    def mix_bytes(self) -> bytes:
        return bytes(self.mix)


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.orc_splitmix64_at.restype = C.c_uint64
        _lib.orc_splitmix64_at.argtypes = [C.c_uint64, C.c_uint64]
        _lib.orc_sha256d_search.restype = C.c_int64
        _lib.orc_sia_search.restype = C.c_int64
        _lib.orc_ethash_search.restype = C.c_int64
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(C.POINTER(C.c_float))


def _u8(b: bytes):
    return (C.c_uint8 * len(b)).from_buffer_copy(b)


# ---------------------------------------------------------------- fusion model
def context(infos, base_line=False, launch_bound=False, imbalanced=True, granule=32,
            reg_file=65536, max_threads=2048) -> Partition:
    """infos: two tuples ((X,Y,Z), reg, exec_time)."""
    arr = (KernelInfo * 2)()
    for i, (dim, reg, t) in enumerate(infos):
        arr[i].block_dim = Dim3(*dim)
        arr[i].reg = reg
        arr[i].exec_time = t
    out = Partition()
    rc = lib().orc_context(arr, int(base_line), int(launch_bound), int(imbalanced),
                           C.c_uint32(granule), C.c_uint32(reg_file), C.c_uint32(max_threads),
                           C.byref(out))
    if rc != 0:
        raise ValueError("orc_context rejected the kernel table")
    return out


class PartitionN(C.Structure):
    _fields_ = [("lo", C.c_uint32 * 4), ("hi", C.c_uint32 * 4), ("block_dim", Dim3 * 4),
                ("launch_threads", C.c_uint32), ("launch_blocks", C.c_uint32)]


def context_n(infos, base_line=False, launch_bound=False, imbalanced=True, granule=32,
              reg_file=65536, max_threads=2048) -> PartitionN:
    """infos: up to four tuples ((X,Y,Z), reg, exec_time): the Context of a list of that many kernels."""
    n = len(infos)
    arr = (KernelInfo * n)()
    for i, (dim, reg, t) in enumerate(infos):
        arr[i].block_dim = Dim3(*dim)
        arr[i].reg = reg
        arr[i].exec_time = t
    out = PartitionN()
    rc = lib().orc_context_n(arr, n, int(base_line), int(launch_bound), int(imbalanced),
                             C.c_uint32(granule), C.c_uint32(reg_file), C.c_uint32(max_threads), C.byref(out))
    if rc != 0:
        raise ValueError("orc_context_n rejected the kernel table")
    return out


def enumerate_splits(infos, granule=32):
    arr = (KernelInfo * 2)()
    for i, (dim, reg, t) in enumerate(infos):
        arr[i].block_dim = Dim3(*dim)
        arr[i].reg = reg
        arr[i].exec_time = t
    out = (C.c_uint32 * 64)()
    n = lib().orc_enumerate_splits(arr, C.c_uint32(granule), out, 64)
    return [out[i] for i in range(n)]


def remap_tid(tid, lo, dim):
    out = Dim3()
    lib().orc_remap_tid(C.c_uint32(tid), C.c_uint32(lo), Dim3(*dim), C.byref(out))
    return out.x, out.y, out.z


# ---------------------------------------------------------------- tensor kernels
def im2col(x, kernel, pad, stride, dil=(1, 1)):
    """x: [channels(, batch folded in), H, W] float32 -> [channels*kh*kw, Hc, Wc]."""
    x, px = _f32(x)
    ch, h, w = x.shape
    kh, kw = kernel
    hc = (h + 2 * pad[0] - (dil[0] * (kh - 1) + 1)) // stride[0] + 1
    wc = (w + 2 * pad[1] - (dil[1] * (kw - 1) + 1)) // stride[1] + 1
    out = np.empty((ch * kh * kw, hc, wc), dtype=np.float32)
    i64 = C.c_int64
    lib().orc_im2col(i64(ch * hc * wc), px, i64(h), i64(w), i64(kh), i64(kw), i64(pad[0]),
                     i64(pad[1]), i64(stride[0]), i64(stride[1]), i64(dil[0]), i64(dil[1]),
                     i64(hc), i64(wc), out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def max_pool(x, kernel, stride, pad, dil=(1, 1)):
    """x: [N,C,H,W] float32 -> (values [N,C,PH,PW] f32, indices int64), floor mode."""
    x, px = _f32(x)
    n, c, h, w = x.shape
    ph = (h + 2 * pad[0] - dil[0] * (kernel[0] - 1) - 1) // stride[0] + 1
    pw = (w + 2 * pad[1] - dil[1] * (kernel[1] - 1) - 1) // stride[1] + 1
    val = np.empty((n, c, ph, pw), dtype=np.float32)
    idx = np.empty((n, c, ph, pw), dtype=np.int64)
    lib().orc_max_pool(C.c_int(val.size), px, n, c, h, w, ph, pw, kernel[0], kernel[1], stride[0],
                       stride[1], pad[0], pad[1], dil[0], dil[1],
                       val.ctypes.data_as(C.POINTER(C.c_float)),
                       idx.ctypes.data_as(C.POINTER(C.c_int64)))
    return val, idx


def upsample_nearest2d(x, out_hw, scales=None):
    x, px = _f32(x)
    n, c, h, w = x.shape
    h2, w2 = out_hw
    hs = np.float32(scales[0]) if scales else np.float32(h) / np.float32(h2)
    ws = np.float32(scales[1]) if scales else np.float32(w) / np.float32(w2)
    out = np.empty((n, c, h2, w2), dtype=np.float32)
    sz = C.c_size_t
    lib().orc_upsample_nearest2d(px, out.ctypes.data_as(C.POINTER(C.c_float)), sz(n * c), sz(h),
                                 sz(w), sz(h2), sz(w2), C.c_float(hs), C.c_float(ws))
    return out


def upsample_bilinear2d(x, out_hw, align_corners=False, scales=None):
    """x [N,C,H,W] float32 -> [N,C,H2,W2]; scales default to PyTorch's area_pixel_compute_scale."""
    x, px = _f32(x)
    n, c, h, w = x.shape
    h2, w2 = out_hw
    if scales:
        rh, rw = np.float32(scales[0]), np.float32(scales[1])
    elif align_corners:
        rh = np.float32(h - 1) / np.float32(h2 - 1) if h2 > 1 else np.float32(0)
        rw = np.float32(w - 1) / np.float32(w2 - 1) if w2 > 1 else np.float32(0)
    else:
        rh, rw = np.float32(h) / np.float32(h2), np.float32(w) / np.float32(w2)
    out = np.empty((n, c, h2, w2), dtype=np.float32)
    lib().orc_upsample_bilinear2d(px, out.ctypes.data_as(C.POINTER(C.c_float)), n, c, h, w, h2, w2,
                                  C.c_float(rh), C.c_float(rw), int(align_corners))
    return out


def histc(x, nbins, lo, hi):
    x, px = _f32(np.ravel(x))
    out = np.zeros(nbins, dtype=np.float32)
    lib().orc_histc(px, C.c_int64(x.size), C.c_int(nbins), C.c_float(lo), C.c_float(hi),
                    out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def bn_stats(x, eps):
    """x: [N,C,L] float32 -> (mean[C], invstd[C]) float32."""
    x, px = _f32(x)
    n, c, l = x.shape
    mean = np.empty(c, dtype=np.float32)
    inv = np.empty(c, dtype=np.float32)
    lib().orc_bn_stats(px, n, c, l, C.c_float(eps), mean.ctypes.data_as(C.POINTER(C.c_float)),
                       inv.ctypes.data_as(C.POINTER(C.c_float)))
    return mean, inv


def bn_stats_f64(x, eps):
    x, px = _f32(x)
    n, c, l = x.shape
    mean = np.empty(c, dtype=np.float64)
    inv = np.empty(c, dtype=np.float64)
    lib().orc_bn_stats_f64(px, n, c, l, C.c_double(eps),
                           mean.ctypes.data_as(C.POINTER(C.c_double)),
                           inv.ctypes.data_as(C.POINTER(C.c_double)))
    return mean, inv


# ---------------------------------------------------------------- seeded data
def splitmix64_at(seed, i):
    return lib().orc_splitmix64_at(C.c_uint64(seed), C.c_uint64(i))


def fill_splitmix64(nwords, seed):
    out = np.empty(nwords, dtype=np.uint64)
    lib().orc_fill_splitmix64(out.ctypes.data_as(C.POINTER(C.c_uint64)), C.c_uint64(nwords),
                              C.c_uint64(seed))
    return out


def seeded_bytes(n, seed) -> bytes:
    return fill_splitmix64((n + 7) // 8, seed).tobytes()[:n]


# ---------------------------------------------------------------- hashes
def sha256(msg: bytes) -> bytes:
    out = (C.c_uint8 * 32)()
    lib().orc_sha256(_u8(msg) if msg else None, C.c_uint64(len(msg)), out)
    return bytes(out)


def sha256d_80(header: bytes, nonce: int) -> bytes:
    out = (C.c_uint8 * 32)()
    lib().orc_sha256d_80(_u8(header), C.c_uint32(nonce), out)
    return bytes(out)


def blake2b(msg: bytes, outlen: int = 64) -> bytes:
    out = (C.c_uint8 * outlen)()
    lib().orc_blake2b(_u8(msg) if msg else None, C.c_uint64(len(msg)), outlen, out)
    return bytes(out)


def sia_blake2b_80(header: bytes, nonce: int) -> bytes:
    out = (C.c_uint8 * 32)()
    lib().orc_sia_blake2b_80(_u8(header), C.c_uint32(nonce), out)
    return bytes(out)


def ccminer_blake2b_80(header: bytes, nonce: int) -> bytes:
    out = (C.c_uint8 * 32)()
    lib().orc_ccminer_blake2b_80(_u8(header), C.c_uint32(nonce), out)
    return bytes(out)


def keccak(msg: bytes, rate: int, pad: int, outlen: int) -> bytes:
    out = (C.c_uint8 * outlen)()
    lib().orc_keccak(_u8(msg) if msg else None, C.c_uint64(len(msg)), rate, C.c_uint8(pad), outlen,
                     out)
    return bytes(out)


def _hits(fn, cap, *args):
    hits = (Hit * cap)()
    found = fn(*args, hits, cap)
    return int(found), [hits[i] for i in range(min(found, cap))]


def sha256d_search(header: bytes, start: int, count: int, target64: int, cap: int = 4096):
    return _hits(lib().orc_sha256d_search, cap, _u8(header), C.c_uint32(start), C.c_uint64(count),
                 C.c_uint64(target64))


def sia_search(header: bytes, start: int, count: int, target64: int, cap: int = 4096):
    return _hits(lib().orc_sia_search, cap, _u8(header), C.c_uint32(start), C.c_uint64(count),
                 C.c_uint64(target64))


def ethash_hash(dag, dag_seed, n_items, header: bytes, nonce: int):
    """dag: uint32 ndarray [n_items*32] or None (then items come from the counter generator)."""
    mix = (C.c_uint8 * 32)()
    fin = (C.c_uint8 * 32)()
    p = dag.ctypes.data_as(C.POINTER(C.c_uint32)) if dag is not None else None
    lib().orc_ethash_hash(p, C.c_uint64(dag_seed), C.c_uint32(n_items), _u8(header),
                          C.c_uint64(nonce), mix, fin)
    return bytes(mix), bytes(fin)


def ethash_search(dag, dag_seed, n_items, header: bytes, start: int, count: int, target64: int,
                  cap: int = 4096):
    p = dag.ctypes.data_as(C.POINTER(C.c_uint32)) if dag is not None else None
    return _hits(lib().orc_ethash_search, cap, p, C.c_uint64(dag_seed), C.c_uint32(n_items),
                 _u8(header), C.c_uint64(start), C.c_uint64(count), C.c_uint64(target64))


def ethash_make_cache(cache_items: int, seed: bytes):
    cache = np.empty(cache_items * 16, dtype=np.uint32)
    lib().orc_ethash_make_cache(C.c_uint32(cache_items), _u8(seed),
                                cache.ctypes.data_as(C.POINTER(C.c_uint32)))
    return cache


def ethash_light(cache, full_size: int, header: bytes, nonce: int):
    mix = (C.c_uint8 * 32)()
    fin = (C.c_uint8 * 32)()
    lib().orc_ethash_light(cache.ctypes.data_as(C.POINTER(C.c_uint32)),
                           C.c_uint32(cache.size // 16), C.c_uint64(full_size), _u8(header),
                           C.c_uint64(nonce), mix, fin)
    return bytes(mix), bytes(fin)


def num_threads() -> int:
    return lib().orc_num_threads()


def set_num_threads(n: int) -> None:
    lib().orc_set_num_threads(int(n))
