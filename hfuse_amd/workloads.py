"""Synthetic workloads of the benchmarked kernels at their benchmark shapes.

Shared by the benchmark and the split tuner: every tensor kernel gets a maker of independent
input/output sets (so repeated launches can rotate through more bytes than the 256 MB
memory-side cache holds) and its algorithmic byte count; the searches get a maker of argument
structs over seeded headers and a seeded synthetic DAG.  Everything is drawn from seeded
generators; nothing here reads a file.
"""
from __future__ import annotations

SEED = 0x48467573

TENSOR_KERNELS = ("im2col_kernel", "MaxPoolForward", "batch_norm_collect_statistics_kernel",
                  "upsample_nearest2d_out_frame", "upsample_bilinear2d_out_frame", "kernelHistogram1D")
SEARCH_KERNELS = ("ethash_search", "sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash", "blake2b_gpu_hash")


# Bytes the smaller read stream of a pair cycles through before a buffer set repeats.  It is the
# inputs alone that have to outgrow the 256 MB memory-side cache: the outputs are written with
# non-temporal stores and take no room there, so ten sets of a 25 MB input still read from cache.
MIN_READ_FOOTPRINT = 600 << 20


class TensorPair:
    """One tensor pair: `nsets` independent input/output sets so repeats miss the last-level cache."""

    def __init__(self, name, k1, k2, make_set, bytes1, bytes2, min_read_footprint=None):
        # Enough sets that even the smaller of the two read streams cycles through more bytes
        # than the 256 MB memory-side cache holds, so neither kernel re-reads cached inputs.
        # (At least three sets whatever the footprint asked for.)
        if min_read_footprint is None:
            min_read_footprint = MIN_READ_FOOTPRINT
        self.name, self.k1, self.k2 = name, k1, k2
        self.bytes1, self.bytes2 = bytes1, bytes2
        self.sets = []
        read_footprint = 0
        while read_footprint < min_read_footprint or len(self.sets) < 3:
            s = make_set(len(self.sets))
            self.sets.append(s)
            read_footprint += s["min_read"]
        self.args1 = [s["a1"] for s in self.sets]
        self.args2 = [s["a2"] for s in self.sets]
        from .launcher import Rotation
        self.rotation = Rotation()   # every timing call on this pair continues where the last one stopped

    def time(self, plan, mode, warmup, iters, grid_blocks=0):
        """Milliseconds of `iters` launches of `plan` in `mode` on this pair's rotating sets."""
        return plan.time(mode, self.args1, self.args2, warmup, iters, grid_blocks, rotation=self.rotation)


def rand(shape, seed, lo=-1.0, hi=1.0, dev="cuda"):
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    return torch.rand(shape, generator=g, device=dev, dtype=torch.float32) * (hi - lo) + lo


def randn(shape, seed, mean, std, dev="cuda"):
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    return torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std + mean


def kernel_workload(kname, variant=""):
    """-> (make(i) -> dict(keep, args, read_bytes), algorithmic bytes) for one tensor kernel at its benchmark shape."""
    import torch
    from . import launcher as H

    def nbytes(*ts):
        return sum(t.numel() * t.element_size() for t in ts)

    if kname == "im2col_kernel":
        def mk(i):
            x = rand((32, 64, 56, 56), SEED + 10 * i)
            col = torch.empty((32, 576, 3136), device="cuda")
            return dict(keep=(x, col), read_bytes=nbytes(x), args=H.im2col_args(x, col))
        return mk, 256901120
    if kname == "MaxPoolForward" and variant == "k2":   # benchmark config 3
        def mk(i):
            y = rand((16, 128, 64, 64), SEED + 10 * i + 5)
            val = torch.empty((16, 128, 32, 32), device="cuda")
            idx = torch.empty((16, 128, 32, 32), dtype=torch.int64, device="cuda")
            return dict(keep=(y, val, idx), read_bytes=nbytes(y),
                        args=H.maxpool_args(y, val, idx, (2, 2), (2, 2), (0, 0)))
        return mk, 58720256
    if kname == "MaxPoolForward":                        # benchmark config 1
        def mk(i):
            y = rand((32, 64, 112, 112), SEED + 10 * i + 1)
            val = torch.empty((32, 64, 56, 56), device="cuda")
            idx = torch.empty((32, 64, 56, 56), dtype=torch.int64, device="cuda")
            return dict(keep=(y, val, idx), read_bytes=nbytes(y),
                        args=H.maxpool_args(y, val, idx, (3, 3), (2, 2), (1, 1)))
        return mk, 179830784
    if kname == "batch_norm_collect_statistics_kernel":
        def mk(i):
            x = randn((32, 256, 28, 28), SEED + 10 * i + 2, 0.5, 2.0)
            mean = torch.empty(256, device="cuda")
            inv = torch.empty(256, device="cuda")
            return dict(keep=(x, mean, inv), read_bytes=nbytes(x), args=H.bn_stats_args(x, mean, inv, 1e-5, 0.0))
        return mk, 25692160
    if kname == "upsample_nearest2d_out_frame":
        def mk(i):
            u = rand((32, 64, 56, 56), SEED + 10 * i + 3)
            out = torch.empty((32, 64, 112, 112), device="cuda")
            return dict(keep=(u, out), read_bytes=nbytes(u), args=H.upsample_nearest_args(u, out))
        return mk, 128450560
    if kname == "upsample_bilinear2d_out_frame":
        def mk(i):
            u = rand((32, 64, 56, 56), SEED + 10 * i + 6)
            out = torch.empty((32, 64, 112, 112), device="cuda")
            return dict(keep=(u, out), read_bytes=nbytes(u), args=H.upsample_bilinear_args(u, out, False))
        return mk, 128450560
    if kname == "kernelHistogram1D":
        def mk(i):
            x = rand((1 << 26,), SEED + 10 * i + 4, 0.0, 1.0)
            hist = torch.zeros(1024, device="cuda")
            return dict(keep=(x, hist), read_bytes=nbytes(x), args=H.histc_args(x, hist, 1024, 0.0, 1.0))
        return mk, 268439552
    raise KeyError(kname)


def build_pair(name, k1, k2, v1="", v2=""):
    mk1, b1 = kernel_workload(k1, v1)
    mk2, b2 = kernel_workload(k2, v2)

    def mk(i):
        s1, s2 = mk1(i), mk2(i)
        return dict(keep=(s1["keep"], s2["keep"]), min_read=min(s1["read_bytes"], s2["read_bytes"]),
                    a1=s1["args"], a2=s2["args"])
    return TensorPair(name, k1, k2, mk, b1, b2)


BENCH_TENSOR_PAIRS = {
    "im2col_maxpool": ("im2col_kernel", "MaxPoolForward", "", ""),
    "bn_upsample": ("batch_norm_collect_statistics_kernel", "upsample_nearest2d_out_frame", "", ""),
    "histc_maxpool": ("kernelHistogram1D", "MaxPoolForward", "", "k2"),
}


def build_tensor_pairs(names):
    return {n: build_pair(n, *BENCH_TENSOR_PAIRS[n]) for n in names if n in BENCH_TENSOR_PAIRS}


def splitmix64_bytes(n: int, seed: int) -> bytes:
    """First n bytes of the SplitMix64 counter stream hf_fill_splitmix64 writes (word i = mix(seed + (i+1)*gamma))."""
    out = bytearray()
    mask = (1 << 64) - 1
    i = 0
    while len(out) < n:
        i += 1
        z = (seed + i * 0x9E3779B97F4A7C15) & mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        out += ((z ^ (z >> 31)) & mask).to_bytes(8, "little")
    return bytes(out[:n])


class SearchPair:
    """Two nonce searches with their constants uploaded: `fresh()` -> (results1, results2, args1, args2).

    The constants live in `self.constants` (a caller-owned set: bind it to a plan with
    `plan.bind_constants(pair.constants)` or pass it to `launch_native`); they are also written to the
    process-wide set, which the split tuner's own plans read, so one SearchPair at a time there.
    `grid` is the grid a native Ethash launch of 128-thread blocks needs for its nonce count (Ethash
    scans gridDim * blockDim nonces); a fused launch divides by Ethash's share of the block instead."""

    ETHASH_ITEMS = 1 << 25            # 4 GiB of 128-byte DAG items
    ETHASH_TARGET = (1 << 40) - 1     # 24 leading zero bits
    TARGET32 = (1 << 32) - 1          # 32 leading zero bits

    def __init__(self, k1: str, k2: str, log2_1: int, log2_2: int, dag_items: int = ETHASH_ITEMS):
        import torch
        from . import launcher as H
        self.k1, self.k2 = k1, k2
        self.nonces = (1 << log2_1, 1 << log2_2)
        self.headers = []
        self.dag_items = dag_items
        self._keep = []
        self.grid = 0
        self.constants = H.Constants()
        for pos, k in enumerate((k1, k2)):
            hdr = splitmix64_bytes(32 if k == "ethash_search" else 80, SEED + 100 + pos)
            self.headers.append(hdr)
            if k == "ethash_search":
                dag = torch.empty(dag_items * 32, dtype=torch.int32, device="cuda")
                H.fill_splitmix64(dag, SEED)
                torch.cuda.synchronize()
                H.ethash_set_constants(dag, dag_items, hdr, self.ETHASH_TARGET)
                self.constants.set_ethash(dag, dag_items, hdr, self.ETHASH_TARGET)
                self._keep.append(dag)
                if pos == 0:
                    self.grid = self.nonces[0] // 128
            elif k == "sha256d_gpu_hash_shared":
                H.sha256d_set_block(hdr, self.TARGET32)
                self.constants.set_sha256d(hdr, self.TARGET32)
            elif k == "sia_blake2b_gpu_hash":
                H.sia_blake2b_set_block(hdr)
                self.constants.set_sia_blake2b(hdr)
            elif k == "blake2b_gpu_hash":
                H.blake2b_set_block(hdr)
                self.constants.set_blake2b(hdr)
            else:
                raise KeyError(k)

    def _args(self, k, results, n):
        from . import launcher as H
        if k == "ethash_search":
            return H.ethash_args(results, 0)
        if k == "sha256d_gpu_hash_shared":
            return H.sha256d_args(results, n, 0)
        return H.blake2b_args(results, n, 0, self.TARGET32)

    def fresh(self):
        from . import launcher as H
        r1, r2 = H.new_search_results(), H.new_search_results()
        return r1, r2, self._args(self.k1, r1, self.nonces[0]), self._args(self.k2, r2, self.nonces[1])


class TensorTriple:
    """Three tensor kernels at their benchmark shapes with rotating buffer sets: `arg_sets[s][k]`."""

    def __init__(self, names, min_read_footprint=None):
        from .launcher import Rotation
        if min_read_footprint is None:
            min_read_footprint = MIN_READ_FOOTPRINT
        makers = [kernel_workload(k) for k in names]
        self.names = tuple(names)
        self.bytes = sum(b for _, b in makers)
        self.sets, read = [], 0
        while read < min_read_footprint or len(self.sets) < 3:
            made = [mk(len(self.sets)) for mk, _ in makers]
            self.sets.append(made)
            read += min(m["read_bytes"] for m in made)
        self.arg_sets = [[m["args"] for m in made] for made in self.sets]
        self.rotation = Rotation()

    def time(self, plan, mode, warmup, iters, grid_blocks=0):
        """Milliseconds of `iters` repetitions (mode 2: the three natives back to back, 3: the fused kernel)."""
        return plan.time_n(mode, self.arg_sets, warmup, iters, grid_blocks, rotation=self.rotation)


class SearchTriple:
    """ccminer-Blake2b + SHA-256d + Ethash (the reference's configs/crypt_four.yaml) over seeded headers and
    the seeded 4 GiB DAG: 2^log2[0] + 2^log2[1] + 2^log2[2] nonces.  Bind `constants` to the plan."""

    KERNELS = ("blake2b_gpu_hash", "sha256d_gpu_hash_shared", "ethash_search")

    def __init__(self, log2=(26, 26, 24), dag_items=SearchPair.ETHASH_ITEMS):
        from . import launcher as H
        self.log2 = tuple(log2)
        self._pair = SearchPair("ethash_search", "sha256d_gpu_hash_shared", log2[2], log2[1], dag_items)
        self.constants = self._pair.constants
        self.constants.set_blake2b(splitmix64_bytes(80, SEED + 102))
        self._results = [H.new_search_results() for _ in range(3)]
        self.args = [H.blake2b_args(self._results[0], 1 << log2[0], 0, SearchPair.TARGET32),
                     H.sha256d_args(self._results[1], 1 << log2[1], 0), H.ethash_args(self._results[2], 0)]

    def grid(self, ethash_threads: int) -> int:
        """Workgroups that make Ethash scan its 2^log2[2] nonces with `ethash_threads` threads a block."""
        return (1 << self.log2[2]) // ethash_threads

    def time(self, plan, mode, iters=1):
        plan.bind_constants(self.constants)
        q = plan.partition_n
        share = 128 if mode == 2 else q.hi[2] - q.lo[2]   # the native Ethash launch runs 128-thread blocks
        return plan.time_n(mode, [self.args], 0, iters, self.grid(share)) / iters
