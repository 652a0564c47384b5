"""Host-side mirror of the reference's interface over the C-ABI.

`Config` is the pair of YAML files of the reference's CLI
(tools/llvm-smart-fuser/main.cpp:263-270), `Plan` one fused variant
(pair x preset x split, main.cpp:215-227), and the `*_args` builders fill each
original kernel's argument list from torch tensors (torch is only the owner of
device memory and streams here).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

from . import _lib as L
from ._lib import HfuseError, check  # noqa: F401


def _stream_ptr(stream=None):
    if stream is None:
        import torch
        stream = torch.cuda.current_stream()
    return C.c_void_p(getattr(stream, "cuda_stream", stream))


class Config:
    """Fusion list + kernel table."""

    def __init__(self, fusion_yaml: Optional[str], kernels_yaml: str):
        self._h = C.c_void_p()
        check(L.lib().hf_config_load_text(fusion_yaml.encode() if fusion_yaml is not None else None,
                                          kernels_yaml.encode() if kernels_yaml is not None else None,
                                          C.byref(self._h)))

    @classmethod
    def from_files(cls, fusion_path: Optional[str], kernels_path: str) -> "Config":
        self = cls.__new__(cls)
        self._h = C.c_void_p()
        check(L.lib().hf_config_load_files(fusion_path.encode() if fusion_path else None,
                                           kernels_path.encode(), C.byref(self._h)))
        return self

    def __del__(self):
        if getattr(self, "_h", None) and L is not None and L._lib is not None:
            L._lib.hf_config_free(self._h)
            self._h = None

    @property
    def num_fusions(self) -> int:
        return check(L.lib().hf_config_num_fusions(self._h))

    @property
    def num_kernels(self) -> int:
        return check(L.lib().hf_config_num_kernels(self._h))

    def fusion(self, i: int):
        f, k1, k2 = C.c_char_p(), C.c_char_p(), C.c_char_p()
        check(L.lib().hf_config_fusion(self._h, i, C.byref(f), C.byref(k1), C.byref(k2)))
        return f.value.decode(), k1.value.decode(), k2.value.decode()

    def fusions(self):
        return [self.fusion(i) for i in range(self.num_fusions)]

    def fusion_kernels(self, i: int):
        """All kernel names of entry i (the schema allows any number; plans exist for pairs)."""
        n = check(L.lib().hf_config_fusion_size(self._h, i))
        out = []
        for k in range(n):
            name = C.c_char_p()
            check(L.lib().hf_config_fusion_kernel(self._h, i, k, C.byref(name)))
            out.append(name.value.decode())
        return out

    def find_fusion_n(self, *kernels: str) -> int:
        """Index of the entry that lists exactly these kernels in this order (any number of them)."""
        for i in range(self.num_fusions):
            if self.fusion_kernels(i) == list(kernels):
                return i
        raise KeyError(f"no fusion of {' + '.join(kernels)} in the fusion list")

    def find_fusion(self, k1: str, k2: str) -> int:
        for i, (_, a, b) in enumerate(self.fusions()):
            if (a, b) == (k1, k2) and check(L.lib().hf_config_fusion_size(self._h, i)) == 2:
                return i
        raise KeyError(f"no fusion of {k1} + {k2} in the fusion list")

    def kernel(self, name: str) -> L.KernelInfo:
        out = L.KernelInfo()
        check(L.lib().hf_config_kernel(self._h, name.encode(), C.byref(out)))
        return out

    def num_splits(self, fusion_index: int) -> int:
        return check(L.lib().hf_plan_num_splits(self._h, fusion_index))

    def plan(self, fusion_index: int, preset: str = "hfuse", split_idx: int = L.HF_SPLIT_TABLE,
             split_threads: int = 0) -> "Plan":
        return Plan(self, fusion_index, preset, split_idx, split_threads)


class Plan:
    """One fused variant of one pair."""

    def __init__(self, cfg: Config, fusion_index: int, preset: str, split_idx: int, split_threads: int):
        self._h = C.c_void_p()
        self._cfg = cfg  # keep the config alive
        check(L.lib().hf_plan_create(cfg._h, fusion_index, preset.encode(), split_idx, split_threads,
                                     C.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None) and L is not None and L._lib is not None:
            L._lib.hf_plan_free(self._h)
            self._h = None

    @property
    def partition(self) -> L.Partition:
        out = L.Partition()
        check(L.lib().hf_plan_partition(self._h, C.byref(out)))
        return out

    @property
    def name(self) -> str:
        return self.partition.name.decode()

    @property
    def num_kernels(self) -> int:
        return check(L.lib().hf_plan_num_kernels(self._h))

    @property
    def partition_n(self) -> L.PartitionN:
        out = L.PartitionN()
        check(L.lib().hf_plan_partition_n(self._h, C.byref(out)))
        return out

    def set_block_n(self, *threads: int) -> None:
        arr = (C.c_int * len(threads))(*threads)
        check(L.lib().hf_plan_set_block_n(self._h, arr, len(threads)))

    def launch_n(self, args: Sequence, grid_blocks: int = 0, stream=None) -> None:
        """Fused launch of a plan of len(args) kernels, argument lists in YAML order."""
        ptrs = (C.c_void_p * len(args))(*[C.addressof(a) for a in args])
        check(L.lib().hf_launch_fused_n(self._h, ptrs, len(args), grid_blocks, _stream_ptr(stream)))

    def time_n(self, mode: int, arg_sets: Sequence[Sequence], warmup: int, iters: int, grid_blocks: int = 0,
               stream=None, rotation: Optional["Rotation"] = None) -> float:
        """Milliseconds for `iters` repetitions of a three-kernel plan (mode 2 natives back to back, 3 fused);
        arg_sets[s][k] is kernel k's argument list of buffer set s."""
        nsets, n = len(arg_sets), len(arg_sets[0])
        flat = [C.addressof(a) for s in arg_sets for a in s]
        ptrs = (C.c_void_p * len(flat))(*flat)
        ms = C.c_float()
        first = rotation.take(nsets, warmup + iters) if rotation is not None else 0
        check(L.lib().hf_time_fused_n(self._h, mode, ptrs, n, nsets, first, warmup, iters, grid_blocks,
                                      _stream_ptr(stream), C.byref(ms)))
        return ms.value

    def set_barrier_mode(self, mode: int) -> None:
        check(L.lib().hf_plan_set_barrier_mode(self._h, mode))

    def set_grids(self, grid1: int = 0, grid2: int = 0) -> None:
        check(L.lib().hf_plan_set_grids(self._h, grid1, grid2))

    def set_block(self, threads1: int, threads2: int) -> None:
        check(L.lib().hf_plan_set_block(self._h, threads1, threads2))

    def set_lending(self, on: bool) -> None:
        check(L.lib().hf_plan_set_lending(self._h, int(on)))

    def set_launch_bound(self, on) -> None:
        """True / False: run the register-bounded / the plain build; None: by the preset."""
        check(L.lib().hf_plan_set_launch_bound(self._h, -1 if on is None else int(bool(on))))

    def set_launch_waves(self, waves: int) -> None:
        """Ask for the register-bounded build at `waves` waves per SIMD (1..8); 0: the occupancy formula's value."""
        check(L.lib().hf_plan_set_launch_waves(self._h, waves))

    @property
    def launch_waves(self):
        """(waves per SIMD the occupancy formula gives, bound of the build a launch runs now; 0 = plain)."""
        f, b = C.c_int(), C.c_int()
        check(L.lib().hf_plan_launch_waves(self._h, C.byref(f), C.byref(b)))
        return f.value, b.value

    def bind_constants(self, constants: Optional["Constants"]) -> None:
        """Fused launches of this plan use a copy of `constants` instead of the process-wide set (None unbinds).

        The copy is a snapshot taken now (later changes of `constants` do not reach the plan) and holds the raw
        device pointer of the Ethash DAG, so the plan keeps `constants` -- and through it the DAG tensor -- alive."""
        check(L.lib().hf_plan_bind_constants(self._h, constants._h if constants is not None else None))
        self._consts = constants

    def local_index(self, half: int, tid: int):
        out = L.Dim3()
        check(L.lib().hf_plan_local_index(self._h, half, tid, C.byref(out)))
        return out.x, out.y, out.z

    def launch(self, args1, args2, grid_blocks: int = 0, stream=None) -> None:
        check(L.lib().hf_launch_fused(self._h, C.byref(args1), C.byref(args2), grid_blocks,
                                      _stream_ptr(stream)))

    def time(self, mode: int, args1: Sequence, args2: Sequence, warmup: int, iters: int,
             grid_blocks: int = 0, stream=None, rotation: Optional["Rotation"] = None) -> float:
        """Milliseconds for `iters` repetitions (mode 0/1 native, 2 back-to-back, 3 fused, 4 two streams).

        With a `rotation` the call starts at the buffer set after the last one any earlier call used
        and moves the cursor on, so short calls keep cycling through all sets."""
        n = len(args1)
        assert n == len(args2) and n > 0
        a1 = (C.c_void_p * n)(*[C.addressof(a) for a in args1])
        a2 = (C.c_void_p * n)(*[C.addressof(a) for a in args2])
        ms = C.c_float()
        first = rotation.take(n, warmup + iters) if rotation is not None else 0
        check(L.lib().hf_time_pair(self._h, mode, a1, a2, n, first, warmup, iters, grid_blocks,
                                   _stream_ptr(stream), C.byref(ms)))
        return ms.value


class Rotation:
    """Cursor over the buffer sets of a workload, shared by every timing call on them."""

    def __init__(self):
        self.cursor = 0

    def take(self, nsets: int, launches: int) -> int:
        first = self.cursor % nsets
        self.cursor = (first + launches) % nsets
        return first


def launch_native(kernel_name: str, args, grid_blocks: int = 0, block_threads: int = 0, stream=None,
                  constants: Optional["Constants"] = None) -> None:
    if constants is not None:
        check(L.lib().hf_launch_native_with(kernel_name.encode(), C.byref(args), constants._h, grid_blocks,
                                            block_threads, _stream_ptr(stream)))
        return
    check(L.lib().hf_launch_native(kernel_name.encode(), C.byref(args), grid_blocks, block_threads,
                                   _stream_ptr(stream)))


class Constants:
    """A caller-owned set of the search kernels' constants (DAG, headers, targets): one per host thread or job."""

    def __init__(self):
        self._h = C.c_void_p()
        self._keep = []
        check(L.lib().hf_constants_create(C.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None) and L is not None and L._lib is not None:
            L._lib.hf_constants_free(self._h)
            self._h = None

    def set_ethash(self, dag, dag_items: int, header: bytes, target: int) -> "Constants":
        assert len(header) == 32
        self._keep = [dag]
        check(L.lib().hf_constants_set_ethash(self._h, C.c_void_p(dag.data_ptr()), dag_items, header, target))
        return self

    def set_sha256d(self, header: bytes, target64: int) -> "Constants":
        assert len(header) == 80
        check(L.lib().hf_constants_set_sha256d(self._h, header, target64))
        return self

    def set_sia_blake2b(self, header: bytes) -> "Constants":
        assert len(header) == 80
        check(L.lib().hf_constants_set_sia_blake2b(self._h, header))
        return self

    def set_blake2b(self, header: bytes) -> "Constants":
        assert len(header) == 80
        check(L.lib().hf_constants_set_blake2b(self._h, header))
        return self


# ------------------------------------------------------------ argument builders
def im2col_args(x, out, kernel=(3, 3), pad=(1, 1), stride=(1, 1), dilation=(1, 1)) -> L.Im2colArgs:
    """x: [..., H, W] contiguous float32 (leading dims are folded into channels);
    out: [..., C*kh*kw, Hc*Wc] float32."""
    h, w = x.shape[-2], x.shape[-1]
    channels = x.numel() // (h * w)
    hc = (h + 2 * pad[0] - (dilation[0] * (kernel[0] - 1) + 1)) // stride[0] + 1
    wc = (w + 2 * pad[1] - (dilation[1] * (kernel[1] - 1) + 1)) // stride[1] + 1
    a = L.Im2colArgs()
    a.n = channels * hc * wc
    a.data_im = x.data_ptr()
    a.height, a.width = h, w
    a.kernel_h, a.kernel_w = kernel
    a.pad_h, a.pad_w = pad
    a.stride_h, a.stride_w = stride
    a.dilation_h, a.dilation_w = dilation
    a.height_col, a.width_col = hc, wc
    a.data_col = out.data_ptr()
    return a


def maxpool_args(x, out, mask, kernel, stride, pad, dilation=(1, 1)) -> L.MaxPoolArgs:
    n, c, h, w = x.shape
    ph, pw = out.shape[-2], out.shape[-1]
    a = L.MaxPoolArgs()
    a.nthreads = out.numel()
    a.bottom_data = x.data_ptr()
    a.num, a.channels, a.height, a.width = n, c, h, w
    a.pooled_height, a.pooled_width = ph, pw
    a.kernel_h, a.kernel_w = kernel
    a.stride_h, a.stride_w = stride
    a.pad_h, a.pad_w = pad
    a.dilation_h, a.dilation_w = dilation
    a.top_data = out.data_ptr()
    a.top_mask = mask.data_ptr()
    return a


def bn_stats_args(x, mean, invstd, eps=1e-5, momentum=0.0) -> L.BnStatsArgs:
    """x: [N, C, ...] float32 viewed as [N, C, L]; mean/invstd: [C] float32."""
    n, c = x.shape[0], x.shape[1]
    l = x.numel() // (n * c)
    x3 = x.reshape(n, c, l)
    a = L.BnStatsArgs()
    a.input.data = x3.data_ptr()
    a.input.sizes[:] = [n, c, l]
    a.input.strides[:] = list(x3.stride())
    a.epsilon = eps
    a.momentum = momentum
    for acc, t in ((a.save_mean, mean), (a.save_transformed_var, invstd)):
        acc.data = t.data_ptr()
        acc.sizes[0] = t.shape[0]
        acc.strides[0] = t.stride(0)
    return a


def upsample_nearest_args(x, out, scales=None) -> L.UpsampleNearestArgs:
    n, c, h1, w1 = x.shape
    h2, w2 = out.shape[-2], out.shape[-1]
    a = L.UpsampleNearestArgs()
    a.idata, a.odata = x.data_ptr(), out.data_ptr()
    a.nc, a.height1, a.width1, a.height2, a.width2 = n * c, h1, w1, h2, w2
    import numpy as np
    a.height_scale = float(np.float32(scales[0])) if scales else float(np.float32(h1) / np.float32(h2))
    a.width_scale = float(np.float32(scales[1])) if scales else float(np.float32(w1) / np.float32(w2))
    return a


def upsample_bilinear_args(x, out, align_corners=False, scales=None) -> L.UpsampleBilinearArgs:
    """x [N,C,H1,W1], out [N,C,H2,W2] float32 (any strides); scales as PyTorch's area_pixel_compute_scale."""
    import numpy as np
    h1, w1 = x.shape[-2], x.shape[-1]
    h2, w2 = out.shape[-2], out.shape[-1]
    a = L.UpsampleBilinearArgs()
    a.n = h2 * w2
    if scales:
        rh, rw = np.float32(scales[0]), np.float32(scales[1])
    elif align_corners:
        rh = np.float32(h1 - 1) / np.float32(h2 - 1) if h2 > 1 else np.float32(0)
        rw = np.float32(w1 - 1) / np.float32(w2 - 1) if w2 > 1 else np.float32(0)
    else:
        rh, rw = np.float32(h1) / np.float32(h2), np.float32(w1) / np.float32(w2)
    a.rheight, a.rwidth, a.align_corners = float(rh), float(rw), int(align_corners)
    for acc, t in ((a.idata, x), (a.odata, out)):
        acc.data = t.data_ptr()
        acc.sizes[:] = list(t.shape)
        acc.strides[:] = list(t.stride())
    return a


def histc_args(x, out, nbins, lo, hi) -> L.HistcArgs:
    a = L.HistcArgs()
    flat = x.reshape(-1)
    a.a.data, a.a.dims = out.data_ptr(), 1
    a.a.sizes[0], a.a.strides[0] = out.shape[0], out.stride(0)
    a.b.data, a.b.dims = flat.data_ptr(), 1
    a.b.sizes[0], a.b.strides[0] = flat.shape[0], flat.stride(0) if flat.numel() > 1 else 1
    a.p.data, a.p.dims = None, 0
    a.nbins, a.minvalue, a.maxvalue = nbins, lo, hi
    a.total_elements = flat.numel()
    a.get_op = None
    return a


# ------------------------------------------------------------ searches
def new_search_results(device="cuda"):
    """Zeroed device buffer holding one hf_search_results."""
    import torch
    return torch.zeros(C.sizeof(L.SearchResults), dtype=torch.uint8, device=device)


def read_search_results(buf):
    """-> (total_found, hits sorted by nonce as (nonce, digest_bytes, mix_bytes))."""
    raw = bytes(buf.cpu().numpy().tobytes())
    res = L.SearchResults.from_buffer_copy(raw)
    hits = [(h.nonce, bytes(h.digest), bytes(h.mix)) for h in res.hit[: min(res.count, L.HF_MAX_SEARCH_RESULTS)]]
    return int(res.count), sorted(hits)


def ethash_args(results, start_nonce: int) -> L.EthashArgs:
    a = L.EthashArgs()
    a.g_output = results.data_ptr()
    a.start_nonce = start_nonce
    return a


def sha256d_args(results, threads: int, start_nonce: int) -> L.Sha256dArgs:
    a = L.Sha256dArgs()
    a.threads, a.start_nonce, a.res_nonces = threads, start_nonce, results.data_ptr()
    return a


def blake2b_args(results, threads: int, start_nonce: int, target64: int) -> L.Blake2bArgs:
    a = L.Blake2bArgs()
    a.threads, a.start_nonce, a.res_nonce = threads, start_nonce, results.data_ptr()
    a.target2[0], a.target2[1] = target64 & 0xFFFFFFFF, target64 >> 32
    return a


def ethash_set_constants(dag, dag_items: int, header: bytes, target: int) -> None:
    assert len(header) == 32
    check(L.lib().hf_ethash_set_constants(C.c_void_p(dag.data_ptr()), dag_items, header, target, None))


def sha256d_set_block(header: bytes, target64: int) -> None:
    assert len(header) == 80
    check(L.lib().hf_sha256d_set_block(header, target64, None))


def sia_blake2b_set_block(header: bytes) -> None:
    assert len(header) == 80
    check(L.lib().hf_sia_blake2b_set_block(header, None))


def blake2b_set_block(header: bytes) -> None:
    assert len(header) == 80
    check(L.lib().hf_blake2b_set_block(header, None))


def fill_splitmix64(t, seed: int, stream=None) -> None:
    """Fill a device tensor (byte size a multiple of 8) with the counter generator."""
    nbytes = t.numel() * t.element_size()
    assert nbytes % 8 == 0
    check(L.lib().hf_fill_splitmix64(C.c_void_p(t.data_ptr()), nbytes // 8, seed, _stream_ptr(stream)))


def copy_f32(src, dst, stream=None) -> None:
    check(L.lib().hf_copy_f32(C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), src.numel(),
                              _stream_ptr(stream)))
