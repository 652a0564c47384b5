"""ctypes binding of libhfuse_gfx950.so (the C-ABI in include/hfuse_gfx950.h).

There is no fallback: if the library has not been built, importing a symbol
from it raises.  Nothing in this package computes results on the CPU.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# HFUSE_LIB names another build of the same library (the timing-only take-apart builds of `make takeapart`)
LIB_PATH = os.environ.get("HFUSE_LIB") or os.path.join(_HERE, "libhfuse_gfx950.so")

HF_OK, HF_EINVAL, HF_EPARSE, HF_ENOTFOUND, HF_EUNSUPPORTED, HF_EHIP, HF_EIO, HF_ENOMEM = 0, -1, -2, -3, -4, -5, -6, -7
HF_BARRIER_NONE, HF_BARRIER_MATCHED, HF_BARRIER_SUBSET, HF_BARRIER_BLOCKIDX = 0, 1, 2, 3
HF_SPLIT_TABLE, HF_SPLIT_EXECTIME = -1, -2
HF_STREAM_EMPTY, HF_STREAM_READ, HF_STREAM_WRITE, HF_STREAM_READ_LINES, HF_STREAM_COPY_1_4 = 0, 1, 2, 3, 4
HF_STREAM_WRITE_STRIDED, HF_STREAM_WRITE_XCD = 5, 6
ABI_VERSION = 300          # what hf_version() of a matching library answers
HF_MAX_SEARCH_RESULTS = 64
HF_MAX_TENSORINFO_DIMS = 8

ERROR_NAMES = {HF_EINVAL: "HF_EINVAL", HF_EPARSE: "HF_EPARSE", HF_ENOTFOUND: "HF_ENOTFOUND",
               HF_EUNSUPPORTED: "HF_EUNSUPPORTED", HF_EHIP: "HF_EHIP", HF_EIO: "HF_EIO", HF_ENOMEM: "HF_ENOMEM"}


class HfuseError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")
        self.code = code
        self.message = message


class Dim3(C.Structure):
    _fields_ = [("x", C.c_uint32), ("y", C.c_uint32), ("z", C.c_uint32)]


class KernelInfo(C.Structure):
    _fields_ = [("kernel_name", C.c_char * 96), ("has_barriers", C.c_int), ("block_dim", Dim3),
                ("reg", C.c_uint32), ("exec_time", C.c_double), ("native_threads", C.c_uint32)]


class Partition(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("lo", C.c_uint32 * 2), ("hi", C.c_uint32 * 2),
                ("block_dim", Dim3 * 2), ("launch_threads", C.c_uint32),
                ("launch_blocks", C.c_uint32), ("barrier_mode", C.c_int)]


HF_MAX_FUSE = 4


class PartitionN(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("n", C.c_int), ("lo", C.c_uint32 * HF_MAX_FUSE), ("hi", C.c_uint32 * HF_MAX_FUSE),
                ("block_dim", Dim3 * HF_MAX_FUSE), ("launch_threads", C.c_uint32), ("launch_blocks", C.c_uint32),
                ("barrier_mode", C.c_int)]


class Im2colArgs(C.Structure):
    _fields_ = [("n", C.c_int64), ("data_im", C.c_void_p)] + \
               [(k, C.c_int64) for k in ("height", "width", "kernel_h", "kernel_w", "pad_h", "pad_w",
                                         "stride_h", "stride_w", "dilation_h", "dilation_w",
                                         "height_col", "width_col")] + [("data_col", C.c_void_p)]


class MaxPoolArgs(C.Structure):
    _fields_ = [("nthreads", C.c_int), ("bottom_data", C.c_void_p)] + \
               [(k, C.c_int) for k in ("num", "channels", "height", "width", "pooled_height",
                                       "pooled_width", "kernel_h", "kernel_w", "stride_h", "stride_w",
                                       "pad_h", "pad_w", "dilation_h", "dilation_w")] + \
               [("top_data", C.c_void_p), ("top_mask", C.c_void_p)]


class Accessor3(C.Structure):
    _fields_ = [("data", C.c_void_p), ("sizes", C.c_int * 3), ("strides", C.c_int * 3)]


class Accessor1(C.Structure):
    _fields_ = [("data", C.c_void_p), ("sizes", C.c_int * 1), ("strides", C.c_int * 1)]


class BnStatsArgs(C.Structure):
    _fields_ = [("input", Accessor3), ("epsilon", C.c_float), ("momentum", C.c_float),
                ("running_mean", Accessor1), ("running_var", Accessor1), ("save_mean", Accessor1),
                ("save_transformed_var", Accessor1)]


class UpsampleNearestArgs(C.Structure):
    _fields_ = [("idata", C.c_void_p), ("odata", C.c_void_p), ("nc", C.c_size_t),
                ("height1", C.c_size_t), ("width1", C.c_size_t), ("height2", C.c_size_t),
                ("width2", C.c_size_t), ("height_scale", C.c_float), ("width_scale", C.c_float)]


class Accessor4(C.Structure):
    _fields_ = [("data", C.c_void_p), ("sizes", C.c_int64 * 4), ("strides", C.c_int64 * 4)]


class UpsampleBilinearArgs(C.Structure):
    _fields_ = [("n", C.c_int), ("rheight", C.c_float), ("rwidth", C.c_float), ("align_corners", C.c_int),
                ("idata", Accessor4), ("odata", Accessor4)]


class TensorInfo(C.Structure):
    _fields_ = [("data", C.c_void_p), ("sizes", C.c_int64 * HF_MAX_TENSORINFO_DIMS),
                ("strides", C.c_int64 * HF_MAX_TENSORINFO_DIMS), ("dims", C.c_int)]


class HistcArgs(C.Structure):
    _fields_ = [("a", TensorInfo), ("p", TensorInfo), ("b", TensorInfo), ("nbins", C.c_int),
                ("minvalue", C.c_float), ("maxvalue", C.c_float), ("total_elements", C.c_int64),
                ("get_op", C.c_void_p)]


class SearchHit(C.Structure):
    _fields_ = [("nonce", C.c_uint64), ("digest", C.c_uint32 * 8), ("mix", C.c_uint32 * 8)]


class SearchResults(C.Structure):
    _fields_ = [("count", C.c_uint32), ("pad", C.c_uint32), ("hit", SearchHit * HF_MAX_SEARCH_RESULTS)]


class EthashArgs(C.Structure):
    _fields_ = [("g_output", C.c_void_p), ("start_nonce", C.c_uint64)]


class Sha256dArgs(C.Structure):
    _fields_ = [("threads", C.c_uint32), ("start_nonce", C.c_uint32), ("res_nonces", C.c_void_p)]


class Blake2bArgs(C.Structure):
    _fields_ = [("threads", C.c_uint32), ("start_nonce", C.c_uint32), ("res_nonce", C.c_void_p),
                ("target2", C.c_uint32 * 2)]


# every symbol include/hfuse_gfx950.h declares, with its prototype
PROTOTYPES = {
    "hf_last_error": (C.c_char_p, []),
    "hf_version": (C.c_int, []),
    "hf_config_load_text": (C.c_int, [C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]),
    "hf_config_load_files": (C.c_int, [C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]),
    "hf_config_free": (None, [C.c_void_p]),
    "hf_config_num_fusions": (C.c_int, [C.c_void_p]),
    "hf_config_num_kernels": (C.c_int, [C.c_void_p]),
    "hf_config_fusion": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p),
                                   C.POINTER(C.c_char_p)]),
    "hf_config_fusion_size": (C.c_int, [C.c_void_p, C.c_int]),
    "hf_config_fusion_kernel": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_char_p)]),
    "hf_config_kernel": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(KernelInfo)]),
    "hf_plan_create": (C.c_int, [C.c_void_p, C.c_int, C.c_char_p, C.c_int, C.c_int, C.POINTER(C.c_void_p)]),
    "hf_plan_free": (None, [C.c_void_p]),
    "hf_plan_set_barrier_mode": (C.c_int, [C.c_void_p, C.c_int]),
    "hf_plan_set_grids": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "hf_plan_set_lending": (C.c_int, [C.c_void_p, C.c_int]),
    "hf_plan_set_launch_bound": (C.c_int, [C.c_void_p, C.c_int]),
    "hf_plan_set_launch_waves": (C.c_int, [C.c_void_p, C.c_int]),
    "hf_plan_launch_waves": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "hf_plan_set_block": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "hf_plan_partition": (C.c_int, [C.c_void_p, C.POINTER(Partition)]),
    "hf_plan_num_kernels": (C.c_int, [C.c_void_p]),
    "hf_plan_partition_n": (C.c_int, [C.c_void_p, C.POINTER(PartitionN)]),
    "hf_plan_set_block_n": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.c_int]),
    "hf_launch_fused_n": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_void_p]),
    "hf_time_fused_n": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                  C.c_int, C.c_void_p, C.POINTER(C.c_float)]),
    "hf_plan_num_splits": (C.c_int, [C.c_void_p, C.c_int]),
    "hf_plan_local_index": (C.c_int, [C.c_void_p, C.c_int, C.c_uint32, C.POINTER(Dim3)]),
    "hf_ethash_set_constants": (C.c_int, [C.c_void_p, C.c_uint32, C.c_char_p, C.c_uint64, C.c_void_p]),
    "hf_sha256d_set_block": (C.c_int, [C.c_char_p, C.c_uint64, C.c_void_p]),
    "hf_sia_blake2b_set_block": (C.c_int, [C.c_char_p, C.c_void_p]),
    "hf_blake2b_set_block": (C.c_int, [C.c_char_p, C.c_void_p]),
    "hf_constants_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "hf_constants_free": (None, [C.c_void_p]),
    "hf_constants_set_ethash": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_char_p, C.c_uint64]),
    "hf_constants_set_sha256d": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64]),
    "hf_constants_set_sia_blake2b": (C.c_int, [C.c_void_p, C.c_char_p]),
    "hf_constants_set_blake2b": (C.c_int, [C.c_void_p, C.c_char_p]),
    "hf_plan_bind_constants": (C.c_int, [C.c_void_p, C.c_void_p]),
    "hf_launch_native": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "hf_launch_native_with": (C.c_int, [C.c_char_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]),
    "hf_launch_fused": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]),
    "hf_time_pair": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_int, C.c_int,
                               C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_float)]),
    "hf_fill_splitmix64": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_void_p]),
    "hf_copy_f32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p]),
    "hf_stream_probe": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p]),
    "hf_time_stream_probe": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_int,
                                       C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_float)]),
}

_lib = None


def lib() -> C.CDLL:
    """Load the built library; raise if it is missing (there is no CPU path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(or `make -C hfuse_amd/csrc`). hfuse_amd has no CPU fallback.")
        handle = C.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        # signatures changed between versions (hf_time_pair gained an argument): a stale build would take shifted arguments
        if handle.hf_version() != ABI_VERSION:
            raise ImportError(f"{LIB_PATH} answers hf_version() = {handle.hf_version()}, this package binds version "
                              f"{ABI_VERSION}: rebuild it (`make -C hfuse_amd/csrc`)")
        _lib = handle
    return _lib


def check(rc: int) -> int:
    if rc < 0:
        raise HfuseError(rc, lib().hf_last_error().decode())
    return rc
