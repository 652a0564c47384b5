"""The argument structs of the C-ABI against the only place the reference pins the original
kernels' argument lists: the kernel-name column of its nvprof traces, kept as the fixture
tests/golden/ref_signatures.json (made by tests/golden/make_ref_signatures.py)."""
import ctypes as C
import json
import os

import pytest

from hfuse_amd import _lib as L

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_signatures.json")

STRUCTS = {
    "im2col_kernel": L.Im2colArgs,
    "MaxPoolForward": L.MaxPoolArgs,
    "batch_norm_collect_statistics_kernel": L.BnStatsArgs,
    "kernelHistogram1D": L.HistcArgs,
    "upsample_bilinear2d_out_frame": L.UpsampleBilinearArgs,
    "ethash_search": L.EthashArgs,
    "sha256d_gpu_hash_shared": L.Sha256dArgs,
    "blake2b_gpu_hash": L.Blake2bArgs,
    "sia_blake2b_gpu_hash": L.Blake2bArgs,
}


def field_class(ctype):
    if ctype is C.c_void_p:
        return "ptr"
    if isinstance(ctype, type) and issubclass(ctype, C.Structure):
        return "opaque"
    if isinstance(ctype, type) and issubclass(ctype, C.Array):
        return "uint2" if ctype._length_ == 2 and ctype._type_ is C.c_uint32 else "opaque"
    return "scalar"


@pytest.mark.parametrize("kernel", sorted(STRUCTS))
def test_argument_struct_follows_the_traced_signature(kernel):
    ref = json.load(open(FIXTURE))[kernel]
    fields = STRUCTS[kernel]._fields_
    assert len(fields) == ref["arity"], f"{kernel}: {len(fields)} fields, reference lists {ref['arity']} ({ref['source']})"
    for i, ((name, ctype), want) in enumerate(zip(fields, ref["params"])):
        if want == "opaque":
            continue  # accessor / TensorInfo struct, functor, or a position nvprof garbled
        got = field_class(ctype)
        assert got == want, f"{kernel} parameter {i} ({name}): {got}, reference has {want}"


def test_fused_argument_order_is_kernel1_then_kernel2():
    """The traced fused kernels list K1's parameters, then K2's (KernelPrinter.cpp:107-115):
    e.g. sia_blake2b_gpu_hash_ethash_search4_0(uint, uint, uint*, uint2, Search_results*, ulong)."""
    ref = json.load(open(FIXTURE))
    sia, eth = ref["sia_blake2b_gpu_hash"], ref["ethash_search"]
    assert sia["params"] + eth["params"] == ["scalar", "scalar", "ptr", "uint2", "ptr", "scalar"]
    assert [field_class(t) for _, t in L.Blake2bArgs._fields_] + [field_class(t) for _, t in L.EthashArgs._fields_] == \
        sia["params"] + eth["params"]
