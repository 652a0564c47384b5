"""Random and mutated argument structs through hf_launch_native on a machine WITHOUT a GPU.

Every validator has to refuse or accept without crashing (a wrapped product once divided by
zero).  Accepted structs reach a launch that fails for want of a device, so this file must never
run where a GPU is visible: there the same calls would launch kernels on made-up pointers."""
import os
import subprocess
import sys
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = textwrap.dedent("""
    import ctypes as C, random, sys
    sys.path.insert(0, %r)
    import torch
    assert not torch.cuda.is_available()
    from hfuse_amd import _lib as L
    lib = L.lib()
    rng = random.Random(777)
    VALS = [0, 1, 2, 3, 4, 7, 8, 16, 56, 64, 112, 256, 1024, 65536, -1, -2, 2**31 - 1, 2**31, 2**32, 2**63 - 1,
            -2**63, 2**40, 3136, 576]
    buf = (C.c_float * 65536)()
    base = C.addressof(buf)
    hdr = bytes([1, 2, 3]) + bytes(77)
    lib.hf_sha256d_set_block(hdr, 1, None); lib.hf_sia_blake2b_set_block(hdr, None); lib.hf_blake2b_set_block(hdr, None)
    lib.hf_ethash_set_constants(base, 128, hdr, 1, None)

    def valid():
        im = L.Im2colArgs(); im.n = 256; im.data_im = im.data_col = base; im.height = im.width = 8
        im.kernel_h = im.kernel_w = 3; im.pad_h = im.pad_w = im.stride_h = im.stride_w = im.dilation_h = im.dilation_w = 1
        im.height_col = im.width_col = 8
        mp = L.MaxPoolArgs(); mp.nthreads = 96; mp.bottom_data = mp.top_data = mp.top_mask = base; mp.num = 2; mp.channels = 3
        mp.height = mp.width = 8; mp.pooled_height = mp.pooled_width = 4; mp.kernel_h = mp.kernel_w = 3
        mp.stride_h = mp.stride_w = 2; mp.pad_h = mp.pad_w = 1; mp.dilation_h = mp.dilation_w = 1
        bn = L.BnStatsArgs(); bn.input.data = base; bn.input.sizes[:] = [4, 8, 16]; bn.input.strides[:] = [128, 16, 1]
        for t in (bn.save_mean, bn.save_transformed_var):
            t.data = base; t.sizes[0] = 8; t.strides[0] = 1
        up = L.UpsampleNearestArgs(); up.idata = up.odata = base; up.nc = 6; up.height1 = up.width1 = 8
        up.height2 = up.width2 = 16; up.height_scale = up.width_scale = 0.5
        bl = L.UpsampleBilinearArgs(); bl.n = 256; bl.rheight = bl.rwidth = 0.5; bl.idata.data = bl.odata.data = base
        bl.idata.sizes[:] = [2, 3, 8, 8]; bl.idata.strides[:] = [192, 64, 8, 1]
        bl.odata.sizes[:] = [2, 3, 16, 16]; bl.odata.strides[:] = [768, 256, 16, 1]
        hi = L.HistcArgs(); hi.a.data = hi.b.data = base; hi.a.dims = hi.b.dims = 1; hi.a.sizes[0] = 16; hi.a.strides[0] = 1
        hi.b.sizes[0] = 4096; hi.b.strides[0] = 1; hi.nbins = 16; hi.minvalue = 0.0; hi.maxvalue = 1.0; hi.total_elements = 4096
        sh = L.Sha256dArgs(); sh.threads = 64; sh.res_nonces = base
        b2 = L.Blake2bArgs(); b2.threads = 64; b2.res_nonce = base
        et = L.EthashArgs(); et.g_output = base
        return [(b"im2col_kernel", im), (b"MaxPoolForward", mp), (b"batch_norm_collect_statistics_kernel", bn),
                (b"upsample_nearest2d_out_frame", up), (b"upsample_bilinear2d_out_frame", bl), (b"kernelHistogram1D", hi),
                (b"sha256d_gpu_hash_shared", sh), (b"sia_blake2b_gpu_hash", b2), (b"blake2b_gpu_hash", b2), (b"ethash_search", et)]

    def poke(a, slots):
        raw = (C.c_uint8 * C.sizeof(a)).from_address(C.addressof(a))
        for _ in range(slots):
            wide = rng.random() < 0.5 and C.sizeof(a) >= 8
            size = 8 if wide else 4
            off = rng.randrange(0, C.sizeof(a) - size + 1, size)
            raw[off:off + size] = (rng.choice(VALS) & (2 ** (8 * size) - 1)).to_bytes(size, "little")

    seen = {}
    for it in range(%d):
        name, a = rng.choice(valid())
        poke(a, C.sizeof(a) // 4 if it %% 4 == 0 else rng.randint(1, 3))
        grid, block = (rng.choice(VALS) & 0x7fffffff, rng.choice(VALS) & 0x7fffffff) if rng.random() < 0.3 else (0, 0)
        rc = lib.hf_launch_native(name, C.byref(a), grid, block, None)
        seen[rc] = seen.get(rc, 0) + 1
    print(sorted(seen.items()))
    assert set(seen) <= {0, L.HF_EINVAL, L.HF_EUNSUPPORTED, L.HF_EHIP}, seen
    assert seen.get(L.HF_EINVAL, 0) > 100 and seen.get(L.HF_EHIP, 0) > 100   # both refused and accepted structs occurred
""")


def test_validators_survive_arbitrary_argument_structs():
    import torch
    if torch.cuda.is_available():
        pytest.skip("runs only without a GPU: accepted structs would be launched on made-up pointers")
    r = subprocess.run([sys.executable, "-c", CHILD % (ROOT, 30000)], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
