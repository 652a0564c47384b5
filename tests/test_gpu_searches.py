"""GPU parity of the nonce searches, native and fused, through the C-ABI: every
found nonce, digest and (for Ethash) mix digest must equal the CPU oracle's."""
import os

import numpy as np
import pytest
import torch

from hfuse_amd import _lib as L
from hfuse_amd import launcher as H
from oracle import oracle as O

pytestmark = pytest.mark.gpu

SEED = 0x48467573
EASY16 = (1 << 48) - 1   # 16 leading zero bits
EASY12 = (1 << 52) - 1
EASY10 = (1 << 54) - 1


def sync():
    torch.cuda.synchronize()


def oracle_hits(found_hits):
    found, hits = found_hits
    return found, [(h.nonce, h.digest_bytes(), h.mix_bytes()) for h in hits]


def test_sha256d_bitcoin_genesis_on_gpu(cuda):
    hdr = bytes.fromhex("01000000" + "00" * 32 +
                        "3ba3edfd7a7b12b27ac72c3e67768f617fc81bc3888a51323a9fb8aa4b1e5e4a" +
                        "29ab5f49" + "ffff001d" + "00000000")
    H.sha256d_set_block(hdr, 0x00000000FFFF0000)
    res = H.new_search_results()
    start = 2083236893 - (1 << 19)
    H.launch_native("sha256d_gpu_hash_shared", H.sha256d_args(res, 1 << 20, start))
    sync()
    found, hits = H.read_search_results(res)
    assert found == 1 and hits[0][0] == 2083236893
    assert hits[0][1][::-1].hex() == "000000000019d6689c085ae165831e934ff763ae46a2a6c172b3f1b60a8ce26f"


@pytest.mark.parametrize("start,count,grid,block", [(0, 1 << 20, 0, 0), (0xFFFFF000, 1 << 14, 0, 0),
                                                    (12345, 100001, 7, 64)])
def test_sha256d_found_set(cuda, start, count, grid, block):
    hdr = O.seeded_bytes(80, SEED + 1)
    H.sha256d_set_block(hdr, EASY16 if count > (1 << 17) else EASY12)
    res = H.new_search_results()
    H.launch_native("sha256d_gpu_hash_shared", H.sha256d_args(res, count, start), grid, block)
    sync()
    want = oracle_hits(O.sha256d_search(hdr, start, count, EASY16 if count > (1 << 17) else EASY12))
    assert want[0] > 0
    assert H.read_search_results(res) == want


@pytest.mark.parametrize("kernel,setter,digest", [
    ("sia_blake2b_gpu_hash", H.sia_blake2b_set_block, O.sia_blake2b_80),
    ("blake2b_gpu_hash", H.blake2b_set_block, O.ccminer_blake2b_80)])
def test_blake2b_found_set(cuda, kernel, setter, digest):
    hdr = O.seeded_bytes(80, SEED + 2)
    setter(hdr)
    res = H.new_search_results()
    start, count = 0xFFFF0000, 1 << 20  # wraps around 2^32 like the original's uint32 nonce
    H.launch_native(kernel, H.blake2b_args(res, count, start, EASY16))
    sync()
    found, hits = H.read_search_results(res)
    assert found > 0 and found == len(hits)
    if kernel == "sia_blake2b_gpu_hash":
        assert (found, hits) == oracle_hits(O.sia_search(hdr, start, count, EASY16))
    else:
        # brute force over the window with the oracle's single-nonce digest
        want = []
        for i in range(count):
            n = (start + i) & 0xFFFFFFFF
            d = digest(hdr, n)
            if int.from_bytes(d[:8], "big") <= EASY16:
                want.append((n, d, bytes(32)))
        assert hits == sorted(want)


def _dag(cuda, n_items, seed):
    dag = torch.empty(n_items * 32, dtype=torch.int32, device=cuda)
    H.fill_splitmix64(dag, seed)
    return dag


def test_fill_splitmix64_matches_oracle(cuda):
    dag = _dag(cuda, 1000, SEED)
    sync()
    want = O.fill_splitmix64(1000 * 16, SEED).view(np.int32)
    assert np.array_equal(dag.cpu().numpy(), want)


@pytest.mark.parametrize("n_items", [1 << 16, 100003])  # power of two (mask) and not (modulo)
def test_ethash_found_set(cuda, n_items):
    dag = _dag(cuda, n_items, SEED)
    header = O.seeded_bytes(32, SEED + 3)
    target = (1 << 54) - 1  # 10 leading zero bits: ~64 hits in 2^16 nonces would overflow; use 2^15
    H.ethash_set_constants(dag, n_items, header, target)
    res = H.new_search_results()
    start, grid = 0x0123456700000000, 256  # 256 blocks x 128 threads = 2^15 nonces
    H.launch_native("ethash_search", H.ethash_args(res, start), grid, 128)
    sync()
    want = oracle_hits(O.ethash_search(None, SEED, n_items, header, start, grid * 128, target))
    assert 0 < want[0] <= 64
    assert H.read_search_results(res) == want


def test_ethash_every_lane_group_position(cuda):
    """With an all-accepting target every nonce is a hit: checks all 8 positions of a lane
    group and all 4 interleaved hashes, mix digest and final hash, against the oracle."""
    n_items = 4099
    dag = _dag(cuda, n_items, SEED + 9)
    header = O.seeded_bytes(32, SEED + 4)
    H.ethash_set_constants(dag, n_items, header, (1 << 64) - 1)
    res = H.new_search_results()
    H.launch_native("ethash_search", H.ethash_args(res, 77), 1, 64)
    sync()
    found, hits = H.read_search_results(res)
    assert found == 64 and [h[0] for h in hits] == list(range(77, 77 + 64))
    for nonce, digest, mix in hits:
        assert (mix, digest) == O.ethash_hash(None, SEED + 9, n_items, header, nonce)


def _search_pair_args(cuda, k, count, start):
    res = H.new_search_results()
    if k == "sha256d_gpu_hash_shared":
        return res, H.sha256d_args(res, count, start)
    if k in ("sia_blake2b_gpu_hash", "blake2b_gpu_hash"):
        return res, H.blake2b_args(res, count, start, EASY16)
    return res, H.ethash_args(res, start)


def test_fused_sha256d_sia(cuda, cfg):
    h1, h2 = O.seeded_bytes(80, SEED + 5), O.seeded_bytes(80, SEED + 6)
    H.sha256d_set_block(h1, EASY16)
    H.sia_blake2b_set_block(h2)
    want1 = oracle_hits(O.sha256d_search(h1, 5, 1 << 20, EASY16))
    want2 = oracle_hits(O.sia_search(h2, 9, (1 << 20) + 333, EASY16))
    i = cfg.find_fusion("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash")
    for plan in (cfg.plan(i), cfg.plan(i, "hfuse", -1, 64), cfg.plan(i, "hfuse_lb", 0), cfg.plan(i, "vfuse")):
        r1, a1 = _search_pair_args(cuda, "sha256d_gpu_hash_shared", 1 << 20, 5)
        r2, a2 = _search_pair_args(cuda, "sia_blake2b_gpu_hash", (1 << 20) + 333, 9)
        plan.launch(a1, a2)
        sync()
        assert H.read_search_results(r1) == want1
        assert H.read_search_results(r2) == want2


def test_fused_search_unequal_grids_with_and_without_lending(cuda, cfg):
    h1, h2 = O.seeded_bytes(80, SEED + 21), O.seeded_bytes(80, SEED + 22)
    H.sha256d_set_block(h1, EASY12)
    H.sia_blake2b_set_block(h2)
    want1 = oracle_hits(O.sha256d_search(h1, 0, 1 << 16, EASY12))
    want2 = oracle_hits(O.sia_search(h2, 0, 1 << 17, EASY12))
    plan = cfg.plan(cfg.find_fusion("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash"))
    for lend in (True, False):
        plan.set_lending(lend)
        for grids in ((5, 40), (40, 5)):
            plan.set_grids(*grids)
            r1, r2 = H.new_search_results(), H.new_search_results()
            plan.launch(H.sha256d_args(r1, 1 << 16, 0), H.blake2b_args(r2, 1 << 17, 0, EASY12))
            sync()
            assert H.read_search_results(r1) == want1
            assert H.read_search_results(r2) == want2


def test_fused_ethash_sia(cuda, cfg):
    n_items = 1 << 16
    dag = _dag(cuda, n_items, SEED)
    header = O.seeded_bytes(32, SEED + 7)
    h2 = O.seeded_bytes(80, SEED + 8)
    target = (1 << 54) - 1
    H.ethash_set_constants(dag, n_items, header, target)
    H.sia_blake2b_set_block(h2)
    grid = 256
    want1 = oracle_hits(O.ethash_search(None, SEED, n_items, header, 1000, grid * 128, target))
    want2 = oracle_hits(O.sia_search(h2, 0, 4 * grid * 128, EASY12))
    i = cfg.find_fusion("ethash_search", "sia_blake2b_gpu_hash")
    j = cfg.find_fusion("sia_blake2b_gpu_hash", "ethash_search")
    for idx, plan in ((i, cfg.plan(i)), (j, cfg.plan(j))):
        r1 = H.new_search_results()
        r2 = H.new_search_results()
        a1 = H.ethash_args(r1, 1000)
        a2 = H.blake2b_args(r2, 4 * grid * 128, 0, EASY12)
        if idx == i:
            plan.launch(a1, a2, grid_blocks=grid)
        else:
            plan.launch(a2, a1, grid_blocks=grid)
        sync()
        assert H.read_search_results(r1) == want1
        assert H.read_search_results(r2) == want2


def test_every_shipped_search_pair(cuda, cfg):
    """All search pairs of the shipped fusion list against the natives' results."""
    n_items = 1 << 14
    dag = _dag(cuda, n_items, SEED)
    header = O.seeded_bytes(32, SEED + 10)
    hs, hb, hc = (O.seeded_bytes(80, SEED + 11 + k) for k in range(3))
    H.ethash_set_constants(dag, n_items, header, (1 << 55) - 1)
    H.sha256d_set_block(hs, EASY10)
    H.sia_blake2b_set_block(hb)
    H.blake2b_set_block(hc)
    grid, count = 128, 128 * 128
    names = ("ethash_search", "sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash", "blake2b_gpu_hash")
    native = {}
    for k in names:
        res, a = _search_pair_args(cuda, k, count, 42)
        if k.endswith("blake2b_gpu_hash"):
            a = H.blake2b_args(res, count, 42, EASY10)
        H.launch_native(k, a, grid, 128)
        sync()
        native[k] = H.read_search_results(res)
        assert native[k][0] > 0
    n = 0
    for i, (_, k1, k2) in enumerate(cfg.fusions()):
        if k1 in names and k2 in names:
            r1, a1 = _search_pair_args(cuda, k1, count, 42)
            r2, a2 = _search_pair_args(cuda, k2, count, 42)
            if k1.endswith("blake2b_gpu_hash"):
                a1 = H.blake2b_args(r1, count, 42, EASY10)
            if k2.endswith("blake2b_gpu_hash"):
                a2 = H.blake2b_args(r2, count, 42, EASY10)
            cfg.plan(i).launch(a1, a2, grid_blocks=grid)
            sync()
            assert H.read_search_results(r1) == native[k1], (k1, k2)
            assert H.read_search_results(r2) == native[k2], (k1, k2)
            # the register-bounded builds (8 waves per SIMD; these spill): same found sets
            for preset in ("hfuse", "vfuse"):
                r1, a1 = _search_pair_args(cuda, k1, count, 42)
                r2, a2 = _search_pair_args(cuda, k2, count, 42)
                if k1.endswith("blake2b_gpu_hash"):
                    a1 = H.blake2b_args(r1, count, 42, EASY10)
                if k2.endswith("blake2b_gpu_hash"):
                    a2 = H.blake2b_args(r2, count, 42, EASY10)
                plan = cfg.plan(i, preset)
                plan.set_launch_bound(True)
                plan.launch(a1, a2, grid_blocks=grid)
                sync()
                assert H.read_search_results(r1) == native[k1], (k1, k2, preset, "bounded")
                assert H.read_search_results(r2) == native[k2], (k1, k2, preset, "bounded")
            n += 1
    assert n == 7


def test_ethash_sia_bounded_builds(cuda, cfg):
    """Ethash + Sia-Blake2b in its register-bounded builds (6 waves per SIMD is the occupancy formula's value for
    128 + 64 threads; 5, 7 and 8 are built as well) against the oracle."""
    n_items = 1 << 14
    dag = _dag(cuda, n_items, SEED)
    header, h2 = O.seeded_bytes(32, SEED + 30), O.seeded_bytes(80, SEED + 31)
    target = (1 << 55) - 1
    consts = H.Constants().set_ethash(dag, n_items, header, target).set_sia_blake2b(h2)
    plan = cfg.plan(cfg.find_fusion("ethash_search", "sia_blake2b_gpu_hash"), "hfuse_lb")
    plan.bind_constants(consts)
    assert plan.launch_waves == (6, 6)
    grid = 64
    share = plan.partition.hi[0] - plan.partition.lo[0]
    want1 = oracle_hits(O.ethash_search(None, SEED, n_items, header, 7, grid * share, target))
    want2 = oracle_hits(O.sia_search(h2, 0, 1 << 15, EASY10))
    assert want1[0] > 0 and want2[0] > 0
    for waves in (0, 5, 7, 8):
        plan.set_launch_waves(waves)
        assert plan.launch_waves[1] == (6 if waves == 0 else waves)
        r1, r2 = H.new_search_results(), H.new_search_results()
        plan.launch(H.ethash_args(r1, 7), H.blake2b_args(r2, 1 << 15, 0, EASY10), grid_blocks=grid)
        sync()
        assert H.read_search_results(r1) == want1 and H.read_search_results(r2) == want2, waves


def test_three_search_kernels_in_one_launch(cuda):
    """configs/crypt_four.yaml: ccminer-Blake2b + SHA-256d + Ethash as one fused kernel (and its vertical
    baseline), found sets of all three against the oracle."""
    import hfuse_amd
    t = hfuse_amd.triples_config()
    i = t.find_fusion_n("blake2b_gpu_hash", "sha256d_gpu_hash_shared", "ethash_search")
    n_items = 100003
    dag = _dag(cuda, n_items, SEED)
    header = O.seeded_bytes(32, SEED + 50)
    hb, hs = O.seeded_bytes(80, SEED + 51), O.seeded_bytes(80, SEED + 52)
    eth_target = (1 << 55) - 1
    consts = H.Constants().set_ethash(dag, n_items, header, eth_target).set_sha256d(hs, EASY10).set_blake2b(hb)
    count = 20000
    want_b = []
    for k in range(count):
        nonce = (0xFFFFF000 + k) & 0xFFFFFFFF
        d = O.ccminer_blake2b_80(hb, nonce)
        if int.from_bytes(d[:8], "big") <= EASY10:
            want_b.append((nonce, d, bytes(32)))
    want_b = (len(want_b), sorted(want_b))
    want_s = oracle_hits(O.sha256d_search(hs, 17, count, EASY10))
    assert want_b[0] > 0 and want_s[0] > 0
    # the list as the reference orders it, and the same three kernels listed in two other orders (the Context partitions
    # in list order, include/KernelFusion.h:45-80: same instantiation, other thread bounds, arguments in list order)
    kernels_yaml = open(os.path.join(hfuse_amd.CONFIG_DIR, "gfx950_kernels.yaml")).read()
    names = ("blake2b_gpu_hash", "sha256d_gpu_hash_shared", "ethash_search")
    cases = [(t, i, (0, 1, 2), preset, block, grid)
             for preset, block, grid in (("hfuse", None, 96), ("hfuse", (64, 128, 192), 64), ("hfuse_lb", None, 32), ("vfuse", None, 96))]
    for order in ((2, 0, 1), (1, 2, 0)):
        text = "- File: permuted\n  Kernels:\n" + "".join(f"    - {names[k]}\n" for k in order) + "  Blocks: [128, 64, 192]\n"
        cases += [(H.Config(text, kernels_yaml), 0, order, "hfuse", None, 48), (H.Config(text, kernels_yaml), 0, order, "vfuse", None, 48)]
    for conf, idx, order, preset, block, grid in cases:
        plan = conf.plan(idx, preset)
        if block:
            plan.set_block_n(*block)
        plan.bind_constants(consts)
        q = plan.partition_n
        pos = order.index(2)                        # where the list names Ethash
        share = q.hi[pos] - q.lo[pos]
        want_e = oracle_hits(O.ethash_search(None, SEED, n_items, header, 1 << 33, grid * share, eth_target))
        assert 0 < want_e[0] <= 64
        rb, rs, re_ = H.new_search_results(), H.new_search_results(), H.new_search_results()
        by_kernel = [H.blake2b_args(rb, count, 0xFFFFF000, EASY10), H.sha256d_args(rs, count, 17), H.ethash_args(re_, 1 << 33)]
        plan.launch_n([by_kernel[k] for k in order], grid_blocks=grid)
        sync()
        assert H.read_search_results(rb) == want_b, (preset, order)
        assert H.read_search_results(rs) == want_s, (preset, order)
        assert H.read_search_results(re_) == want_e, (preset, order)
    with pytest.raises(H.HfuseError) as e:          # three kernels that are none of the built lists: said when the plan is made
        H.Config("- File: x\n  Kernels: [blake2b_gpu_hash, sia_blake2b_gpu_hash, ethash_search]\n", kernels_yaml).plan(0)
    assert e.value.code == L.HF_EUNSUPPORTED


def _strict(found_hits, limit, key):
    """The sub-set of an easy-target found set that also meets the stricter target `limit`."""
    hits = [h for h in found_hits[1] if key(h[1]) <= limit]
    return len(hits), hits


def test_fused_sha256d_sia_full_benchmark_size(cuda, cfg):
    """Benchmark configuration 4 at its full size: the fused kernel over 2^30 SHA-256d nonces and 2^30
    Sia-Blake2b nonces at the 32-leading-zero-bit targets; found sets (most likely empty: P(hit) is 22 % per
    hash) equal to a full scan by the oracle.  Because an empty set says little about coverage, the same
    launch is repeated at 26 leading zero bits (about 16 hits per hash expected) against the same scans."""
    from hfuse_amd.workloads import splitmix64_bytes
    n = 1 << 30
    h1, h2 = splitmix64_bytes(80, SEED + 100), splitmix64_bytes(80, SEED + 101)   # the benchmark's headers
    t32, t26 = (1 << 32) - 1, (1 << 38) - 1
    easy1 = oracle_hits(O.sha256d_search(h1, 0, n, t26))      # one full scan per hash at the easy target ...
    easy2 = oracle_hits(O.sia_search(h2, 0, n, t26))
    assert 1 <= easy1[0] <= 64 and 1 <= easy2[0] <= 64
    strict1 = _strict(easy1, t32, lambda d: int.from_bytes(d[24:32], "little"))   # ... holds the strict one too
    strict2 = _strict(easy2, t32, lambda d: int.from_bytes(d[:8], "big"))
    plan = cfg.plan(cfg.find_fusion("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash"))
    for target, want1, want2 in ((t32, strict1, strict2), (t26, easy1, easy2)):
        c = H.Constants().set_sha256d(h1, target).set_sia_blake2b(h2)
        plan.bind_constants(c)
        r1, r2 = H.new_search_results(), H.new_search_results()
        plan.launch(H.sha256d_args(r1, n, 0), H.blake2b_args(r2, n, 0, target))
        sync()
        assert H.read_search_results(r1) == want1, hex(target)
        assert H.read_search_results(r2) == want2, hex(target)


def test_fused_ethash_sia_full_benchmark_size(cuda, cfg):
    """Benchmark configuration 5 at its full size: Ethash over the 4 GiB synthetic DAG (item byte offsets
    beyond 2^32), 2^28 nonces at 24 leading zero bits, fused with 2^30 Sia-Blake2b nonces; nonces, final
    hashes and mix digests equal to a full scan by the oracle over the same DAG (items evaluated on the fly)."""
    from hfuse_amd.workloads import SearchPair
    sp = SearchPair("ethash_search", "sia_blake2b_gpu_hash", 28, 30)
    i = cfg.find_fusion("ethash_search", "sia_blake2b_gpu_hash")
    plan = cfg.plan(i)
    plan.bind_constants(sp.constants)
    r1, r2, a1, a2 = sp.fresh()
    share = plan.partition.hi[0] - plan.partition.lo[0]
    plan.launch(a1, a2, grid_blocks=sp.nonces[0] // share)
    n1 = H.new_search_results()
    H.launch_native("ethash_search", H.ethash_args(n1, 0), sp.grid, 128, constants=sp.constants)
    sync()
    got = H.read_search_results(r1)
    assert got == H.read_search_results(n1)
    want = oracle_hits(O.ethash_search(None, SEED, sp.dag_items, sp.headers[0], 0, sp.nonces[0], sp.ETHASH_TARGET))
    assert 1 <= want[0] <= 64
    assert got == want
    # the Blake2b half of the same launch: found set against a full scan (the other full-size test pins
    # the same 2^30 range at an easier target as well)
    assert H.read_search_results(r2) == oracle_hits(O.sia_search(sp.headers[1], 0, sp.nonces[1], sp.TARGET32))


def test_two_threads_with_their_own_constants(cuda, cfg):
    """Two host threads search different headers at once, each with its own hf_constants (one bound to a
    plan, one passed per call) and its own stream: neither sees the other's header."""
    import threading
    hdrs = [O.seeded_bytes(80, SEED + 40 + k) for k in range(2)]
    want = [oracle_hits(O.sha256d_search(h, 0, 1 << 16, EASY12)) for h in hdrs]   # about 16 hits each
    assert want[0] != want[1] and 0 < want[0][0] < 64 and 0 < want[1][0] < 64
    i = cfg.find_fusion("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash")
    errors = []

    def work(k):
        try:
            stream = torch.cuda.Stream()
            consts = H.Constants().set_sha256d(hdrs[k], EASY12).set_sia_blake2b(hdrs[1 - k])
            plan = cfg.plan(i)
            plan.bind_constants(consts)
            for rep in range(20):
                r1, r2 = H.new_search_results(), H.new_search_results()
                with torch.cuda.stream(stream):
                    if rep % 2:
                        plan.launch(H.sha256d_args(r1, 1 << 16, 0), H.blake2b_args(r2, 1 << 10, 0, EASY12), stream=stream)
                    else:
                        H.launch_native("sha256d_gpu_hash_shared", H.sha256d_args(r1, 1 << 16, 0), stream=stream, constants=consts)
                stream.synchronize()
                assert H.read_search_results(r1) == want[k], (k, rep)
        except Exception as e:   # surfaces in the main thread
            errors.append(e)

    threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_zero_nonces_find_nothing(cuda, cfg):
    hdr = O.seeded_bytes(80, SEED + 5)
    H.sha256d_set_block(hdr, EASY12)
    H.sia_blake2b_set_block(O.seeded_bytes(80, SEED + 6))
    r1, r2 = H.new_search_results(), H.new_search_results()
    H.launch_native("sha256d_gpu_hash_shared", H.sha256d_args(r1, 0, 0))
    H.launch_native("sia_blake2b_gpu_hash", H.blake2b_args(r2, 0, 0, EASY12))
    sync()
    assert H.read_search_results(r1)[0] == 0 and H.read_search_results(r2)[0] == 0
    # an empty half next to a working one: the working half's found set is unchanged
    i = cfg.find_fusion("sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash")
    cfg.plan(i).launch(H.sha256d_args(r1, 1 << 14, 0), H.blake2b_args(r2, 0, 0, EASY12))
    sync()
    want = oracle_hits(O.sha256d_search(hdr, 0, 1 << 14, EASY12))
    assert want[0] > 0 and H.read_search_results(r1) == want
    assert H.read_search_results(r2)[0] == 0


def test_random_fused_search_configurations(cuda, cfg):
    """Seeded random walk over the seven search pairs: random nonce windows (wrapping 2^32 too),
    fused block shapes up to 512 threads, lending, partition mode, caller grids.  The fused found
    sets must equal the oracle's for the same windows."""
    import random
    from hfuse_amd import _lib as L
    rng = random.Random(0xE7A5)
    n_items = 4099                      # not a power of two: the modulo path
    dag = _dag(cuda, n_items, SEED)
    header = O.seeded_bytes(32, SEED + 20)
    hs, hb, hc = (O.seeded_bytes(80, SEED + 21 + k) for k in range(3))
    eth_target = (1 << 55) - 1          # about one hit in 500 nonces: stays below the 64 records kept
    H.ethash_set_constants(dag, n_items, header, eth_target)
    H.sha256d_set_block(hs, EASY10)
    H.sia_blake2b_set_block(hb)
    H.blake2b_set_block(hc)
    names = ("ethash_search", "sha256d_gpu_hash_shared", "sia_blake2b_gpu_hash", "blake2b_gpu_hash")
    pairs = [(i, k1, k2) for i, (_, k1, k2) in enumerate(cfg.fusions()) if k1 in names and k2 in names]
    assert len(pairs) == 7

    def expected(k, start, count):
        if k == "ethash_search":
            return oracle_hits(O.ethash_search(None, SEED, n_items, header, start, count, eth_target))
        if k == "sha256d_gpu_hash_shared":
            return oracle_hits(O.sha256d_search(hs, start, count, EASY10))
        if k == "sia_blake2b_gpu_hash":
            return oracle_hits(O.sia_search(hb, start, count, EASY10))
        want = []                        # ccminer layout: brute force with the oracle's single-nonce digest
        for t in range(count):
            nonce = (start + t) & 0xFFFFFFFF
            d = O.ccminer_blake2b_80(hc, nonce)
            if int.from_bytes(d[:8], "big") <= EASY10:
                want.append((nonce, d, bytes(32)))
        return len(want), sorted(want)

    for case in range(24):
        i, k1, k2 = rng.choice(pairs)
        grid = rng.choice([8, 24, 33]) if "ethash_search" in (k1, k2) else rng.choice([0, 0, 5, 19])
        starts = [rng.choice([0, 12345, 0xFFFFFF00, rng.randrange(1 << 32)]) for _ in range(2)]
        plan = cfg.plan(i, rng.choice(["hfuse", "hfuse_lb", "vfuse"]))
        threads = [128, 128]             # the kernel table's blocks; a vertical plan keeps them
        if "vfuse" not in plan.name:
            t1 = 64 * rng.randint(1, 7)
            t2 = 64 * rng.randint(1, 8 - t1 // 64)
            plan.set_block(t1, t2)
            plan.set_lending(rng.random() < 0.5)
            if rng.random() < 0.3:
                plan.set_barrier_mode(L.HF_BARRIER_BLOCKIDX)
            threads = [t1, t2]
        # Ethash scans gridDim * blockDim nonces like the original: its share of the fused block counts
        counts = [grid * threads[h] if k == "ethash_search" else rng.choice([1, 1000, 4096, 10007]) for h, k in enumerate((k1, k2))]
        res, args = [], []
        for k, st, cnt in zip((k1, k2), starts, counts):
            r = H.new_search_results()
            res.append(r)
            if k == "ethash_search":
                args.append(H.ethash_args(r, st))
            elif k == "sha256d_gpu_hash_shared":
                args.append(H.sha256d_args(r, cnt, st))
            else:
                args.append(H.blake2b_args(r, cnt, st, EASY10))
        label = f"case {case}: {k1}[{starts[0]:#x}+{counts[0]}] + {k2}[{starts[1]:#x}+{counts[1]}] grid {grid} block {threads}"
        plan.launch(args[0], args[1], grid_blocks=grid)
        sync()
        for k, r, st, cnt in zip((k1, k2), res, starts, counts):
            if k == "ethash_search" and st + cnt > (1 << 32):
                continue   # 64-bit nonces do not wrap; the 32-bit window helpers above do
            assert H.read_search_results(r) == expected(k, st, cnt), f"{label}: {k}"
