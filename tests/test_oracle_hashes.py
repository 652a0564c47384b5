"""Pins of the oracle's hash functions: none of these retypes the oracle's own
formulas -- they are hashlib, published known-answer vectors and a real block."""
import hashlib
import os

import pytest

from oracle import oracle as O

MSGS = [b"", b"abc", b"a" * 55, b"a" * 56, b"a" * 63, b"a" * 64, b"a" * 119, b"a" * 120, b"q" * 128,
        b"z" * 129, bytes(range(256)) * 5]


@pytest.mark.parametrize("m", MSGS, ids=lambda m: f"len{len(m)}")
def test_sha256_vs_hashlib(m):
    assert O.sha256(m) == hashlib.sha256(m).digest()


def test_sha256_nist_abc():
    assert O.sha256(b"abc").hex() == "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad"


def test_sha256d_bitcoin_genesis():
    # version | prev (zero) | merkle root | time | bits | nonce  -- block 0 of Bitcoin
    hdr = bytes.fromhex("01000000" + "00" * 32 +
                        "3ba3edfd7a7b12b27ac72c3e67768f617fc81bc3888a51323a9fb8aa4b1e5e4a" +
                        "29ab5f49" + "ffff001d" + "00000000")
    d = O.sha256d_80(hdr, 2083236893)
    assert d[::-1].hex() == "000000000019d6689c085ae165831e934ff763ae46a2a6c172b3f1b60a8ce26f"
    # the search finds exactly that nonce in a window around it (target from bits 0x1d00ffff)
    found, hits = O.sha256d_search(hdr, 2083236893 - 3000, 6000, 0x00000000FFFF0000)
    assert found == 1 and hits[0].nonce == 2083236893 and hits[0].digest_bytes() == d


def test_sha256d_80_vs_hashlib_random_nonces():
    hdr = os.urandom(80)
    for nonce in (0, 1, 0xFFFFFFFF, 0x12345678):
        h = hdr[:76] + nonce.to_bytes(4, "little")
        assert O.sha256d_80(hdr, nonce) == hashlib.sha256(hashlib.sha256(h).digest()).digest()


@pytest.mark.parametrize("m", MSGS, ids=lambda m: f"len{len(m)}")
def test_blake2b_vs_hashlib(m):
    assert O.blake2b(m, 64) == hashlib.blake2b(m, digest_size=64).digest()
    assert O.blake2b(m, 32) == hashlib.blake2b(m, digest_size=32).digest()


def test_blake2b_rfc7693_appendix_a():
    assert O.blake2b(b"abc", 64).hex() == (
        "ba80a53f981c4d0d6a2797b69f12f6e94c212f14685ac4b74b12bb6fdbffa2d1"
        "7d87c5392aab792dc252d5de4533cc9518d38aa8dbf1925ab92386edd4009923")


def test_sia_and_ccminer_layouts_vs_hashlib():
    hdr = os.urandom(80)
    for nonce in (0, 7, 0xFFFFFFFF, 0xCAFEBABE):
        sia = hdr[:32] + nonce.to_bytes(4, "little") + hdr[36:]
        cc = hdr[:76] + nonce.to_bytes(4, "little")
        assert O.sia_blake2b_80(hdr, nonce) == hashlib.blake2b(sia, digest_size=32).digest()
        assert O.ccminer_blake2b_80(hdr, nonce) == hashlib.blake2b(cc, digest_size=32).digest()


def test_sia_search_bruteforce_window():
    hdr = O.seeded_bytes(80, 11)
    target = (1 << 52) - 1  # 12 leading zero bits
    found, hits = O.sia_search(hdr, 100, 1 << 16, target)
    want = []
    for n in range(100, 100 + (1 << 16)):
        d = hashlib.blake2b(hdr[:32] + n.to_bytes(4, "little") + hdr[36:], digest_size=32).digest()
        if int.from_bytes(d[:8], "big") <= target:
            want.append((int.from_bytes(hdr[36:40], "little") << 32 | n, d))
    assert found == len(want) > 0
    assert [(h.nonce, h.digest_bytes()) for h in hits] == want


@pytest.mark.parametrize("m", MSGS, ids=lambda m: f"len{len(m)}")
def test_keccak_pad06_is_sha3(m):
    assert O.keccak(m, 136, 0x06, 32) == hashlib.sha3_256(m).digest()
    assert O.keccak(m, 72, 0x06, 64) == hashlib.sha3_512(m).digest()


def test_keccak_pad01_empty_string_digests():
    assert O.keccak(b"", 136, 0x01, 32).hex() == \
        "c5d2460186f7233c927e7db2dcc703c0e500b653ca82273b7bfad8045d85a470"
    assert O.keccak(b"", 72, 0x01, 64).hex() == (
        "0eab42de4c3ceb9235fc91acffe746b29c29a8c366b7c60e4e67c466f36a4304"
        "c00fa9caf9d87976ba469bcbe06713b435f091ef2769fb160cdab33d3670680e")


def test_ethash_block22_light_client_vector():
    """libethash's published block-22 check (epoch 0): cache 16776896 B, DAG 1073739904 B."""
    cache = O.ethash_make_cache(16776896 // 64, bytes(32))
    header = bytes.fromhex("372eca2454ead349c3df0ab5d00b0b706b23e49d469387db91811cee0358fc6d")
    mix, fin = O.ethash_light(cache, 1073739904, header, 0x495732e0ed7a801c)
    assert mix.hex() == "2f74cdeb198af0b9abe65d22d372e22fb2d474371774a9583c1cc427a07939f5"
    assert fin.hex() == "00000b184f1fdd88bfd94c86c39e65db0c36144d5e43f745f722196e730cb614"


def test_ethash_zero_dag_closed_form():
    """All-zero DAG: fnv(m, 0) = m * prime, so after 64 accesses mix = seed * prime^64."""
    import numpy as np
    n_items = 64
    dag = np.zeros(n_items * 32, dtype=np.uint32)
    header = O.seeded_bytes(32, 5)
    nonce = 0x0123456789ABCDEF
    mix, fin = O.ethash_hash(dag, 0, n_items, header, nonce)
    s = O.keccak(header + nonce.to_bytes(8, "little"), 72, 0x01, 64)
    sw = [int.from_bytes(s[4 * i:4 * i + 4], "little") for i in range(16)]
    p64 = pow(0x01000193, 64, 1 << 32)
    m = [(sw[k % 16] * p64) & 0xFFFFFFFF for k in range(32)]
    fnv = lambda a, b: ((a * 0x01000193) & 0xFFFFFFFF) ^ b
    cm = [fnv(fnv(fnv(m[4 * k], m[4 * k + 1]), m[4 * k + 2]), m[4 * k + 3]) for k in range(8)]
    cmb = b"".join(x.to_bytes(4, "little") for x in cm)
    assert mix == cmb
    assert fin == O.keccak(s + cmb, 136, 0x01, 32)


def test_ethash_resident_dag_equals_generated_dag():
    import numpy as np
    n_items, seed = 1000, 0x48467573  # not a power of two
    dag = O.fill_splitmix64(n_items * 16, seed).view(np.uint32)
    header = O.seeded_bytes(32, 9)
    for nonce in (0, 1, 12345678901234):
        assert O.ethash_hash(dag, 0, n_items, header, nonce) == O.ethash_hash(None, seed, n_items, header, nonce)


def test_splitmix64_known_sequence():
    # SplitMix64 with seed 0: first outputs of the reference implementation (Vigna)
    assert O.splitmix64_at(0, 0) == 0xE220A8397B1DCDAF
    assert O.splitmix64_at(0, 1) == 0x6E789E6AA1B965F4
    assert O.splitmix64_at(0, 2) == 0x06C45D188009454F


def test_ethash_search_is_the_brute_force_over_ethash_hash():
    """orc_ethash_search (compare + collect + sort) against one loop over orc_ethash_hash: same hits, same
    order, same count, for a window that crosses 2^32 and a target that about one nonce in 16 meets."""
    seed, n_items = 0x48467573, 1021
    header = O.seeded_bytes(32, 77)
    target = (1 << 60) - 1
    start, count = (1 << 32) - 300, 600
    want = []
    for nonce in range(start, start + count):
        mix, fin = O.ethash_hash(None, seed, n_items, header, nonce)
        if int.from_bytes(fin[:8], "big") <= target:
            want.append((nonce, fin, mix))
    found, hits = O.ethash_search(None, seed, n_items, header, start, count, target)
    assert 10 < found == len(want)
    assert [(h.nonce, h.digest_bytes(), h.mix_bytes()) for h in hits] == want
    # more hits than the caller's capacity: the count is still the total, the kept ones are valid hits
    found2, hits2 = O.ethash_search(None, seed, n_items, header, start, count, target, 5)
    assert found2 == found and len(hits2) == 5
    assert all((h.nonce, h.digest_bytes(), h.mix_bytes()) in want for h in hits2)
    # an unreachable target finds nothing
    assert O.ethash_search(None, seed, n_items, header, start, count, 0)[0] == 0
