"""The content hash behind the prepared-weight cache of the host entry points (fastertnn_amd/csrc/host_hash.cpp):
deterministic, sensitive to every bit and to the length, in both implementations (AES rounds where the CPU has them,
multiply-rotate lanes everywhere) and in the sliced form that large buffers take.  CPU only: the hash never touches
the device."""
import numpy as np
import pytest


@pytest.fixture(scope="module")
def lib():
    import fastertnn_amd.lib as lib
    return lib


@pytest.mark.parametrize("portable", [False, True], ids=["cache_form", "portable"])
def test_hash_is_stable_and_sees_every_bit(lib, portable):
    rng = np.random.default_rng(1)
    for nbytes in (32, 64, 96, 100, 4096 + 32, 150016, (1 << 20) + 64, (3 << 20) + 160):
        a = rng.integers(0, 256, size=nbytes, dtype=np.uint8)
        h = lib.host_hash128(a, portable)
        assert h == lib.host_hash128(a.copy(), portable)                 # the address plays no part
        assert h[0] != h[1]
        seen = {h}
        for pos in sorted({0, 1, 15, 16, 31, 32, 63, nbytes // 2, nbytes - 33, nbytes - 1} & set(range(nbytes))):
            for bit in (0, 7):
                b = a.copy()
                b[pos] ^= np.uint8(1 << bit)
                hb = lib.host_hash128(b, portable)
                assert hb[0] != h[0] and hb[1] != h[1], (nbytes, pos, bit)
                seen.add(hb)
        assert len(seen) == 1 + 2 * len({0, 1, 15, 16, 31, 32, 63, nbytes // 2, nbytes - 33, nbytes - 1} & set(range(nbytes)))


@pytest.mark.parametrize("portable", [False, True], ids=["cache_form", "portable"])
def test_length_is_part_of_the_hash(lib, portable):
    """a buffer and the same buffer with zero bytes appended hash differently (the tail is zero-padded internally)"""
    for nbytes in (32, 48, 64, 1 << 20):
        a = np.zeros(nbytes + 64, np.uint8)
        a[:nbytes] = 7
        hs = {lib.host_hash128(a[:n], portable) for n in (nbytes, nbytes + 1, nbytes + 16, nbytes + 32, nbytes + 64)}
        assert len(hs) == 5


def test_two_implementations_are_independent(lib):
    a = np.arange(4096, dtype=np.uint8)
    if lib._L.ftnn_host_hash_uses_aes():
        assert lib.host_hash128(a, False) != lib.host_hash128(a, True)
    else:
        assert lib.host_hash128(a, False) == lib.host_hash128(a, True)


def test_no_collisions_among_many_similar_buffers(lib):
    """64 K buffers that differ in one word each: 128-bit hashes, and each 64-bit half on its own, all distinct"""
    base = np.random.default_rng(5).integers(-2 ** 63, 2 ** 63, size=512, dtype=np.int64)
    full, lo, hi = set(), set(), set()
    for i in range(512):
        for delta in range(1, 129):
            b = base.copy()
            b[i] += delta
            h = lib.host_hash128(b)
            full.add(h), lo.add(h[0]), hi.add(h[1])
    assert len(full) == len(lo) == len(hi) == 512 * 128
