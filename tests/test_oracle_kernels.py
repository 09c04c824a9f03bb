"""Pins the CPU twins of the device kernels by known answers and by independent numpy
computations (not by re-typing the C loops)."""
import ctypes as C

import numpy as np

import oracle as O

CH = 65536


def scan(orc, buf):
    n = (buf.nbytes + CH - 1) // CH
    flags = np.zeros(n, dtype=np.uint8)
    sums = np.zeros((n, 2), dtype=np.uint64)
    assert orc.oracle_zero_scan(buf.ctypes.data, buf.nbytes, flags.ctypes.data, sums.ctypes.data) == n
    return flags, sums


def test_scan_known_answers(orc):
    z = np.zeros(CH, dtype=np.uint8)
    f, s = scan(orc, z)
    assert f[0] == 1 and s[0, 0] == 0 and s[0, 1] == 0            # all-zero chunk -> (true, 0, 0)
    for word_index in (0, 1, 7, 16382, 16383):                     # one non-zero uint32 word w at index i
        b = np.zeros(CH // 4, dtype=np.uint32)
        w = 0xDEADBEEF
        b[word_index] = w
        f, s = scan(orc, b.view(np.uint8))
        assert f[0] == 0 and s[0, 0] == w and s[0, 1] == w << (32 * (word_index % 2))
    b = np.zeros(CH // 8, dtype=np.uint64)                         # two identical uint64 words: xor cancels, sum does not
    b[3] = b[900] = 0x0123456789ABCDEF
    f, s = scan(orc, b.view(np.uint8))
    assert f[0] == 0 and s[0, 1] == 0 and s[0, 0] == 2 * (0x01234567 + 0x89ABCDEF)
    b = np.zeros(CH, dtype=np.uint8)                               # a single non-zero byte at either end
    b[0] = 1
    assert scan(orc, b)[0][0] == 0
    b[:] = 0
    b[-1] = 0x80
    f, s = scan(orc, b)
    assert f[0] == 0 and s[0, 0] == 0x80000000 and s[0, 1] == 0x80 << 56
    full = np.full(CH // 4, 0xFFFFFFFF, dtype=np.uint32)           # largest possible sum: no wrap
    f, s = scan(orc, full.view(np.uint8))
    assert s[0, 0] == 0xFFFFFFFF * (CH // 4) and s[0, 1] == 0


def test_scan_matches_numpy_on_random_ragged_input(orc):
    rng = np.random.default_rng(7)
    nbytes = 5 * CH + 4096                                         # last chunk is short
    buf = rng.integers(0, 256, nbytes, dtype=np.uint8)
    buf[CH:2 * CH] = 0                                             # chunk 1 zero
    buf[3 * CH + 16:4 * CH] = 0                                    # chunk 3 almost zero
    f, s = scan(orc, buf)
    for c in range(6):
        part = buf[c * CH:(c + 1) * CH]
        assert f[c] == (0 if part.any() else 1)
        assert s[c, 0] == int(part.view(np.uint32).astype(np.uint64).sum())
        assert s[c, 1] == int(np.bitwise_xor.reduce(part.view(np.uint64)))
    assert list(f) == [0, 1, 0, 0, 0, 0]


def test_pack_unpack_match_numpy_slicing(orc):
    rng = np.random.default_rng(11)
    src = rng.integers(0, 256, 1 << 20, dtype=np.uint8)
    pieces = [(4096, 0, 8192), (65536 + 16, 8192, 48), (300000, 8240, 100000 - 100000 % 16)]
    descs = (O.CopyDesc * len(pieces))(*[O.CopyDesc(src.ctypes.data + a, off, n) for a, off, n in pieces])
    staging = np.full(1 << 18, 0xCC, dtype=np.uint8)
    orc.oracle_gather_pack(descs, len(pieces), staging.ctypes.data)
    expect = np.full(1 << 18, 0xCC, dtype=np.uint8)
    for a, off, n in pieces:
        expect[off:off + n] = src[a:a + n]
    assert np.array_equal(staging, expect)
    dst = np.full(1 << 20, 0x11, dtype=np.uint8)
    d2 = [O.CopyDesc(dst.ctypes.data + a, off, n) for a, off, n in pieces]
    d2.append(O.CopyDesc(dst.ctypes.data + 500000, O.DESC_ZERO, 4096))
    orc.oracle_scatter_unpack((O.CopyDesc * len(d2))(*d2), len(d2), staging.ctypes.data)
    want = np.full(1 << 20, 0x11, dtype=np.uint8)
    for a, off, n in pieces:
        want[a:a + n] = src[a:a + n]
    want[500000:504096] = 0
    assert np.array_equal(dst, want)
