"""The synthetic footprint generator against an independent pure-Python restatement of its
RNG, and against the totals the benchmark configurations are specified with."""
import numpy as np

from asystem_amem_amd import footprint as F

M64 = (1 << 64) - 1


def splitmix64(x):
    x = (x + 0x9E3779B97F4A7C15) & M64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & M64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & M64
    return x ^ (x >> 31)


class XorShift:
    def __init__(self, state):
        self.s = state or 1

    def next64(self):
        x = self.s
        x ^= (x << 13) & M64
        x ^= x >> 7
        x ^= (x << 17) & M64
        self.s = x
        return x

    def next32(self):
        return self.next64() >> 32


def test_splitmix_known_answers():
    # first outputs of splitmix64 seeded with 0 (published test vector of the algorithm)
    L = F.lib()
    assert L.amem_fp_splitmix64(0) == 0xE220A8397B1DCDAF
    assert L.amem_fp_splitmix64(0x9E3779B97F4A7C15) == 0x6E789E6AA1B965F4


def test_xorshift_matches_python():
    import ctypes as C
    L = F.lib()
    st = C.c_uint64()
    L.amem_fp_rng_init(C.byref(st), 5, 2)
    py = XorShift(splitmix64(5 * 4 + 2))
    assert st.value == py.s
    for _ in range(100):
        assert L.amem_fp_next64(C.byref(st)) == py.next64()
    a = L.amem_fp_next32(C.byref(st))
    assert a == py.next32()


def test_config_sizes():
    MiB = 1 << 20
    f1 = F.Footprint(1, 0)
    r = XorShift(splitmix64(0))
    assert [int(s) for s in f1.sizes] == [2 * MiB * (1 + r.next32() % 16) for _ in range(64)]
    f2 = F.Footprint(2, 1)
    assert len(f2.sizes) == 256 and f2.total_bytes == 1216 * MiB  # 128x4 + 96x2 + 32x16 MiB
    f3 = F.Footprint(3, 2, byte_budget=10 << 30)
    assert f3.total_bytes >= 10 << 30 and f3.total_bytes - int(f3.sizes[-1]) < 10 << 30
    assert all(2 * MiB <= int(s) < 64 * MiB and int(s) % (2 * MiB) == 0 for s in f3.sizes)
    f3all = F.Footprint(3, 2)
    assert len(f3all.sizes) == 2560 and np.array_equal(f3all.sizes[:len(f3.sizes)], f3.sizes)
    f4 = F.Footprint(4, 3)
    assert len(f4.sizes) == 100000
    assert all(4096 <= int(s) < 65536 and int(s) % 4096 == 0 for s in f4.sizes[:2000])


def test_zero_mask_fraction_and_contents():
    f2 = F.Footprint(2, 1)
    frac = f2.zero_chunks() / f2.nchunks
    assert 0.48 < frac < 0.52
    r = XorShift(splitmix64(1 * 4 + 1))
    assert [int(r.next32() % 100 < 50) for _ in range(200)] == [int(m) for m in f2.mask[:200]]
    # region bytes: zero chunks are zero, others match the per-chunk stream
    b = f2.region_bytes(0).reshape(-1, F.CHUNK)
    key = splitmix64(1 * 4 + 2)
    for k in range(4):
        if f2.mask[k]:
            assert not b[k].any()
        else:
            st = XorShift(splitmix64((key + k * 0x9E3779B97F4A7C15) & M64))
            words = np.array([st.next64() for _ in range(16)], dtype=np.uint64)
            assert np.array_equal(b[k][:128].view(np.uint64), words)
    assert f2.check_region(0, b.reshape(-1)) == 0
    b2 = b.reshape(-1).copy()
    b2[12345] ^= 0xFF
    assert f2.check_region(0, b2) == 1


def test_mutation_changes_both_ways():
    f = F.Footprint(2, 1, max_regions=16)
    before_mask = f.mask.copy()
    before = [f.chunk_bytes(c).copy() for c in range(f.nchunks)]
    touched = f.mutate(0, fraction=0.2)
    to_zero = [c for c in touched if not before_mask[c] and f.mask[c]]
    from_zero = [c for c in touched if before_mask[c] and not f.mask[c]]
    assert to_zero and from_zero
    for c in range(f.nchunks):
        same = np.array_equal(before[c], f.chunk_bytes(c))
        assert same == (c not in set(int(t) for t in touched)) or (before_mask[c] and f.mask[c])


def test_packed_granules_layout():
    """Configuration 4's sub-allocations inside 2 MiB granules: none straddles a granule, every byte of a
    granule is either the sub-allocation's own stream or a zero gap, and the check finds a flipped byte."""
    pg = F.PackedGranules(3, 400, threads=2)
    g = pg.GRANULE
    ends = pg.starts + pg.sub.sizes.astype(np.int64)
    assert (pg.starts // g == (ends - 1) // g).all() and (pg.starts[1:] >= ends[:-1]).all()
    assert pg.ngranules == ends[-1] // g + (ends[-1] % g != 0) and pg.payload_bytes == int(pg.sub.sizes.sum())
    k = pg.ngranules // 2
    img = pg.region_bytes(k).copy()
    live = np.zeros(g, dtype=bool)
    for s in range(int(pg.first[k]), int(pg.first[k + 1])):
        a, n = int(pg.starts[s]) - k * g, int(pg.sub.sizes[s])
        assert np.array_equal(img[a:a + n], pg.sub.region_bytes(s))
        live[a:a + n] = True
    assert int(pg.first[k + 1]) > int(pg.first[k]) and not img[~live].any()
    assert pg.check_region(k, img) == 0
    img[12345] ^= 1
    assert pg.check_region(k, img) == 1
