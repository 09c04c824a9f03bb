"""amem_zero_scan_noalloc, the scan entry point that allocates nothing: the tables its kernel needs live
in a fixed device array of the library instead of growable buffers. Called through the C ABI and held to
the results of amem_zero_scan (and, for one region, of the CPU oracle), bit for bit, on two calls in a
row of which the second is smaller, so that what the first call left in the shared array would show."""
import ctypes as C

import numpy as np
import pytest

from asystem_amem_amd import binding as B
from asystem_amem_amd import harness as H
from asystem_amem_amd.footprint import CHUNK, Footprint

pytestmark = pytest.mark.gpu
MiB = 1 << 20


def _extents(pairs):
    return (B.Extent * len(pairs))(*[B.Extent(int(v), int(b)) for v, b in pairs])


def _scan(fn, pairs, want_sums=True):
    ext = _extents(pairs)
    n = sum((int(b) + CHUNK - 1) // CHUNK for _, b in pairs)
    flags = np.full(n, 0xEE, dtype=np.uint8)
    sums = np.full((n, 2), 0xEEEEEEEEEEEEEEEE, dtype=np.uint64)
    ms = C.c_float(-1)
    rc = fn(ext, len(pairs), flags.ctypes.data, sums.ctypes.data if want_sums else None, C.byref(ms))
    return rc, flags, sums, ms.value


def test_scan_without_allocation_equals_the_allocating_scan(gpu, fresh, orc):
    lib = fresh
    fp = Footprint(2, 21, max_regions=24, threads=4)       # 4 MiB regions, half of the chunks zero
    regs = H.Regions(lib, fp, register=False)
    try:
        big = [(regs.va[i], regs.alloc[i]) for i in range(len(regs.va))]
        # smaller and ragged: fewer extents, one starting inside a region, one ending inside a chunk
        small = [(regs.va[3], 2 * MiB), (regs.va[7] + 3 * CHUNK + 4096, 5 * CHUNK + 160), (regs.va[1], CHUNK)]
        rc, f_ref, s_ref, _ = _scan(lib.amem_zero_scan, big)
        assert rc == 0
        rc, f_ref2, s_ref2, _ = _scan(lib.amem_zero_scan, small)
        assert rc == 0
        assert 0 < int(f_ref.sum()) < len(f_ref)            # both kinds of chunk are present
        rc, f1, s1, ms1 = _scan(lib.amem_zero_scan_noalloc, big)
        assert rc == 0 and ms1 > 0
        assert np.array_equal(f1, f_ref) and np.array_equal(s1, s_ref)
        free0 = H.mem_free(lib)                             # set-up and the runtime's own first-use work are over
        rc, f2, s2, _ = _scan(lib.amem_zero_scan_noalloc, small)          # the second call, smaller
        assert rc == 0
        assert np.array_equal(f2, f_ref2) and np.array_equal(s2, s_ref2)
        rc, f3, s3, _ = _scan(lib.amem_zero_scan_noalloc, big)            # and the large one again
        assert rc == 0 and np.array_equal(f3, f_ref) and np.array_equal(s3, s_ref)
        rc, f4, s4, _ = _scan(lib.amem_zero_scan_noalloc, small, want_sums=False)   # flags only
        assert rc == 0 and np.array_equal(f4, f_ref2) and (s4 == 0xEEEEEEEEEEEEEEEE).all()
        assert H.mem_free(lib) == free0                     # no device memory came or went
        # the oracle's scan of the same bytes (region 0)
        n0 = int(fp.sizes[0])
        host = np.ascontiguousarray(fp.region_bytes(0))
        of = np.zeros(n0 // CHUNK, dtype=np.uint8)
        osum = np.zeros((n0 // CHUNK, 2), dtype=np.uint64)
        orc.oracle_zero_scan(host.ctypes.data, n0, of.ctypes.data, osum.ctypes.data)
        assert np.array_equal(of, f1[:n0 // CHUNK]) and np.array_equal(osum, s1[:n0 // CHUNK])
        # nothing to scan
        assert lib.amem_zero_scan_noalloc(_extents(big), 0, None, None, None) == 0
    finally:
        regs.free()


def test_scan_without_allocation_rejects_what_its_fixed_tables_cannot_hold(gpu, fresh, capfd):
    lib = fresh
    va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
    assert lib.amem_vmm_alloc(64 * MiB, 0, C.byref(va), C.byref(h), C.byref(asz)) == 0
    try:
        per = 64 * MiB // CHUNK
        too_many_chunks = [(va.value, 64 * MiB)] * (B.NOALLOC_MAX_CHUNKS // per + 1)
        too_many_extents = [(va.value, CHUNK)] * (B.NOALLOC_MAX_EXTENTS + 1)
        for pairs, word in ((too_many_chunks, "chunks"), (too_many_extents, "extents")):
            capfd.readouterr()
            rc, flags, _, _ = _scan(lib.amem_zero_scan_noalloc, pairs)
            assert rc == 1 and (flags == 0xEE).all()        # refused before anything ran
            out = capfd.readouterr().out
            assert "at most" in out and word in out         # the error names the limit that was hit
        # exactly at the limit it runs, and agrees with the allocating scan
        at_limit = [(va.value, 64 * MiB)] * (B.NOALLOC_MAX_CHUNKS // per)
        rc, f1, s1, _ = _scan(lib.amem_zero_scan_noalloc, at_limit)
        rc2, f2, s2, _ = _scan(lib.amem_zero_scan, at_limit)
        assert rc == 0 and rc2 == 0 and np.array_equal(f1, f2) and np.array_equal(s1, s2)
        # misaligned input is refused like amem_zero_scan refuses it
        assert _scan(lib.amem_zero_scan_noalloc, [(va.value + 8, CHUNK)])[0] == 1
    finally:
        lib.amem_vmm_free(va.value, asz.value, h.value)
