"""Synthetic footprints of the benchmark configurations: region sizes, zero-chunk masks and
chunk contents, produced by the integer-only generator in csrc/footprint.c so that the CPU
oracle, the tests and the GPU benchmark all see the same bytes."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libamem_footprint.so")
CHUNK = 65536
MiB = 1 << 20

_lib = None


def build():
    os.makedirs(os.path.dirname(LIB_PATH), exist_ok=True)
    import subprocess
    cmd = ["gcc", "-O3", "-std=c11", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall",
           os.path.join(HERE, "csrc", "footprint.c"), "-o", LIB_PATH, "-lpthread"]
    subprocess.run(cmd, check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run __graft_entry__.build()" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        u64, p = C.c_uint64, C.c_void_p
        L.amem_fp_splitmix64.restype = u64
        L.amem_fp_splitmix64.argtypes = [u64]
        L.amem_fp_rng_init.argtypes = [C.POINTER(u64), u64, u64]
        L.amem_fp_next64.restype = u64
        L.amem_fp_next64.argtypes = [C.POINTER(u64)]
        L.amem_fp_next32.restype = C.c_uint32
        L.amem_fp_next32.argtypes = [C.POINTER(u64)]
        L.amem_fp_sizes.restype = u64
        L.amem_fp_sizes.argtypes = [C.c_int, u64, p, u64, u64]
        L.amem_fp_zero_mask.argtypes = [u64, u64, C.c_int, p]
        L.amem_fp_fill.argtypes = [u64, u64, u64, p, p, p, C.c_int]
        L.amem_fp_check.restype = u64
        L.amem_fp_check.argtypes = [u64, u64, u64, p, p, p, C.c_int]
        L.amem_fp_mutate.argtypes = [u64, u64, u64, u64, p, p, p]
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


class Footprint:
    """Region sizes plus per-chunk zero mask and content generation of one configuration.

    cfg 1: 64 regions of 2 MiB x U{1..16}, no zero chunks
    cfg 2: 128 x 4 MiB + 96 x 2 MiB + 32 x 16 MiB, 50 % zero chunks
    cfg 3: log-uniform [2, 64) MiB regions, 30 % zero chunks; `byte_budget` cuts the draw list
           at the shortest prefix that reaches it (the 10 GiB headline), 0 keeps all 2560
    cfg 4: 100000 sub-allocations log-uniform [4, 64) KiB, no zero chunks
    """

    ZERO_PCT = {1: 0, 2: 50, 3: 30, 4: 0}

    def __init__(self, cfg, seed, byte_budget=0, max_regions=None, threads=8):
        L = lib()
        cap = {1: 64, 2: 256, 3: 2560, 4: 100000}[cfg]
        if max_regions is not None:
            cap = min(cap, max_regions)
        sizes = np.zeros(cap, dtype=np.uint64)
        n = L.amem_fp_sizes(cfg, seed, _ptr(sizes), cap, byte_budget)
        self.cfg, self.seed, self.threads = cfg, seed, threads
        self.sizes = sizes[:n].copy()
        chunks = (self.sizes + np.uint64(CHUNK - 1)) // np.uint64(CHUNK)
        self.first_chunk = np.concatenate([[0], np.cumsum(chunks)]).astype(np.uint64)
        self.nchunks = int(self.first_chunk[-1])
        self.mask = np.zeros(max(self.nchunks, 1), dtype=np.uint8)
        if self.ZERO_PCT[cfg]:
            L.amem_fp_zero_mask(seed, self.nchunks, self.ZERO_PCT[cfg], _ptr(self.mask))
        self.gen = np.zeros(max(self.nchunks, 1), dtype=np.uint32)
        self.total_bytes = int(self.sizes.sum())

    @classmethod
    def with_sizes(cls, sizes, seed, zero_pct=30, threads=8):
        """A footprint of the given region sizes (bytes, multiples of 16) instead of a configuration's
        draw list; zero mask and contents come from the same generator, keyed by seed and chunk number."""
        self = cls.__new__(cls)
        self.cfg, self.seed, self.threads = 0, seed, threads
        self.sizes = np.array(sizes, dtype=np.uint64)
        chunks = (self.sizes + np.uint64(CHUNK - 1)) // np.uint64(CHUNK)
        self.first_chunk = np.concatenate([[0], np.cumsum(chunks)]).astype(np.uint64)
        self.nchunks = int(self.first_chunk[-1])
        self.mask = np.zeros(max(self.nchunks, 1), dtype=np.uint8)
        if zero_pct:
            lib().amem_fp_zero_mask(seed, self.nchunks, zero_pct, _ptr(self.mask))
        self.gen = np.zeros(max(self.nchunks, 1), dtype=np.uint32)
        self.total_bytes = int(self.sizes.sum())
        return self

    def region_bytes(self, i, out=None):
        """Bytes of region i as a uint8 array."""
        n = int(self.sizes[i])
        if out is None:
            out = np.empty(n, dtype=np.uint8)
        lib().amem_fp_fill(self.seed, int(self.first_chunk[i]), n, _ptr(self.mask), _ptr(self.gen), _ptr(out),
                           self.threads)
        return out[:n]

    def check_region(self, i, buf):
        """Number of bytes of `buf` that differ from region i's expected contents."""
        n = int(self.sizes[i])
        assert buf.nbytes >= n
        return int(lib().amem_fp_check(self.seed, int(self.first_chunk[i]), n, _ptr(self.mask), _ptr(self.gen),
                                       _ptr(buf), self.threads))

    def mutate(self, cycle, fraction=0.01):
        """Writes between cycles: returns the sorted, de-duplicated chunk numbers touched."""
        count = max(1, int(self.nchunks * fraction))
        touched = np.zeros(count, dtype=np.uint64)
        lib().amem_fp_mutate(self.seed, cycle, self.nchunks, count, _ptr(self.mask), _ptr(self.gen), _ptr(touched))
        return np.unique(touched)

    def chunk_region(self, c):
        """(region index, byte offset inside the region) of global chunk number c."""
        i = int(np.searchsorted(self.first_chunk, np.uint64(c), side="right") - 1)
        return i, (int(c) - int(self.first_chunk[i])) * CHUNK

    def chunk_bytes(self, c):
        i, off = self.chunk_region(c)
        n = min(CHUNK, int(self.sizes[i]) - off)
        out = np.empty(n, dtype=np.uint8)
        # a one-chunk "region" starting at global chunk c
        lib().amem_fp_fill(self.seed, int(c), n, _ptr(self.mask), _ptr(self.gen), _ptr(out), 1)
        return out

    def zero_chunks(self):
        return int(self.mask[:self.nchunks].sum())


class PackedGranules:
    """Configuration 4 as an allocator sees it: the sub-allocations of a Footprint(4, ...) bump-packed
    into 2 MiB granules (none straddles a granule; the gaps read zero). Each granule is one region.
    Offers the part of Footprint's interface that harness.Regions uses."""

    GRANULE = 2 << 20

    def __init__(self, seed=3, count=100000, threads=8):
        self.sub = Footprint(4, seed, max_regions=count, threads=threads)
        g = self.GRANULE
        sz = self.sub.sizes.astype(np.int64)
        self.starts = np.zeros(len(sz), dtype=np.int64)
        cur = 0
        for i, n in enumerate(sz):
            if cur % g + n > g:
                cur = (cur // g + 1) * g
            self.starts[i] = cur
            cur += int(n)
        self.ngranules = (cur + g - 1) // g
        self.sizes = np.full(self.ngranules, g, dtype=np.uint64)
        self.total_bytes = int(self.ngranules) * g
        self.payload_bytes = int(sz.sum())
        # sub-allocations of granule k: [first[k], first[k + 1])
        self.first = np.searchsorted(self.starts // g, np.arange(self.ngranules + 1), side="left")

    def region_bytes(self, i, out=None):
        g = self.GRANULE
        if out is None:
            out = np.empty(g, dtype=np.uint8)
        out[:g] = 0
        for s in range(int(self.first[i]), int(self.first[i + 1])):
            a = int(self.starts[s]) - i * g
            self.sub.region_bytes(s, out[a:a + int(self.sub.sizes[s])])
        return out[:g]

    def check_region(self, i, buf):
        return int(np.count_nonzero(buf[:self.GRANULE] != self.region_bytes(i)))
