"""Device kernels through the C ABI against the CPU oracle: bit-exact flags, checksums and
copied bytes on seeded inputs, edge cases (empty, ragged, single byte, unaligned rejects),
and size-independent properties at full benchmark size."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from asystem_amem_amd import binding as B
from asystem_amem_amd.footprint import CHUNK, Footprint

pytestmark = pytest.mark.gpu
MiB = 1 << 20


class DevBuf:
    def __init__(self, lib, nbytes):
        self.lib, self.n = lib, nbytes
        va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert lib.amem_vmm_alloc(nbytes, 0, C.byref(va), C.byref(h), C.byref(asz)) == 0
        self.va, self.handle, self.alloc = va.value, h.value, asz.value

    def put(self, arr, off=0):
        a = np.ascontiguousarray(arr).view(np.uint8)
        assert self.lib.amem_copy_to_device(self.va + off, a.ctypes.data, a.nbytes) == 0

    def get(self, n=None, off=0):
        out = np.empty(n if n is not None else self.alloc, dtype=np.uint8)
        assert self.lib.amem_copy_from_device(out.ctypes.data, self.va + off, out.nbytes) == 0
        return out

    def free(self):
        self.lib.amem_vmm_free(self.va, self.alloc, 0)


def gpu_scan(lib, extents):
    ext = (B.Extent * len(extents))(*[B.Extent(v, n) for v, n in extents])
    n = lib.amem_chunk_count(ext, len(extents))
    flags = np.full(max(n, 1), 7, dtype=np.uint8)
    sums = np.zeros((max(n, 1), 2), dtype=np.uint64)
    ms = C.c_float()
    assert lib.amem_zero_scan(ext, len(extents), flags.ctypes.data, sums.ctypes.data, C.byref(ms)) == 0
    return flags[:n], sums[:n], ms.value


def cpu_scan(orc, host):
    n = (host.nbytes + CHUNK - 1) // CHUNK
    f = np.zeros(n, dtype=np.uint8)
    s = np.zeros((n, 2), dtype=np.uint64)
    orc.oracle_zero_scan(host.ctypes.data, host.nbytes, f.ctypes.data, s.ctypes.data)
    return f, s


def test_scan_matches_oracle_on_seeded_regions(gpu, orc):
    fp = Footprint(2, 1, max_regions=12)
    bufs, host = [], []
    for i in range(len(fp.sizes)):
        b = DevBuf(gpu, int(fp.sizes[i]))
        h = fp.region_bytes(i).copy()
        b.put(h)
        bufs.append(b)
        host.append(h)
    flags, sums, _ = gpu_scan(gpu, [(b.va, int(fp.sizes[i])) for i, b in enumerate(bufs)])
    c0 = 0
    for h in host:
        f, s = cpu_scan(orc, h)
        assert np.array_equal(flags[c0:c0 + len(f)], f)
        assert np.array_equal(sums[c0:c0 + len(f)], s)
        c0 += len(f)
    assert c0 == len(flags)
    assert np.array_equal(flags, fp.mask[:fp.nchunks])          # the generator's zero mask, seen from the GPU
    for b in bufs:
        b.free()


def test_scan_edge_cases(gpu, orc):
    b = DevBuf(gpu, 2 * MiB)
    host = np.zeros(2 * MiB, dtype=np.uint8)
    host[0] = 1                      # first byte of chunk 0
    host[2 * CHUNK - 1] = 0x80       # last byte of chunk 1
    host[3 * CHUNK + 4:3 * CHUNK + 8] = [0xEF, 0xBE, 0xAD, 0xDE]   # one word at odd index in chunk 3
    host[5 * CHUNK:6 * CHUNK].view(np.uint64)[[3, 900]] = 0x0123456789ABCDEF  # xor cancels, sum does not
    host[6 * CHUNK:7 * CHUNK] = 0xFF                                 # largest sum
    b.put(host)
    flags, sums, _ = gpu_scan(gpu, [(b.va, 2 * MiB)])
    f, s = cpu_scan(orc, host)
    assert np.array_equal(flags, f) and np.array_equal(sums, s)
    assert list(flags[:8]) == [0, 0, 1, 0, 1, 0, 0, 1]
    assert int(sums[3, 0]) == 0xDEADBEEF and int(sums[3, 1]) == 0xDEADBEEF << 32
    assert int(sums[5, 1]) == 0 and int(sums[5, 0]) == 2 * (0x01234567 + 0x89ABCDEF)
    assert int(sums[6, 0]) == 0xFFFFFFFF * (CHUNK // 4)
    # ragged: extents that are not chunk multiples, starting mid-buffer, plus an empty one
    ext = [(b.va + 16, 48), (b.va + CHUNK, CHUNK + 4096), (b.va + 3 * CHUNK, 0), (b.va + 6 * CHUNK - 32, 64)]
    flags, sums, _ = gpu_scan(gpu, ext)
    want_f, want_s = [], []
    for va, n in ext:
        if n == 0:
            continue
        ff, ss = cpu_scan(orc, host[va - b.va:va - b.va + n].copy())
        want_f += list(ff)
        want_s += [tuple(x) for x in ss]
    assert list(flags) == want_f and [tuple(x) for x in sums] == want_s
    assert len(flags) == 1 + 2 + 0 + 1
    # nothing to scan
    flags, sums, _ = gpu_scan(gpu, [])
    assert len(flags) == 0
    # misaligned input is rejected, not scanned
    bad = (B.Extent * 1)(B.Extent(b.va + 8, 64))
    one = (C.c_uint8 * 1)()
    assert gpu.amem_zero_scan(bad, 1, one, None, None) != 0
    bad = (B.Extent * 1)(B.Extent(b.va, 24))
    assert gpu.amem_zero_scan(bad, 1, one, None, None) != 0
    b.free()


def _descs(pairs):
    return (B.CopyDesc * len(pairs))(*[B.CopyDesc(v, o, n) for v, o, n in pairs])


@pytest.mark.parametrize("host_side", [0, 1])
def test_pack_unpack_match_oracle(gpu, orc, host_side):
    rng = np.random.default_rng(3)
    src = DevBuf(gpu, 8 * MiB)
    data = rng.integers(0, 256, 8 * MiB, dtype=np.uint8)
    src.put(data)
    # ragged descriptor list: 16-byte pieces, pieces crossing tile and chunk boundaries, an empty one
    pieces, off = [], 0
    for a, n in [(0, 16), (4096 + 16, 16368), (65536 - 32, 64), (1 * MiB, 3 * 16384 + 48), (5 * MiB + 256, 700000 - 700000 % 16),
                 (7 * MiB, 0), (2 * MiB, 1 * MiB)]:
        pieces.append((a, off, n))
        off += n + 32            # leave gaps in staging: they must stay untouched
    total = off
    if host_side:
        # pinned host memory straight from the HIP runtime the library is linked against
        hip = C.CDLL("libamdhip64.so")
        hip.hipHostMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.c_uint]
        hip.hipHostFree.argtypes = [C.c_void_p]
        pinned = C.c_void_p()
        assert hip.hipHostMalloc(C.byref(pinned), total, 0) == 0
        stage_ptr = pinned.value
        stage_np = np.frombuffer((C.c_uint8 * total).from_address(stage_ptr), dtype=np.uint8)
        stage_np[:] = 0xCC
    else:
        stage = DevBuf(gpu, total)
        stage.put(np.full(stage.alloc, 0xCC, dtype=np.uint8))
        stage_ptr = stage.va
    ms = C.c_float()
    rc = gpu.amem_gather_pack(_descs([(src.va + a, o, n) for a, o, n in pieces]), len(pieces), stage_ptr, total,
                              host_side, C.byref(ms))
    assert rc == 0
    got = stage_np.copy() if host_side else stage.get(total)
    want = np.full(total, 0xCC, dtype=np.uint8)
    od = (O.CopyDesc * len(pieces))(*[O.CopyDesc(data.ctypes.data + a, o, n) for a, o, n in pieces])
    orc.oracle_gather_pack(od, len(pieces), want.ctypes.data)
    assert np.array_equal(got, want)
    # scatter into a second buffer, with zero-fill descriptors
    dst = DevBuf(gpu, 8 * MiB)
    dst.put(np.full(8 * MiB, 0x11, dtype=np.uint8))
    sc = [(dst.va + a, o, n) for a, o, n in pieces] + [(dst.va + 6 * MiB, B.DESC_ZERO, 65536 + 16), (dst.va + 4 * MiB, B.DESC_ZERO, 16)]
    assert gpu.amem_scatter_unpack(_descs(sc), len(sc), stage_ptr, total, host_side, C.byref(ms)) == 0
    want_dst = np.full(8 * MiB, 0x11, dtype=np.uint8)
    osc = [O.CopyDesc(want_dst.ctypes.data + a, o, n) for a, o, n in pieces] + \
          [O.CopyDesc(want_dst.ctypes.data + 6 * MiB, O.DESC_ZERO, 65536 + 16), O.CopyDesc(want_dst.ctypes.data + 4 * MiB, O.DESC_ZERO, 16)]
    orc.oracle_scatter_unpack((O.CopyDesc * len(osc))(*osc), len(osc), want.ctypes.data)
    assert np.array_equal(dst.get(8 * MiB), want_dst)
    # rejected inputs: misaligned, out of staging bounds, zero-fill on gather
    assert gpu.amem_gather_pack(_descs([(src.va + 8, 0, 16)]), 1, stage_ptr, total, host_side, None) != 0
    assert gpu.amem_gather_pack(_descs([(src.va, total - 16, 32)]), 1, stage_ptr, total, host_side, None) != 0
    assert gpu.amem_gather_pack(_descs([(src.va, B.DESC_ZERO, 32)]), 1, stage_ptr, total, host_side, None) != 0
    assert gpu.amem_gather_pack(_descs([]), 0, stage_ptr, total, host_side, None) == 0
    src.free(); dst.free()
    if host_side:
        del stage_np
        assert hip.hipHostFree(pinned) == 0
    else:
        stage.free()


@pytest.mark.parametrize("count", [2000, 100000])
def test_fragmented_descriptor_list_round_trip(gpu, orc, count, measured):
    """benchmark configuration 4 (100,000 sub-allocations of 4-64 KiB bump-packed into 2 MiB granules, seed 3;
    also at 1/50 scale): gathered into contiguous staging and scattered back into fresh memory."""
    fp = Footprint(4, 3, max_regions=count, threads=16)
    granule = 2 * MiB
    sizes = fp.sizes.astype(np.int64)
    starts = np.zeros(len(sizes), dtype=np.int64)
    cur = 0
    for i, sz in enumerate(sizes):                       # bump allocation, no sub-allocation straddles a granule
        if cur % granule + sz > granule:
            cur = (cur // granule + 1) * granule
        starts[i] = cur
        cur += sz
    total = int((cur + granule - 1) // granule * granule)
    src, dst = DevBuf(gpu, total), DevBuf(gpu, total)
    host = np.zeros(total, dtype=np.uint8)
    for i in range(len(sizes)):
        fp.region_bytes(i, host[starts[i]:starts[i] + sizes[i]])
    src.put(host)
    dst.put(np.full(total, 0x77, dtype=np.uint8))
    packed = int(sizes.sum())
    stage = DevBuf(gpu, packed)
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    garr = np.empty((len(sizes), 3), dtype=np.uint64)
    garr[:, 0] = src.va + starts
    garr[:, 1] = offs[:-1]
    garr[:, 2] = sizes
    ms = C.c_float()
    assert gpu.amem_gather_pack(garr.ctypes.data_as(C.POINTER(B.CopyDesc)), len(sizes), stage.va, packed, 0, C.byref(ms)) == 0
    gather_ms = ms.value
    live = np.zeros(total, dtype=bool)
    idx = np.concatenate([np.arange(a, a + n) for a, n in zip(starts[:4000], sizes[:4000])])   # spot-check layout
    got = stage.get(packed)
    assert np.array_equal(got[:len(idx)], host[idx])
    for a, n in zip(starts, sizes):
        live[a:a + n] = True
    assert np.array_equal(got, host[live])              # packed order == address order for a bump allocator
    sarr = garr.copy()
    sarr[:, 0] = dst.va + starts
    assert gpu.amem_scatter_unpack(sarr.ctypes.data_as(C.POINTER(B.CopyDesc)), len(sizes), stage.va, packed, 0, C.byref(ms)) == 0
    back = dst.get(total)
    assert np.array_equal(back[live], host[live]) and (back[~live] == 0x77).all()
    if count == 100000:
        measured("config 4's %d sub-allocations as one descriptor each, %.2f GB packed: gather %.2f ms = %.2f TB/s, scatter %.2f ms "
                 "= %.2f TB/s (S read + S written; first launches)" % (len(sizes), packed / 1e9, gather_ms, 2 * packed / gather_ms / 1e9,
                                                                      ms.value, 2 * packed / ms.value / 1e9))
    src.free(); dst.free(); stage.free()


def test_scan_properties_at_benchmark_size(gpu):
    """2 GiB in one launch: flags equal the generator's mask; checksum of checksums is
    unchanged by a gather + scatter round trip through device staging."""
    fp = Footprint(3, 2, byte_budget=2 << 30, threads=16)
    bufs = []
    for i in range(len(fp.sizes)):
        b = DevBuf(gpu, int(fp.sizes[i]))
        b.put(fp.region_bytes(i))
        bufs.append(b)
    ext = [(b.va, int(fp.sizes[i])) for i, b in enumerate(bufs)]
    flags, sums, ms = gpu_scan(gpu, ext)
    assert np.array_equal(flags, fp.mask[:fp.nchunks])
    assert (sums[flags == 1] == 0).all() and (sums[flags == 0, 0] != 0).all()
    total = int(fp.sizes.sum())
    stage = DevBuf(gpu, total)
    offs = np.concatenate([[0], np.cumsum(fp.sizes)]).astype(np.uint64)
    g = _descs([(b.va, int(offs[i]), int(fp.sizes[i])) for i, b in enumerate(bufs)])
    assert gpu.amem_gather_pack(g, len(bufs), stage.va, total, 0, None) == 0
    f2, s2, _ = gpu_scan(gpu, [(stage.va, total)])
    assert np.array_equal(f2, flags) and np.array_equal(s2, sums)     # packing moved chunks, not bits
    for b in bufs:
        b.put(np.full(b.alloc, 0x5A, dtype=np.uint8))
    assert gpu.amem_scatter_unpack(g, len(bufs), stage.va, total, 0, None) == 0
    f3, s3, _ = gpu_scan(gpu, ext)
    assert np.array_equal(f3, flags) and np.array_equal(s3, sums)
    assert ms > 0 and total / (ms * 1e-3) / 1e9 > 500                  # sanity: far above any host-side rate
    for b in bufs:
        b.free()
    stage.free()
