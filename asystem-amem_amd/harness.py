"""Test and benchmark harness over the C ABI: builds a synthetic footprint out of real VMM
allocations, registers it through the allocator hook, and checks a pause/resume cycle.

Everything here goes through `binding.load()`; nothing is computed on the host except the
expected bytes, which come from the footprint generator.
"""
import ctypes as C
import os

import numpy as np

from . import binding as B
from .footprint import CHUNK, Footprint


def enable_env():
    """Environment the library reads at load time (amem_nccl.cpp:711-718 of the reference)."""
    os.environ.setdefault("AMEM_ENABLE", "1")
    os.environ.setdefault("GMM_LOG", "2")


class Regions:
    """A set of VMM allocations filled from a Footprint and registered with the engine."""

    def __init__(self, lib, fp, dev=0, caller=B.CALLER_P2P, register=True):
        self.lib, self.fp, self.dev = lib, fp, dev
        self.va = np.zeros(len(fp.sizes), dtype=np.uint64)
        self.handle = np.zeros(len(fp.sizes), dtype=np.uint64)
        self.alloc = np.zeros(len(fp.sizes), dtype=np.uint64)
        self.registered = False
        self._scratch = np.empty(int(fp.sizes.max()) if len(fp.sizes) else 0, dtype=np.uint8)
        for i, sz in enumerate(fp.sizes):
            va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
            rc = lib.amem_vmm_alloc(int(sz), dev, C.byref(va), C.byref(h), C.byref(asz))
            if rc != 0:
                raise RuntimeError("amem_vmm_alloc failed: %d" % rc)
            self.va[i], self.handle[i], self.alloc[i] = va.value, h.value, asz.value
        self.fill_all()
        if register:
            self.register(caller)

    def fill_all(self):
        for i in range(len(self.va)):
            buf = self.fp.region_bytes(i, self._scratch)
            rc = self.lib.amem_copy_to_device(int(self.va[i]), buf.ctypes.data_as(C.c_void_p), buf.nbytes)
            assert rc == 0
            # allocations are rounded up to 2 MiB; bytes past the requested size are cleared
            tail = int(self.alloc[i]) - buf.nbytes
            if tail:
                z = np.zeros(tail, dtype=np.uint8)
                self.lib.amem_copy_to_device(int(self.va[i]) + buf.nbytes, z.ctypes.data_as(C.c_void_p), tail)

    def write_chunks(self, chunks):
        """Write the current expected contents of the given global chunk numbers to the device."""
        for c in chunks:
            i, off = self.fp.chunk_region(int(c))
            buf = self.fp.chunk_bytes(int(c))
            rc = self.lib.amem_copy_to_device(int(self.va[i]) + off, buf.ctypes.data_as(C.c_void_p), buf.nbytes)
            assert rc == 0

    def register(self, caller=B.CALLER_P2P):
        for i in range(len(self.va)):
            rc = self.lib.amem_add_alloc_info(int(self.va[i]), int(self.alloc[i]), B.TYPE_LOCAL, self.dev,
                                              int(self.handle[i]), -1, 0, None, caller)
            if rc != 0:
                raise RuntimeError("amem_add_alloc_info rc=%d" % rc)
        self.registered = True

    def mismatched_bytes(self):
        """Read every region back and count bytes that differ from the footprint."""
        bad = 0
        for i in range(len(self.va)):
            n = int(self.fp.sizes[i])
            buf = self._scratch[:n]
            rc = self.lib.amem_copy_from_device(buf.ctypes.data_as(C.c_void_p), int(self.va[i]), n)
            if rc != 0:
                raise RuntimeError("amem_copy_from_device rc=%d" % rc)
            bad += self.fp.check_region(i, buf)
            tail = int(self.alloc[i]) - n
            if tail:
                t = np.empty(tail, dtype=np.uint8)
                self.lib.amem_copy_from_device(t.ctypes.data_as(C.c_void_p), int(self.va[i]) + n, tail)
                bad += int(np.count_nonzero(t))
        return bad

    def table(self):
        return region_table(self.lib, self.dev)

    def free(self):
        for i in range(len(self.va)):
            if self.registered:
                self.lib.amem_del_alloc_info(int(self.va[i]), 0, 0)
            self.lib.amem_vmm_free(int(self.va[i]), int(self.alloc[i]), 0)
        self.registered = False
        self.va = self.va[:0]


def region_table(lib, dev=0):
    """The registry of `dev` as {va: dict of fields}."""
    out = {}
    info = B.RegionInfo()
    for k in range(lib.amem_region_count(dev)):
        if lib.amem_region_at(dev, k, C.byref(info)) == 0:
            out[info.va] = info.as_dict()
    return out


def counters(lib):
    c = B.Counters()
    lib.amem_get_counters(C.byref(c))
    d = {k: getattr(c, k) for k, _ in c._fields_ if k != "alloc_bytes"}
    d["alloc_bytes"] = list(c.alloc_bytes)
    return d


def cycle_stats(lib):
    s = B.CycleStats()
    lib.amem_get_cycle_stats(C.byref(s))
    return s.as_dict()


def mem_free(lib):
    f, t = C.c_uint64(), C.c_uint64()
    rc = lib.amem_device_mem_info(C.byref(f), C.byref(t))
    assert rc == 0
    return f.value


# Fields of a region that a pause/resume cycle must leave unchanged (everything the
# reference's amem_allocMdata holds except the handle, amem_nccl.h:87-138).
STABLE_FIELDS = ("va", "mc_handle", "alloc_sz", "tags", "peers", "user_info", "dev", "pid", "refcount",
                 "shared_fd", "type", "state", "has_peer", "oos_flag")


def compare_tables(before, after):
    """List of differences between two region tables, keyed by VA; handles must be fresh."""
    diffs = []
    if set(before) != set(after):
        diffs.append(("keys", sorted(set(before) ^ set(after))))
    for va in before:
        if va not in after:
            continue
        a, b = before[va], after[va]
        for f in STABLE_FIELDS:
            if a[f] != b[f]:
                diffs.append((hex(va), f, a[f], b[f]))
        if b["handle"] == 0:
            diffs.append((hex(va), "handle is zero"))
        if b["type"] <= B.TYPE_LOCAL_SYMM and b["handle_gen"] != a["handle_gen"] + 1:
            diffs.append((hex(va), "handle_gen", a["handle_gen"], b["handle_gen"]))
    return diffs


def nonzero_runs(fp, vas):
    """Pack descriptors of a footprint as it stands: one {va, off, bytes} per run of non-zero 64 KiB
    chunks of each region, offsets consecutive in region order. Returns (array[n, 3] uint64, bytes)."""
    from .footprint import CHUNK
    rows, off = [], 0
    for i, va in enumerate(vas):
        c0, c1 = int(fp.first_chunk[i]), int(fp.first_chunk[i + 1])
        live = (fp.mask[c0:c1] == 0).astype(np.int8)
        edges = np.flatnonzero(np.diff(np.concatenate([[0], live, [0]])))
        size = int(fp.sizes[i])
        for a, b in zip(edges[0::2], edges[1::2]):
            start, end = int(a) * CHUNK, min(int(b) * CHUNK, size)
            rows.append((int(va) + start, off, end - start))
            off += end - start
    return np.array(rows, dtype=np.uint64).reshape(-1, 3), off
