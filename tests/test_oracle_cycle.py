"""The oracle's pause/resume on its host-memory VMM stand-in: identity of bytes, same VA,
table and counter closed forms (reference amem_nccl.cpp:467-677), physical release, and
the cross-process bookkeeping with simulated processes."""
import ctypes as C
import json
import os

import numpy as np

import oracle as O
from asystem_amem_amd.footprint import Footprint

HERE = os.path.dirname(os.path.abspath(__file__))
MiB = 1 << 20
LOCAL, PEER = 0, 3
ST_ALLOC, ST_HOLE = 1, 3


def view(va, n):
    return np.frombuffer((C.c_uint8 * n).from_address(va), dtype=np.uint8)


def alloc(orc, nbytes):
    va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
    assert orc.oracle_vmm_alloc(nbytes, C.byref(va), C.byref(h), C.byref(asz)) == 0
    return va.value, h.value, asz.value


def make_local(orc, ctx, fp, caller=1):
    regs = []
    for i, sz in enumerate(fp.sizes):
        va, h, asz = alloc(orc, int(sz))
        view(va, int(sz))[:] = fp.region_bytes(i)
        assert orc.oracle_add_alloc_info(ctx, va, asz, LOCAL, 0, h, -1, 0, 0, caller) == 0
        regs.append((va, h, asz))
    return regs


def test_config1_cycle_identity_table_and_release(fresh_orc):
    """benchmark configuration 1 at its full size (64 regions of 2 MiB x U{1..16}, seed 0, about 1 GiB):
    host-memcpy pause to a host buffer then restore; byte compare plus region-table compare."""
    orc = fresh_orc
    fp = Footprint(1, 0)
    assert len(fp.sizes) == 64
    live0 = orc.oracle_vmm_live_bytes()
    regs = make_local(orc, 0, fp)
    assert orc.oracle_vmm_live_bytes() - live0 == fp.total_bytes
    before = O.region_table(orc, 0)
    assert orc.oracle_mem_pause(0) == 0
    # post-conditions of amem_memPause: every entry HOLE, handle 0, not in handleTable, memory gone
    c = O.counters(orc, 0)
    assert (c["paused"], c["pause_cnt"], c["offload_cnt"], c["release_local_cnt"], c["release_shadow_cnt"],
            c["handle_count"]) == (1, 1, 64, 0, 0, 0)
    assert orc.oracle_check_paused(0) == 1                                                  # the gate, amem_nccl.cpp:452-464
    assert orc.oracle_vmm_live_bytes() == live0
    for va, t in O.region_table(orc, 0).items():
        assert t["state"] == ST_HOLE and t["handle"] == 0 and t["cpu_addr"] != 0
    assert orc.oracle_mem_pause(0) == 0 and O.counters(orc, 0)["pause_cnt"] == 1          # idempotent (:483-485)
    assert orc.oracle_add_alloc_info(0, 0x1234000, 2 * MiB, LOCAL, 0, 5, -1, 0, 0, 1) == 1  # :133-137
    assert orc.oracle_mem_resume(0) == 0
    after = O.region_table(orc, 0)
    c = O.counters(orc, 0)
    assert (c["paused"], c["resume_cnt"], c["offload_cnt"], c["handle_count"]) == (0, 1, 0, 64)
    assert orc.oracle_check_paused(0) == 0
    assert orc.oracle_mem_resume(0) == 0 and O.counters(orc, 0)["resume_cnt"] == 1         # idempotent (:591-593)
    assert set(after) == set(before)
    for va in before:
        a, b = before[va], after[va]
        for f in ("alloc_sz", "tags", "type", "state", "refcount", "peers", "has_peer", "oos_flag", "user_info", "dev", "pid"):
            assert a[f] == b[f], f
        assert b["handle"] not in (0, a["handle"])
        assert orc.oracle_handle_lookup(0, 0, b["handle"]) == va and orc.oracle_handle_lookup(0, 0, a["handle"]) == 0
    for i, (va, h, asz) in enumerate(regs):           # same VA, same bytes
        assert fp.check_region(i, view(va, int(fp.sizes[i]))) == 0
    cpu1 = {va: t["cpu_addr"] for va, t in after.items()}
    orc.oracle_mem_pause(0); orc.oracle_mem_resume(0)
    assert {va: t["cpu_addr"] for va, t in O.region_table(orc, 0).items()} == cpu1  # host buffers are kept (:505-508)


def test_threaded_copy_is_identical(fresh_orc):
    orc = fresh_orc
    fp = Footprint(1, 0, max_regions=8)
    regs = make_local(orc, 0, fp)
    assert orc.oracle_mem_pause_mt(0, 4) == 0 and orc.oracle_mem_resume_mt(0, 4) == 0
    for i, (va, h, asz) in enumerate(regs):
        assert fp.check_region(i, view(va, int(fp.sizes[i]))) == 0


def test_refcount_extra_releases(fresh_orc):
    """amem_cuMemReleaseHandle drops `refcount` extra references (amem_nccl.h:154-158): memory
    that a caller retained twice more is freed by pause only when amem_addRefcount told it so."""
    orc = fresh_orc
    live0 = orc.oracle_vmm_live_bytes()
    va, h, asz = alloc(orc, 2 * MiB)
    orc.oracle_add_alloc_info(0, va, asz, LOCAL, 0, h, -1, 0, 0, 1)
    assert orc.oracle_vmm_retain(va) == h and orc.oracle_vmm_retain(va) == h
    orc.oracle_mem_pause(0)
    assert orc.oracle_vmm_live_bytes() - live0 == asz      # two references outlive the pause
    orc.oracle_mem_resume(0)
    assert orc.oracle_vmm_live_bytes() - live0 == 2 * asz  # the old memory plus the new
    assert orc.oracle_vmm_retain(va) and orc.oracle_vmm_retain(va)
    assert orc.oracle_add_refcount(0, va, 2) == 0
    orc.oracle_mem_pause(0)
    assert orc.oracle_vmm_live_bytes() - live0 == asz      # the new memory is gone, the leaked old one stays
    orc.oracle_mem_resume(0)


def test_two_process_refcounted_release_and_remap(fresh_orc):
    """Owner (context 0) exports a region, importer (context 1) maps it. Pause: the
    importer drops its mapping first, the owner's release then frees the memory. Resume: the
    owner re-creates and re-exports, the importer maps the new memory at its original VA."""
    orc = fresh_orc
    live0 = orc.oracle_vmm_live_bytes()
    va, h, asz = alloc(orc, 4 * MiB)
    view(va, asz)[:] = np.arange(asz, dtype=np.uint64).view(np.uint8)[:asz]
    assert orc.oracle_add_alloc_info(0, va, asz, LOCAL, 0, h, -1, 0, 0, 1) == 0
    fd = C.c_int()
    assert orc.oracle_vmm_export(h, C.byref(fd)) == 0
    pva, ph = C.c_uint64(), C.c_uint64()
    assert orc.oracle_vmm_import(fd.value, asz, C.byref(pva), C.byref(ph)) == 0
    os.close(fd.value)
    assert orc.oracle_add_alloc_info(1, pva.value, asz, PEER, 0, ph.value, 0, h, 0, 7) == 0
    assert np.array_equal(view(pva.value, 4096), view(va, 4096))
    # owner pauses alone: the importer still holds the memory
    assert orc.oracle_mem_pause(0) == 0
    assert orc.oracle_vmm_live_bytes() - live0 == asz
    assert O.counters(orc, 0)["release_local_cnt"] == 1
    # importer pauses: last reference gone
    assert orc.oracle_mem_pause(1) == 0
    assert orc.oracle_vmm_live_bytes() == live0
    c1 = O.counters(orc, 1)
    assert (c1["release_shadow_cnt"], c1["offload_cnt"]) == (1, 0)
    assert O.region_table(orc, 1)[pva.value]["state"] == ST_HOLE
    # importer resumes first: must wait for the owner (amem_nccl.cpp:659-662)
    assert orc.oracle_mem_resume(1) == 2 and O.counters(orc, 1)["paused"] == 1
    assert orc.oracle_mem_resume(0) == 0
    c0 = O.counters(orc, 0)
    assert (c0["release_local_cnt"], c0["offload_cnt"], c0["paused"]) == (0, 0, 0)
    assert orc.oracle_mem_resume(1) == 0
    c1 = O.counters(orc, 1)
    assert (c1["release_shadow_cnt"], c1["paused"], c1["resume_cnt"]) == (0, 0, 1)
    assert O.region_table(orc, 1)[pva.value]["state"] == ST_ALLOC
    expect = np.arange(asz, dtype=np.uint64).view(np.uint8)[:asz]
    assert np.array_equal(view(va, asz), expect) and np.array_equal(view(pva.value, asz), expect)
    view(va, 8)[:] = 0xEE                       # still one physical memory behind both addresses
    assert (view(pva.value, 8) == 0xEE).all()


def test_counters_match_published_log_line(fresh_orc):
    """The one pause log the reference publishes (8 ranks, docs/images/run_result.webp) reads
    offload:549 releaseLocal:448 releasePeer:448. Rebuild that rank's table shape: 549 local
    regions of which 64 are imported by each of the 7 other ranks, and 64 regions imported
    from each of those 7 ranks; the counters then follow from amem_nccl.cpp:511, :524, :547-550."""
    orc = fresh_orc
    g = json.load(open(os.path.join(HERE, "golden", "run_result_counters.json")))
    me, others = 0, list(range(1, 8))
    nlocal, nshared = g["offload"], g["releaseLocal"] // 7
    my_regs = []
    for k in range(nlocal):
        va, h, asz = alloc(orc, 2 * MiB)
        assert orc.oracle_add_alloc_info(me, va, asz, LOCAL, 0, h, -1, 0, 0, 1) == 0
        my_regs.append((va, h, asz))
    for o in others:
        # this rank's first `nshared` regions are imported by rank o ...
        for k in range(nshared):
            va, h, asz = my_regs[k]
            assert orc.oracle_add_alloc_info(o, 0x700000000000 + (o << 36) + (k << 24), asz, PEER, 0, 0xF000 + k, me, h, 0, 7) == 0
        # ... and rank o owns `nshared` regions that this rank imports
        for k in range(nshared):
            ova, oh, oasz = alloc(orc, 2 * MiB)
            assert orc.oracle_add_alloc_info(o, ova, oasz, LOCAL, 0, oh, -1, 0, 0, 1) == 0
            fd = C.c_int()
            orc.oracle_vmm_export(oh, C.byref(fd))
            pva, ph = C.c_uint64(), C.c_uint64()
            orc.oracle_vmm_import(fd.value, oasz, C.byref(pva), C.byref(ph))
            os.close(fd.value)
            assert orc.oracle_add_alloc_info(me, pva.value, oasz, PEER, 0, ph.value, o, oh, 0, 7) == 0
    # rank 0's importers hold fake mappings, so only rank 0 is paused here
    assert orc.oracle_mem_pause(me) == 0
    c = O.counters(orc, me)
    assert (c["offload_cnt"], c["release_local_cnt"], c["release_shadow_cnt"]) == \
        (g["offload"], g["releaseLocal"], g["releasePeer"])


def test_config5_layout_four_processes(fresh_orc):
    """benchmark configuration 5 at a quarter of its size: four simulated processes (seeds 4-7), each
    owning the first 64 regions of configuration 2's layout, exporting every one of them and importing
    all 192 regions of the other three. Coordinated pause and resume; every importer then reads the
    owner's bytes at its original address. Counter closed forms from amem_nccl.cpp:511 (offload per
    local region), :524 (releasePeer per import), :547-550 (releaseLocal per recorded importer)."""
    orc = fresh_orc
    live0 = orc.oracle_vmm_live_bytes()
    P, N = 4, 64
    fps = [Footprint(2, 4 + p, max_regions=N, threads=4) for p in range(P)]
    own = [make_local(orc, p, fps[p]) for p in range(P)]
    imports = {p: [] for p in range(P)}                      # importer -> (owner, region index, address)
    for o in range(P):
        for i, (va, h, asz) in enumerate(own[o]):
            fd = C.c_int()
            assert orc.oracle_vmm_export(h, C.byref(fd)) == 0
            for q in range(P):
                if q == o:
                    continue
                pva, ph = C.c_uint64(), C.c_uint64()
                assert orc.oracle_vmm_import(fd.value, asz, C.byref(pva), C.byref(ph)) == 0
                assert orc.oracle_add_alloc_info(q, pva.value, asz, PEER, 0, ph.value, o, h, 0, 7) == 0
                imports[q].append((o, i, pva.value))
            os.close(fd.value)
    total = sum(fp.total_bytes for fp in fps)
    # the stand-in counts what every handle holds: one handle per owner and one per import
    assert orc.oracle_vmm_live_bytes() - live0 == P * total
    for p in range(P):
        assert len(O.region_table(orc, p)) == N + 3 * N
        t = O.region_table(orc, p)[own[p][0][0]]
        assert t["has_peer"] == 1 and sum(1 for x in t["peers"] if x) == 3
    # everybody pauses; memory is only gone once the last importer has let go
    for p in range(P):
        assert orc.oracle_mem_pause(p) == 0
        c = O.counters(orc, p)
        assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"]) == (N, 3 * N, 3 * N)
    assert orc.oracle_vmm_live_bytes() == live0
    # an importer that resumes before its owners has to wait (amem_nccl.cpp:659-662) ...
    assert orc.oracle_mem_resume(3) == 2
    # ... owners re-create and re-export in any order; each resume serves the importers on record
    for p in (1, 0, 2):
        rc = orc.oracle_mem_resume(p)
        assert rc in (0, 2)                                   # 2 while some of p's own imports still wait
    for p in range(P):
        assert orc.oracle_mem_resume(p) == 0                  # idempotent once complete
        c = O.counters(orc, p)
        assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"], c["paused"]) == (0, 0, 0, 0)
    assert orc.oracle_vmm_live_bytes() - live0 == P * total
    for p in range(P):
        for i, (va, h, asz) in enumerate(own[p]):
            assert fps[p].check_region(i, view(va, int(fps[p].sizes[i]))) == 0
        for o, i, pva in imports[p]:
            assert fps[o].check_region(i, view(pva, int(fps[o].sizes[i]))) == 0
    view(own[2][5][0], 8)[:] = 0xC3                           # still shared memory behind all four addresses
    for q in (0, 1, 3):
        pva = [a for (o, i, a) in imports[q] if o == 2 and i == 5][0]
        assert (view(pva, 8) == 0xC3).all()
