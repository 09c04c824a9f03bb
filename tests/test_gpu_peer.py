"""Several processes sharing the one GPU (benchmark configuration 5 at reduced size): every process
owns regions, exports them as POSIX fds, imports all peers' regions; coordinated pause (importers
let go first, owners' release then frees the memory) and resume (owners re-create and re-export,
importers remap at their original VA). Reference: amem_nccl.cpp:517-526, :633-662;
gmm_client_impl.cpp:479-532. Each process checks bytes at original VAs, counters, and that no fd leaks."""
import ctypes as C
import multiprocessing as mp
import os
import tempfile
import time
from multiprocessing import reduction

import numpy as np
import pytest

from peer_worker import _nfds, run_world

pytestmark = pytest.mark.gpu
MiB = 1 << 20


def _probe_owner(conn):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", AMEM_IPC="0")
    from asystem_amem_amd import binding as B
    lib = B.load()
    va, h, asz, fd = C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_int(-1)
    assert lib.amem_vmm_alloc(2 * MiB, 0, C.byref(va), C.byref(h), C.byref(asz)) == 0
    assert lib.amem_vmm_export(h.value, C.byref(fd)) == 0
    reduction.send_handle(conn, fd.value, None)
    conn.recv()
    lib.amem_vmm_free(va.value, asz.value, h.value)


def _probe_importer(conn, result):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="0", AMEM_IPC="0")
    from asystem_amem_amd import binding as B
    lib = B.load()
    fd = reduction.recv_handle(conn)
    va, h = C.c_uint64(), C.c_uint64()
    rc = lib.amem_vmm_import(fd, 2 * MiB, 0, C.byref(va), C.byref(h))
    if rc == 0:
        lib.amem_vmm_free(va.value, 2 * MiB, h.value)
    result.send(rc)
    conn.send("done")


_CROSS_PROCESS_IMPORT = None


def cross_process_import_works():
    """Whether this machine's runtime can import, in one process, a VMM fd that another process
    exported. On the GPU pool this build is developed on it cannot: hipMemImportFromShareableHandle
    returns hipErrorInvalidValue (HSA status 0x100D from hsa_amd_vmem_import_shareable_handle), although
    the same import inside the exporting process works and the exported dma-buf (exporter name
    'kfdproxy') is accepted by the raw KFD import ioctl."""
    global _CROSS_PROCESS_IMPORT
    if _CROSS_PROCESS_IMPORT is None:
        ctx = mp.get_context("spawn")
        a, b = ctx.Pipe(duplex=True)
        r_out, r_in = ctx.Pipe(duplex=False)
        po = ctx.Process(target=_probe_owner, args=(a,))
        pi = ctx.Process(target=_probe_importer, args=(b, r_in))
        po.start(); pi.start()
        rc = r_out.recv() if r_out.poll(120) else -1
        po.join(30); pi.join(30)
        for p in (po, pi):
            if p.is_alive():
                p.kill()
        _CROSS_PROCESS_IMPORT = (rc == 0)
    return _CROSS_PROCESS_IMPORT


@pytest.mark.parametrize("world", [2, 4])
def test_processes_sharing_one_gpu(gpu, world):
    if not cross_process_import_works():
        pytest.skip("this machine's HIP runtime cannot import a VMM fd exported by another process "
                    "(hipMemImportFromShareableHandle -> invalid argument); the same path is covered in one "
                    "process by test_peer_path_in_loopback and between processes on the CPU by tests/test_ipc_host.py")
    run_world(world)


@pytest.mark.parametrize("nregions", [5, 256])
def test_peer_path_in_loopback(gpu, fresh, nregions):
    """(256 regions: the per-process layout of benchmark configuration 5, every region exported and
    imported once, 256 descriptor messages per resume.)
    The whole cross-process path inside one process: the process imports its own exported
    regions at second addresses and, with peer_loopback on, registers them with its own socket
    service as if it were another process. Pause must drop the imported mappings first and
    really free the memory; resume must re-create, re-export through the socket (SCM_RIGHTS)
    and have the service thread map the new memory at the importer's original address."""
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = fresh
    assert lib.amem_set_option(b"peer_loopback", 1) == 0
    try:
        fp = Footprint(2, 11 if nregions == 5 else 4, max_regions=nregions, threads=8)
        regs = H.Regions(lib, fp)
        n = len(regs.va)
        assert n == nregions
        slot = lib.amem_get_slot()
        assert slot >= 0
        imports = []
        for i in range(len(regs.va)):
            fd = C.c_int(-1)
            assert lib.amem_vmm_export(int(regs.handle[i]), C.byref(fd)) == 0
            va, h = C.c_uint64(), C.c_uint64()
            assert lib.amem_vmm_import(fd.value, int(regs.alloc[i]), 0, C.byref(va), C.byref(h)) == 0
            os.close(fd.value)
            assert lib.amem_add_alloc_info(va.value, int(regs.alloc[i]), B.TYPE_PEER_POSIX, 0, h.value, slot,
                                           int(regs.handle[i]), None, B.CALLER_P2P_PEER) == 0
            imports.append(va.value)

        def imports_match():
            bad = 0
            for i, va in enumerate(imports):
                buf = np.empty(int(fp.sizes[i]), dtype=np.uint8)
                assert lib.amem_copy_from_device(buf.ctypes.data, va, buf.nbytes) == 0
                bad += fp.check_region(i, buf)
            return bad

        assert imports_match() == 0
        tab = H.region_table(lib, 0)
        assert len(tab) == 2 * n
        for i in range(n):
            t = tab[int(regs.va[i])]
            assert t["has_peer"] == 1 and t["peers"][slot] == imports[i]
        c = H.counters(lib)
        assert c["alloc_bytes"][B.CALLER_P2P_PEER] == fp.total_bytes and c["alloc_bytes"][B.CALLER_P2P] == fp.total_bytes
        before = H.region_table(lib, 0)
        lib.amem_mem_pause(0, 0); lib.amem_mem_resume(0, 0)     # warm cycle (engine scratch appears)
        fds0, free0 = _nfds(), H.mem_free(lib)
        for cycle in range(2):
            assert lib.amem_mem_pause(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_local_cnt"], c["release_shadow_cnt"]) == (n, n, n)
            assert H.mem_free(lib) - free0 >= fp.total_bytes - 8 * MiB      # both references are gone
            assert all(t["state"] == B.STATE_HOLE for t in H.region_table(lib, 0).values())
            assert lib.amem_mem_resume(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_local_cnt"], c["release_shadow_cnt"], c["paused"]) == (0, 0, 0, 0)
            assert regs.mismatched_bytes() == 0 and imports_match() == 0
            assert _nfds() == fds0
        after = H.region_table(lib, 0)
        assert [d for d in H.compare_tables(before, after) if d[1] != "handle_gen"] == []
        tag = np.full(4096, 0xA7, dtype=np.uint8)                 # one physical memory behind both addresses
        assert lib.amem_copy_to_device(int(regs.va[0]), tag.ctypes.data, 4096) == 0
        buf = np.empty(4096, dtype=np.uint8)
        assert lib.amem_copy_from_device(buf.ctypes.data, imports[0], 4096) == 0
        assert (buf == 0xA7).all()
        for i, va in enumerate(imports):
            lib.amem_del_alloc_info(va, 0, 0)
            lib.amem_vmm_free(va, int(regs.alloc[i]), 0)
        regs.free()
    finally:
        lib.amem_mem_resume(0, 0)
        assert lib.amem_set_option(b"peer_loopback", 0) == 0


def test_importer_times_out_when_owner_never_re_exports(gpu, fresh):
    """Failure handling the reference lacks (its resume spins forever, amem_nccl.cpp:659-662): an
    importer whose owner forgot the region before resume gives up after peer_timeout_ms, reports
    an error and stays consistent. Forced from the host: nothing on the GPU hangs or faults."""
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = fresh
    old_to = lib.amem_get_option(b"peer_timeout_ms")
    assert lib.amem_set_option(b"peer_loopback", 1) == 0 and lib.amem_set_option(b"peer_timeout_ms", 300) == 0
    try:
        fp = Footprint(2, 12, max_regions=2, threads=2)
        regs = H.Regions(lib, fp)
        slot = lib.amem_get_slot()
        fd, va, h = C.c_int(-1), C.c_uint64(), C.c_uint64()
        assert lib.amem_vmm_export(int(regs.handle[0]), C.byref(fd)) == 0
        assert lib.amem_vmm_import(fd.value, int(regs.alloc[0]), 0, C.byref(va), C.byref(h)) == 0
        os.close(fd.value)
        assert lib.amem_add_alloc_info(va.value, int(regs.alloc[0]), B.TYPE_PEER_POSIX, 0, h.value, slot,
                                       int(regs.handle[0]), None, B.CALLER_P2P_PEER) == 0
        # the "owner" drops its record of region 0: nobody will re-export it
        assert lib.amem_del_alloc_info(int(regs.va[0]), int(regs.handle[0]), 0) == 0
        assert lib.amem_mem_pause(0, 0) == 0
        assert H.counters(lib)["release_shadow_cnt"] == 1
        t0 = time.perf_counter()
        rc = lib.amem_mem_resume(0, 0)
        waited = time.perf_counter() - t0
        assert rc != 0 and 0.25 < waited < 5.0
        c = H.counters(lib)
        assert c["paused"] == 0 and c["release_shadow_cnt"] == 1            # reported, not hidden
        assert H.region_table(lib, 0)[va.value]["state"] == B.STATE_HOLE    # the orphaned import is still a hole
        buf = np.empty(int(fp.sizes[1]), dtype=np.uint8)                    # everything else came back
        assert lib.amem_copy_from_device(buf.ctypes.data, int(regs.va[1]), buf.nbytes) == 0
        assert fp.check_region(1, buf) == 0
        lib.amem_del_alloc_info(va.value, 0, 0)
        lib.amem_vmm_free(va.value, int(regs.alloc[0]), 0)
        lib.amem_vmm_free(int(regs.va[0]), int(regs.alloc[0]), 0)          # still mapped: it was never paused
        lib.amem_del_alloc_info(int(regs.va[1]), 0, 0)
        lib.amem_vmm_free(int(regs.va[1]), int(regs.alloc[1]), 0)
    finally:
        lib.amem_mem_resume(0, 0)
        lib.amem_set_option(b"peer_loopback", 0)
        lib.amem_set_option(b"peer_timeout_ms", old_to)


def test_owner_forgets_an_importer_whose_process_is_gone(gpu, fresh):
    """An owner holds the address of an importer in a slot nobody holds (its process died). Resume
    finds that out from the slot's lock, drops the stale entry and succeeds; the next cycle no
    longer tries. Nothing is killed here: the slot simply never had a holder."""
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = fresh
    fp = Footprint(2, 14, max_regions=3, threads=2)
    regs = H.Regions(lib, fp)
    ghost = (lib.amem_get_slot() + 3) % 8
    assert lib.amem_add_peer_info(int(regs.va[1]), 0x7f5500000000, ghost) == 0
    assert H.region_table(lib, 0)[int(regs.va[1])]["has_peer"] == 1
    assert lib.amem_mem_pause(0, 0) == 0
    assert H.counters(lib)["release_local_cnt"] == 1
    t0 = time.perf_counter()
    assert lib.amem_mem_resume(0, 0) == 0
    assert time.perf_counter() - t0 < 5.0                      # no waiting for a peer that cannot answer
    r = H.region_table(lib, 0)[int(regs.va[1])]
    assert r["has_peer"] == 0 and not any(r["peers"]) and H.counters(lib)["release_local_cnt"] == 0
    assert regs.mismatched_bytes() == 0
    assert lib.amem_mem_pause(0, 0) == 0 and H.counters(lib)["release_local_cnt"] == 0
    assert lib.amem_mem_resume(0, 0) == 0 and regs.mismatched_bytes() == 0
    regs.free()



def test_config5_shape_three_importer_ranks_in_one_process(gpu, fresh, measured):
    """Benchmark configuration 5 at its full per-process shape, in the one form this machine's runtime
    allows (it refuses a VMM descriptor exported by another process): the process holds four slots, each
    with its own lock, socket and service thread; the first owns the 256 regions of configuration 2's
    layout (1,216 MiB), each of the other three imports all 256 at addresses of its own. 768 registration
    requests, and per resume 768 descriptor messages (SCM_RIGHTS) to three different services, each of
    which maps the new memory at its importer's original address. Counter closed forms as for the oracle's
    tests/test_oracle_cycle.py::test_config5_layout_four_processes (amem_nccl.cpp:511 offload per local
    region, :524 releasePeer per import, :547-550 releaseLocal per recorded importer)."""
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = fresh
    assert lib.amem_set_option(b"peer_loopback", 1) == 0
    try:
        N, R = 256, 3
        fp = Footprint(2, 4, max_regions=N, threads=8)
        regs = H.Regions(lib, fp)
        assert len(regs.va) == N and fp.total_bytes == 1216 * MiB
        owner = lib.amem_get_slot()
        ranks = [lib.amem_ipc_claim_slot() for _ in range(R)]
        assert owner >= 0 and len({owner, *ranks}) == R + 1 and min(ranks) >= 0
        imports = {}                                         # (rank slot, region) -> importer's address
        for s in ranks:
            assert lib.amem_ipc_act_as(s) == 0
            for i in range(N):
                fd, va, h = C.c_int(-1), C.c_uint64(), C.c_uint64()
                assert lib.amem_vmm_export(int(regs.handle[i]), C.byref(fd)) == 0
                assert lib.amem_vmm_import(fd.value, int(regs.alloc[i]), 0, C.byref(va), C.byref(h)) == 0
                os.close(fd.value)
                assert lib.amem_add_alloc_info(va.value, int(regs.alloc[i]), B.TYPE_PEER_POSIX, 0, h.value, owner,
                                               int(regs.handle[i]), None, B.CALLER_P2P_PEER) == 0
                imports[(s, i)] = va.value
        assert lib.amem_ipc_act_as(-1) == 0
        assert len(set(imports.values())) == R * N

        def imports_match():
            bad = 0
            buf = np.empty(int(fp.sizes.max()), dtype=np.uint8)
            for (s, i), va in imports.items():
                n = int(fp.sizes[i])
                assert lib.amem_copy_from_device(buf.ctypes.data, va, n) == 0
                bad += fp.check_region(i, buf[:n])
            return bad

        tab = H.region_table(lib, 0)
        assert len(tab) == N + R * N
        for i in range(N):                                   # every owner entry knows its three importers
            t = tab[int(regs.va[i])]
            assert t["has_peer"] == 1
            assert {s: p for s, p in enumerate(t["peers"]) if p} == {s: imports[(s, i)] for s in ranks}
        c = H.counters(lib)
        assert c["alloc_bytes"][B.CALLER_P2P] == fp.total_bytes and c["alloc_bytes"][B.CALLER_P2P_PEER] == R * fp.total_bytes
        assert imports_match() == 0
        before = H.region_table(lib, 0)
        assert lib.amem_mem_pause(0, 0) == 0 and lib.amem_mem_resume(0, 0) == 0     # warm cycle: engine scratch, pinned pool
        fds0, free0 = _nfds(), H.mem_free(lib)
        times = []
        for cycle in range(2):
            assert lib.amem_mem_pause(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"]) == (N, R * N, R * N)
            assert H.mem_free(lib) - free0 >= fp.total_bytes - 8 * MiB   # all four references to every region are gone
            assert all(t["state"] == B.STATE_HOLE for t in H.region_table(lib, 0).values())
            assert lib.amem_check_paused(0) == 1
            assert lib.amem_mem_resume(0, 0) == 0
            st = H.cycle_stats(lib)
            times.append((st["pause_ms"], st["resume_ms"], st["resume_peer_ms"]))
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"], c["paused"]) == (0, 0, 0, 0)
            assert _nfds() == fds0                           # 256 exported and 768 received descriptors, all closed
            assert regs.mismatched_bytes() == 0              # the owner's bytes at the owner's addresses
            assert imports_match() == 0                      # and at all 768 importer addresses
        after = H.region_table(lib, 0)
        assert [d for d in H.compare_tables(before, after) if d[1] != "handle_gen"] == []
        assert all(after[va]["handle_gen"] == before[va]["handle_gen"] + 3 for va in before)   # three cycles, three new handles each
        measured("config-5 shape, one owner: %d regions x %d importers, pause/resume/peer ms per cycle: %s" %
                 (N, R, ", ".join("%.0f/%.0f/%.0f" % t for t in times)))
        # one physical memory behind all four addresses of a region
        tag = np.full(4096, 0xC3, dtype=np.uint8)
        assert lib.amem_copy_to_device(int(regs.va[5]), tag.ctypes.data, 4096) == 0
        for s in ranks:
            buf = np.empty(4096, dtype=np.uint8)
            assert lib.amem_copy_from_device(buf.ctypes.data, imports[(s, 5)], 4096) == 0
            assert (buf == 0xC3).all()
        for (s, i), va in imports.items():
            lib.amem_del_alloc_info(va, 0, 0)
            lib.amem_vmm_free(va, int(regs.alloc[i]), 0)
        regs.free()
    finally:
        lib.amem_mem_resume(0, 0)
        lib.amem_ipc_act_as(-1)
        assert lib.amem_set_option(b"peer_loopback", 0) == 0


def test_config5_every_rank_owns_and_imports_in_one_process(gpu, fresh, measured):
    """Benchmark configuration 5's full matrix in the one form this machine's runtime allows (one process):
    four slots, each with its own lock, socket and service thread; EVERY slot owns the 256 regions of
    configuration 2's layout (seeds 4, 5, 6, 7: 4 x 1,216 MiB) and imports the 768 regions of the other
    three at addresses of its own. 1,024 owned + 3,072 imported mappings; 3,072 registration requests spread
    over four services; per resume 3,072 descriptor messages (SCM_RIGHTS), each owner's regions going to
    three different services while the same process's services map what the other owners send. Closed forms
    (amem_nccl.cpp:511 one offload per local region, :524 one releasePeer per imported mapping, :547-550 one
    releaseLocal per recorded importer): 1,024 / 3,072 / 3,072 at pause, 0 / 0 / 0 after resume."""
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = fresh
    assert lib.amem_set_option(b"peer_loopback", 1) == 0
    try:
        N, W = 256, 4
        slots = [lib.amem_ipc_start()] + [lib.amem_ipc_claim_slot() for _ in range(W - 1)]
        assert min(slots) >= 0 and len(set(slots)) == W
        fps = [Footprint(2, 4 + k, max_regions=N, threads=8) for k in range(W)]
        owned = [H.Regions(lib, fp) for fp in fps]          # rank k's own regions (local memory has no slot of its own)
        assert all(len(r.va) == N and fp.total_bytes == 1216 * MiB for r, fp in zip(owned, fps))
        total = sum(fp.total_bytes for fp in fps)
        imports = {}                                         # (importing rank, owning rank, region) -> importer's address
        for k in range(W):                                   # rank k imports from every other rank j
            assert lib.amem_ipc_act_as(slots[k]) == 0
            for j in range(W):
                if j == k:
                    continue
                for i in range(N):
                    fd, va, h = C.c_int(-1), C.c_uint64(), C.c_uint64()
                    assert lib.amem_vmm_export(int(owned[j].handle[i]), C.byref(fd)) == 0
                    assert lib.amem_vmm_import(fd.value, int(owned[j].alloc[i]), 0, C.byref(va), C.byref(h)) == 0
                    os.close(fd.value)
                    assert lib.amem_add_alloc_info(va.value, int(owned[j].alloc[i]), B.TYPE_PEER_POSIX, 0, h.value,
                                                   slots[j], int(owned[j].handle[i]), None, B.CALLER_P2P_PEER) == 0
                    imports[(k, j, i)] = va.value
        assert lib.amem_ipc_act_as(-1) == 0
        assert len(set(imports.values())) == W * (W - 1) * N

        def imports_match():
            bad = 0
            buf = np.empty(max(int(fp.sizes.max()) for fp in fps), dtype=np.uint8)
            for (k, j, i), va in imports.items():
                n = int(fps[j].sizes[i])
                assert lib.amem_copy_from_device(buf.ctypes.data, va, n) == 0
                bad += fps[j].check_region(i, buf[:n])
            return bad

        def owned_match():
            return sum(r.mismatched_bytes() for r in owned)

        tab = H.region_table(lib, 0)
        assert len(tab) == W * N + W * (W - 1) * N == 4096
        for j in range(W):                                   # every owned region names exactly the three other slots
            for i in range(N):
                t = tab[int(owned[j].va[i])]
                assert t["has_peer"] == 1
                assert {s: p for s, p in enumerate(t["peers"]) if p} == \
                    {slots[k]: imports[(k, j, i)] for k in range(W) if k != j}
        assert all(tab[va]["type"] == B.TYPE_PEER_POSIX for va in imports.values())

        def served():
            out = {}
            for s in slots:
                n = (C.c_uint64 * 3)()
                assert lib.amem_ipc_served(s, n) == 0
                out[s] = tuple(n)
            return out

        # every owner's service took the registrations of the three other ranks, nobody else's
        assert served() == {s: ((W - 1) * N, 0, 0) for s in slots}
        c = H.counters(lib)
        assert c["alloc_bytes"][B.CALLER_P2P] == total and c["alloc_bytes"][B.CALLER_P2P_PEER] == (W - 1) * total
        assert owned_match() == 0 and imports_match() == 0
        before = H.region_table(lib, 0)
        assert lib.amem_mem_pause(0, 0) == 0 and lib.amem_mem_resume(0, 0) == 0     # warm cycle: engine scratch, pinned pool
        fds0, free0 = _nfds(), H.mem_free(lib)
        times = []
        for cycle in range(2):
            assert lib.amem_mem_pause(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"]) == \
                (W * N, W * (W - 1) * N, W * (W - 1) * N) == (1024, 3072, 3072)
            assert H.mem_free(lib) - free0 >= total - 16 * MiB   # all four references to every region are gone
            assert all(t["state"] == B.STATE_HOLE for t in H.region_table(lib, 0).values())
            assert lib.amem_check_paused(0) == 1
            assert lib.amem_mem_resume(0, 0) == 0
            st = H.cycle_stats(lib)
            times.append((st["pause_ms"], st["resume_ms"], st["resume_peer_ms"]))
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"], c["paused"]) == (0, 0, 0, 0)
            assert _nfds() == fds0                           # 1,024 exported and 3,072 received descriptors, all closed
            # every rank's service mapped the 768 descriptors the three other owners sent it (warm cycle included)
            assert served() == {s: ((W - 1) * N, (cycle + 2) * (W - 1) * N, 0) for s in slots}
            assert owned_match() == 0                        # 1,024 owner addresses against the four seeds
            assert imports_match() == 0                      # and all 3,072 importer addresses
        after = H.region_table(lib, 0)
        assert [d for d in H.compare_tables(before, after) if d[1] != "handle_gen"] == []
        assert all(after[va]["handle_gen"] == before[va]["handle_gen"] + 3 for va in before)
        measured("config-5 matrix, one process: %d ranks x %d regions, each imported by %d: pause/resume/peer ms per cycle: %s" %
                 (W, N, W - 1, ", ".join("%.0f/%.0f/%.0f" % t for t in times)))
        # one physical memory behind all four addresses of a region, for a region of every owner
        for j in range(W):
            tag = np.full(4096, 0xC0 + j, dtype=np.uint8)
            assert lib.amem_copy_to_device(int(owned[j].va[7]), tag.ctypes.data, 4096) == 0
            for k in range(W):
                if k != j:
                    buf = np.empty(4096, dtype=np.uint8)
                    assert lib.amem_copy_from_device(buf.ctypes.data, imports[(k, j, 7)], 4096) == 0
                    assert (buf == 0xC0 + j).all()
        for (k, j, i), va in imports.items():
            lib.amem_del_alloc_info(va, 0, 0)
            lib.amem_vmm_free(va, int(owned[j].alloc[i]), 0)
        for r in owned:
            r.free()
    finally:
        lib.amem_mem_resume(0, 0)
        lib.amem_ipc_act_as(-1)
        assert lib.amem_set_option(b"peer_loopback", 0) == 0


def test_more_shared_regions_than_descriptors_may_be_open(gpu, fresh, measured):
    """This runtime lets a process keep 1,024 exported descriptors open and no more (the 1,025th export
    fails, and beside 1,024 open ones no imported mapping can be given access; probed with plain HIP calls
    through amem_vmm_export / amem_vmm_import below). A resume therefore exports each region only when it
    tells that region's importers and closes the descriptor before the next (as the reference's loop does,
    amem_nccl.cpp:613, :646): 1,100 owned regions of 2 MiB, each imported once by a second rank of the
    process, go through two cycles with every byte checked at both addresses."""
    from asystem_amem_amd import binding as B, harness as H
    lib = fresh
    assert lib.amem_set_option(b"peer_loopback", 1) == 0
    N = 1100
    try:
        owner = lib.amem_ipc_start()
        rank = lib.amem_ipc_claim_slot()
        assert owner >= 0 and rank >= 0 and rank != owner
        rng = np.random.default_rng(77)
        owned, imports, data = [], [], []
        for i in range(N):
            va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
            assert lib.amem_vmm_alloc(2 * MiB, 0, C.byref(va), C.byref(h), C.byref(asz)) == 0
            d = rng.integers(0, 256, 4096, dtype=np.uint8)     # one page of its own per region, the rest stays zero
            assert lib.amem_copy_to_device(va.value + (i % 32) * 65536, d.ctypes.data, 4096) == 0
            assert lib.amem_add_alloc_info(va.value, asz.value, B.TYPE_LOCAL, 0, h.value, -1, 0, None, B.CALLER_P2P) == 0
            owned.append((va.value, h.value, asz.value)); data.append(d)
        # the limit itself, with nothing of the engine involved
        fds = []
        for va, h, asz in owned:
            fd = C.c_int(-1)
            if lib.amem_vmm_export(h, C.byref(fd)) != 0:
                break
            fds.append(fd.value)
        open_at_once = len(fds)
        for fd in fds:
            os.close(fd)
        assert lib.amem_ipc_act_as(rank) == 0
        for va, h, asz in owned:
            fd, iva, ih = C.c_int(-1), C.c_uint64(), C.c_uint64()
            assert lib.amem_vmm_export(h, C.byref(fd)) == 0
            assert lib.amem_vmm_import(fd.value, asz, 0, C.byref(iva), C.byref(ih)) == 0
            os.close(fd.value)
            assert lib.amem_add_alloc_info(iva.value, asz, B.TYPE_PEER_POSIX, 0, ih.value, owner, h, None, B.CALLER_P2P_PEER) == 0
            imports.append(iva.value)
        assert lib.amem_ipc_act_as(-1) == 0

        def bad():
            n, buf = 0, np.empty(4096, dtype=np.uint8)
            for i in range(N):
                for base in (owned[i][0], imports[i]):
                    assert lib.amem_copy_from_device(buf.ctypes.data, base + (i % 32) * 65536, 4096) == 0
                    n += int(np.count_nonzero(buf != data[i]))
            return n

        assert bad() == 0
        assert lib.amem_mem_pause(0, 0) == 0 and lib.amem_mem_resume(0, 0) == 0     # warm cycle: engine scratch, pinned pool
        fds0 = _nfds()
        for cycle in range(2):
            assert lib.amem_mem_pause(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"]) == (N, N, N)
            assert lib.amem_mem_resume(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"], c["paused"]) == (0, 0, 0, 0)
            assert _nfds() == fds0 and bad() == 0
        st = H.cycle_stats(lib)
        measured("exported descriptors this runtime lets a process hold open: %d; %d shared regions resumed, "
                 "pause %.0f ms, resume %.0f ms of which %.0f ms export + notify + wait" %
                 (open_at_once, N, st["pause_ms"], st["resume_ms"], st["resume_peer_ms"]))
        for i in range(N):
            lib.amem_del_alloc_info(imports[i], 0, 0)
            lib.amem_vmm_free(imports[i], owned[i][2], 0)
            lib.amem_del_alloc_info(owned[i][0], 0, 0)
            lib.amem_vmm_free(owned[i][0], owned[i][2], 0)
    finally:
        lib.amem_mem_resume(0, 0)
        lib.amem_ipc_act_as(-1)
        assert lib.amem_set_option(b"peer_loopback", 0) == 0
