"""Worker processes of the several-processes-one-GPU test (benchmark configuration 5 at reduced size),
shared by the GPU test (tests/test_gpu_peer.py) and by the CPU test that runs the same processes against
the host stand-in build of the library (tests/test_peer_processes_host.py). Every process owns regions,
exports them as POSIX fds, imports all peers' regions; coordinated pause (importers let go first, the
owners' release then frees the memory) and resume (owners re-create and re-export, importers remap at
their original address). Reference: amem_nccl.cpp:517-526, :633-662; gmm_client_impl.cpp:479-532."""
import ctypes as C
import multiprocessing as mp
import os
import tempfile
import time
from multiprocessing import reduction

import numpy as np

MiB = 1 << 20
NREG = 6          # default regions per process (config-2 distribution: 4 MiB channel buffers first); 256 = all of it


def _nfds():
    return len(os.listdir("/proc/self/fd"))


def _worker(rank, world, ipc_dir, gid, conns, ctrl, lib_path=None, NREG=NREG):
    """conns[j]: duplex connection to rank j (None for self); ctrl: connection to the parent;
    lib_path: library to load instead of the shipped one (the host stand-in build);
    NREG: regions this process owns (and imports from every peer)."""
    try:
        import threading
        os.environ.update(AMEM_ENABLE="1", GMM_LOG="2", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid), AMEM_SLOT=str(rank))
        from asystem_amem_amd import binding as B, harness as H
        from asystem_amem_amd.footprint import Footprint
        lib = B.load(lib_path)
        lib.amem_set_option(b"peer_timeout_ms", 60000)
        fp = Footprint(2, 4 + rank, max_regions=NREG, threads=2)
        regs = H.Regions(lib, fp)                      # local regions, registered
        assert lib.amem_get_slot() == rank
        ctrl.send(("ready", rank)); assert ctrl.recv() == "go"
        # export to every peer; on a thread of its own, so that with hundreds of regions two processes
        # that both have a full socket towards each other still drain what the other one sends
        def export_all():
            for j in range(world):
                if j == rank:
                    continue
                for i in range(NREG):
                    fd = C.c_int(-1)
                    assert lib.amem_vmm_export(int(regs.handle[i]), C.byref(fd)) == 0
                    conns[j].send((i, int(regs.handle[i]), int(regs.alloc[i])))
                    reduction.send_handle(conns[j], fd.value, None)
                    os.close(fd.value)
        exporter = threading.Thread(target=export_all)
        exporter.start()
        # import from every peer and register with the owner
        imported = {}   # (owner, i) -> (va, size)
        for j in range(world):
            if j == rank:
                continue
            for _ in range(NREG):
                i, owner_handle, size = conns[j].recv()
                fd = reduction.recv_handle(conns[j])
                va, h = C.c_uint64(), C.c_uint64()
                assert lib.amem_vmm_import(fd, size, 0, C.byref(va), C.byref(h)) == 0
                os.close(fd)
                rc = lib.amem_add_alloc_info(va.value, size, B.TYPE_PEER_POSIX, 0, h.value, j, owner_handle, None,
                                             B.CALLER_P2P_PEER)
                assert rc == 0, ("register with owner failed", rank, j, i, rc)
                imported[(j, i)] = (va.value, size)
        exporter.join()
        assert len(imported) == NREG * (world - 1)
        ctrl.send(("imported", rank)); assert ctrl.recv() == "go"
        peers_fp = {j: Footprint(2, 4 + j, max_regions=NREG, threads=2) for j in range(world) if j != rank}

        def check_imports():
            bad = 0
            for (j, i), (va, size) in imported.items():
                n = int(peers_fp[j].sizes[i])
                buf = np.empty(n, dtype=np.uint8)
                assert lib.amem_copy_from_device(buf.ctypes.data, va, n) == 0
                bad += peers_fp[j].check_region(i, buf)
            return bad

        assert check_imports() == 0
        tab = H.region_table(lib, 0)
        for i in range(NREG):                          # every owner entry knows all its importers
            t = tab[int(regs.va[i])]
            assert t["has_peer"] == 1 and sum(1 for p in t["peers"] if p) == world - 1 and t["peers"][rank] == 0
        before = {va: dict(t) for va, t in tab.items()}
        fds0 = _nfds()
        free0 = H.mem_free(lib)
        ctrl.send(("checked", rank, free0)); assert ctrl.recv() == "go"
        timings = []
        for cycle in range(2):
            assert lib.amem_mem_pause(0, 0) == 0
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_local_cnt"], c["release_shadow_cnt"]) == \
                (NREG, NREG * (world - 1), NREG * (world - 1))
            for va, t in H.region_table(lib, 0).items():
                assert t["state"] == B.STATE_HOLE
            ctrl.send(("paused", rank)); assert ctrl.recv() == "go"
            freed = H.mem_free(lib) - free0            # all ranks paused: everybody's memory is gone
            assert freed >= world * fp.total_bytes - 64 * MiB, (freed, world * fp.total_bytes)
            ctrl.send(("freed", rank)); assert ctrl.recv() == "go"
            if cycle == 1 and rank == 0:
                time.sleep(0.3)                        # importers must wait for a late owner, not fail
            assert lib.amem_mem_resume(0, 0) == 0
            st = H.cycle_stats(lib)
            timings.append((st["pause_ms"], st["resume_ms"], st["resume_peer_ms"]))
            c = H.counters(lib)
            assert (c["offload_cnt"], c["release_local_cnt"], c["release_shadow_cnt"], c["paused"]) == (0, 0, 0, 0)
            ctrl.send(("resumed", rank)); assert ctrl.recv() == "go"
            assert regs.mismatched_bytes() == 0        # own bytes
            assert check_imports() == 0                # peers' bytes at this process's original VAs
            after = H.region_table(lib, 0)
            diffs = [d for d in H.compare_tables(before, after) if d[1] != "handle_gen"]
            assert diffs == [], diffs
            assert _nfds() == fds0, (fds0, _nfds())    # exported and received fds are all closed
            ctrl.send(("verified", rank)); assert ctrl.recv() == "go"
        # an owner's write after resume is visible through the importers' old addresses
        if rank == 0:
            tag = np.full(4096, 0xA7, dtype=np.uint8)
            assert lib.amem_copy_to_device(int(regs.va[0]), tag.ctypes.data, 4096) == 0
        ctrl.send(("tagged", rank)); assert ctrl.recv() == "go"
        if rank != 0:
            buf = np.empty(4096, dtype=np.uint8)
            assert lib.amem_copy_from_device(buf.ctypes.data, imported[(0, 0)][0], 4096) == 0
            assert (buf == 0xA7).all()
        ctrl.send(("done", rank)); assert ctrl.recv() == "go"
        for (j, i), (va, size) in imported.items():
            lib.amem_del_alloc_info(va, 0, 0)
            lib.amem_vmm_free(va, size, 0)
        regs.free()
        lib.amem_shutdown()
        ctrl.send(("exit", rank, timings))
    except BaseException as e:  # report instead of hanging the barrier
        import traceback
        ctrl.send(("error", rank, traceback.format_exc()))
        raise




def run_world(world, lib_path=None, gid_base=0x6000, nreg=NREG, phase_timeout=120):
    """Start `world` worker processes, each owning `nreg` regions, walk them through the phases in lock
    step, and insist that every one of them finishes cleanly."""
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        gid = gid_base + os.getpid() % 4096 + world
        pair = {}
        for a in range(world):
            for b in range(a + 1, world):
                pair[(a, b)], pair[(b, a)] = ctx.Pipe(duplex=True)
        ctrls = [ctx.Pipe(duplex=True) for _ in range(world)]
        procs = []
        for r in range(world):
            conns = [pair.get((r, j)) for j in range(world)]
            p = ctx.Process(target=_worker, args=(r, world, ipc_dir, gid, conns, ctrls[r][1], lib_path, nreg))
            p.start()
            procs.append(p)
        try:
            phases = ["ready", "imported", "checked"] + ["paused", "freed", "resumed", "verified"] * 2 + ["tagged", "done"]
            for phase in phases:
                for r in range(world):
                    assert ctrls[r][0].poll(phase_timeout), "rank %d did not reach %s" % (r, phase)
                    msg = ctrls[r][0].recv()
                    assert msg[0] == phase, msg
                for r in range(world):
                    ctrls[r][0].send("go")
            timings = []
            for r in range(world):
                assert ctrls[r][0].poll(60)
                msg = ctrls[r][0].recv()
                assert msg[0] == "exit"
                timings.append(msg[2])
            for p in procs:
                p.join(60)
                assert p.exitcode == 0
            return timings          # per rank: (pause ms, resume ms, of which export + notify + wait) of each cycle
        finally:
            for p in procs:
                if p.is_alive():
                    p.kill()
