"""Benchmark configuration 5 between real processes, on the CPU: 2 and 4 processes, each loading the
host stand-in build of the library (tests/host_standin: the library's own sources, unchanged, with the
HIP calls answered on host memory), own regions, export them as file descriptors, import everybody
else's, and go through two coordinated pause/resume cycles. What runs is the engine's real code on every
side of the exchange: importers unmap before owners release (amem_nccl.cpp:517-526), owners re-create,
re-export and send one descriptor per (region, importer) over the socket service
(amem_nccl.cpp:633-649, gmm_client_impl.cpp:509-532), the importer's service thread maps it at the
original address while its main thread waits in resume (amem_nccl.cpp:385-409, :659-662), including an
owner that resumes late and an owner that has died. The GPU twin of the first test
(tests/test_gpu_peer.py::test_processes_sharing_one_gpu) runs the same worker code with the shipped
library where the machine's runtime can import another process's descriptor."""
import ctypes as C
import multiprocessing as mp
import os
import sys
import tempfile
import time
from multiprocessing import reduction

import numpy as np
import pytest

from peer_worker import run_world

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "host_standin"))
MiB = 1 << 20


@pytest.fixture(scope="module")
def standin():
    import build_standin
    return build_standin.build(os.path.join(HERE, "host_standin", "_build"))


@pytest.mark.parametrize("world", [2, 4])
def test_processes_through_pause_and_resume(standin, world):
    run_world(world, lib_path=standin, gid_base=0x6800)


def test_four_processes_at_the_full_shape_of_configuration_5(standin):
    """Benchmark configuration 5 at its stated shape between real processes: 4 processes, each owning all
    256 regions of configuration 2's layout (1,216 MiB, seeds 4-7), exporting 256 descriptors to each of
    the three others and importing their 768. Per resume every process re-exports 768 descriptors over
    three sockets and its service thread maps 768 received ones (amem_nccl.cpp:517-526, :633-662); the
    descriptor count of every process is the same after each cycle as before the first."""
    run_world(4, lib_path=standin, gid_base=0x6c00, nreg=256, phase_timeout=300)


def _owner_that_dies(ipc_dir, gid, lib_path, conn, ctrl):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid), AMEM_SLOT="0")
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = B.load(lib_path)
    fp = Footprint(2, 31, max_regions=3, threads=2)
    regs = H.Regions(lib, fp)
    for i in range(3):
        fd = C.c_int(-1)
        assert lib.amem_vmm_export(int(regs.handle[i]), C.byref(fd)) == 0
        conn.send((int(regs.handle[i]), int(regs.alloc[i])))
        reduction.send_handle(conn, fd.value, None)
        os.close(fd.value)
    ctrl.send("exported"); assert ctrl.recv() == "pause"
    assert lib.amem_mem_pause(0, 0) == 0
    c = H.counters(lib)
    ctrl.send(("paused", c["offload_cnt"], c["release_local_cnt"]))
    time.sleep(3600)                                   # killed by the parent while paused


def _importer_of_a_dead_owner(ipc_dir, gid, lib_path, conn, ctrl):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid), AMEM_SLOT="1")
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = B.load(lib_path)
    lib.amem_set_option(b"peer_timeout_ms", 60000)     # the point: it must not take this long
    fp = Footprint(2, 32, max_regions=4, threads=2)
    regs = H.Regions(lib, fp)
    imported = []
    for _ in range(3):
        owner_handle, size = conn.recv()
        fd = reduction.recv_handle(conn)
        va, h = C.c_uint64(), C.c_uint64()
        assert lib.amem_vmm_import(fd, size, 0, C.byref(va), C.byref(h)) == 0
        os.close(fd)
        assert lib.amem_add_alloc_info(va.value, size, B.TYPE_PEER_POSIX, 0, h.value, 0, owner_handle, None,
                                       B.CALLER_P2P_PEER) == 0
        imported.append((va.value, size))
    ctrl.send("imported"); assert ctrl.recv() == "pause"
    assert lib.amem_mem_pause(0, 0) == 0
    assert H.counters(lib)["release_shadow_cnt"] == 3
    ctrl.send("paused"); assert ctrl.recv() == "owner is dead"
    t0 = time.perf_counter()
    rc = lib.amem_mem_resume(0, 0)
    waited = time.perf_counter() - t0
    c = H.counters(lib)
    tab = H.region_table(lib, 0)
    ctrl.send(("resumed", rc, waited, c["paused"], c["release_shadow_cnt"], c["offload_cnt"],
               [tab[va]["state"] for va, _ in imported], regs.mismatched_bytes()))
    assert ctrl.recv() == "exit"
    for va, size in imported:
        lib.amem_del_alloc_info(va, 0, 0)
        lib.amem_vmm_free(va, size, 0)
    regs.free()
    lib.amem_shutdown()


def test_importer_whose_owner_died_while_paused_gets_an_error_not_a_hang(standin):
    """The reference's resume polls forever for owners that will never re-export (amem_nccl.cpp:659-662).
    Here the owner process is killed between pause and resume: the importer's resume restores the
    importer's own regions, notices from the owner's slot lock that nobody will ever send the missing
    mappings, and returns an error within moments, un-paused, with the orphaned imports still holes."""
    from asystem_amem_amd import binding as B
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        gid = 0x6900 + os.getpid() % 1024
        a, b = ctx.Pipe(duplex=True)
        oc, ic = ctx.Pipe(duplex=True), ctx.Pipe(duplex=True)
        owner = ctx.Process(target=_owner_that_dies, args=(ipc_dir, gid, standin, a, oc[1]))
        imp = ctx.Process(target=_importer_of_a_dead_owner, args=(ipc_dir, gid, standin, b, ic[1]))
        owner.start(); imp.start()
        try:
            assert oc[0].poll(60) and oc[0].recv() == "exported"
            assert ic[0].poll(60) and ic[0].recv() == "imported"
            ic[0].send("pause")                            # importers first, as the reference's callers order it
            assert ic[0].poll(60) and ic[0].recv() == "paused"
            oc[0].send("pause")
            assert oc[0].poll(60)
            assert oc[0].recv() == ("paused", 3, 3)        # three regions saved, three importer mappings on record
            owner.kill()                                   # exactly this process, by its pid
            owner.join(30)
            ic[0].send("owner is dead")
            assert ic[0].poll(60)
            tag, rc, waited, paused, shadow, offload, states, bad = ic[0].recv()
            assert tag == "resumed" and rc != 0 and waited < 5.0
            assert paused == 0 and shadow == 3 and offload == 0
            assert states == [B.STATE_HOLE] * 3 and bad == 0
            ic[0].send("exit")
            imp.join(30)
            assert imp.exitcode == 0
        finally:
            for p in (owner, imp):
                if p.is_alive():
                    p.kill()


def _plain_owner(ipc_dir, gid, lib_path, conn, ctrl):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid), AMEM_SLOT="0")
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = B.load(lib_path)
    fp = Footprint(2, 33, max_regions=3, threads=2)
    regs = H.Regions(lib, fp)
    for i in range(3):
        fd = C.c_int(-1)
        assert lib.amem_vmm_export(int(regs.handle[i]), C.byref(fd)) == 0
        conn.send((int(regs.handle[i]), int(regs.alloc[i])))
        reduction.send_handle(conn, fd.value, None)
        os.close(fd.value)
    for cycle in range(2):
        ctrl.send("ready"); assert ctrl.recv() == "pause"
        assert lib.amem_mem_pause(0, 0) == 0
        ctrl.send("paused"); assert ctrl.recv() == "resume"
        assert lib.amem_mem_resume(0, 0) == 0
        assert regs.mismatched_bytes() == 0
        ctrl.send("resumed")
    assert ctrl.recv() == "exit"
    regs.free()
    lib.amem_shutdown()


def _importer_without_memory_of_its_own(ipc_dir, gid, lib_path, conn, ctrl):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid), AMEM_SLOT="1")
    from asystem_amem_amd import binding as B, harness as H
    from asystem_amem_amd.footprint import Footprint
    lib = B.load(lib_path)
    fp = Footprint(2, 33, max_regions=3, threads=2)      # the owner's footprint, to check the bytes against
    imported = []
    for _ in range(3):
        owner_handle, size = conn.recv()
        fd = reduction.recv_handle(conn)
        va, h = C.c_uint64(), C.c_uint64()
        assert lib.amem_vmm_import(fd, size, 0, C.byref(va), C.byref(h)) == 0
        os.close(fd)
        assert lib.amem_add_alloc_info(va.value, size, B.TYPE_PEER_POSIX, 0, h.value, 0, owner_handle, None,
                                       B.CALLER_P2P_PEER) == 0
        imported.append((va.value, size))

    def bad_bytes():
        bad = 0
        for i, (va, size) in enumerate(imported):
            buf = np.empty(int(fp.sizes[i]), dtype=np.uint8)
            assert lib.amem_copy_from_device(buf.ctypes.data, va, buf.nbytes) == 0
            bad += fp.check_region(i, buf)
        return bad

    assert bad_bytes() == 0
    for cycle in range(2):
        ctrl.send("ready"); assert ctrl.recv() == "pause"
        assert lib.amem_mem_pause(0, 0) == 0                 # nothing of its own to save: mappings dropped, nothing copied
        c, st = H.counters(lib), H.cycle_stats(lib)
        assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"], c["paused"]) == (0, 3, 0, 1)
        assert st["parked_bytes"] == 0 and st["local_regions"] == 0 and st["peer_regions"] == 3
        ctrl.send("paused"); assert ctrl.recv() == "resume"
        assert lib.amem_mem_resume(0, 0) == 0                # returns once the owner has re-exported all three
        c = H.counters(lib)
        assert (c["release_shadow_cnt"], c["paused"]) == (0, 0)
        assert bad_bytes() == 0
        ctrl.send("resumed")
    assert ctrl.recv() == "exit"
    for va, size in imported:
        lib.amem_del_alloc_info(va, 0, 0)
        lib.amem_vmm_free(va, size, 0)
    lib.amem_shutdown()


def test_process_that_only_imports(standin):
    """A process whose whole registry is other processes' memory (an importer with no buffers of its own):
    its pause has nothing to scan or copy and only drops mappings, its resume only waits for the owner."""
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        gid = 0x6a00 + os.getpid() % 1024
        a, b = ctx.Pipe(duplex=True)
        oc, ic = ctx.Pipe(duplex=True), ctx.Pipe(duplex=True)
        owner = ctx.Process(target=_plain_owner, args=(ipc_dir, gid, standin, a, oc[1]))
        imp = ctx.Process(target=_importer_without_memory_of_its_own, args=(ipc_dir, gid, standin, b, ic[1]))
        owner.start(); imp.start()
        try:
            for cycle in range(2):
                for c in (oc[0], ic[0]):
                    assert c.poll(60) and c.recv() == "ready"
                ic[0].send("pause")
                assert ic[0].poll(60) and ic[0].recv() == "paused"
                oc[0].send("pause")
                assert oc[0].poll(60) and oc[0].recv() == "paused"
                # the importer resumes first in the second cycle and has to wait for the owner
                first, second = (oc[0], ic[0]) if cycle == 0 else (ic[0], oc[0])
                first.send("resume")
                if cycle == 1:
                    time.sleep(0.3)
                second.send("resume")
                for c in (oc[0], ic[0]):
                    assert c.poll(60) and c.recv() == "resumed"
            oc[0].send("exit"); ic[0].send("exit")
            owner.join(30); imp.join(30)
            assert owner.exitcode == 0 and imp.exitcode == 0
        finally:
            for p in (owner, imp):
                if p.is_alive():
                    p.kill()
