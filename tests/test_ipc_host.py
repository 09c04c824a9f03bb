"""Cross-process registration over the UNIX-socket service, without a GPU: an importer process
tells the owner process which VA maps the owner's handle (reference: register_peer,
gmm_client_impl.cpp:479-505 -> worker dispatch gmm_worker_impl.cpp:375-382 ->
amem_registerPeerInfo, amem_nccl.cpp:297-329). Handles and addresses are made up; only the
bookkeeping is exercised."""
import ctypes as C
import multiprocessing as mp
import os
import tempfile

MiB = 1 << 20
OWNER_VA, OWNER_HANDLE = 0x7f1000000000, 0xABCDE0


def _owner(ipc_dir, gid, to_parent, from_parent):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid))
    from asystem_amem_amd import binding as B, harness as H
    lib = B.load()
    assert lib.amem_add_alloc_info(OWNER_VA, 4 * MiB, B.TYPE_LOCAL, 0, OWNER_HANDLE, -1, 0, None, B.CALLER_P2P) == 0
    to_parent.send(("slot", lib.amem_get_slot()))
    assert from_parent.recv() == "check"
    t = H.region_table(lib, 0)[OWNER_VA]
    to_parent.send(("table", t["has_peer"], t["peers"]))
    assert from_parent.recv() == "exit"
    lib.amem_shutdown()


def _importer(ipc_dir, gid, owner_slot, to_parent, from_parent):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid))
    from asystem_amem_amd import binding as B, harness as H
    lib = B.load()
    lib.amem_set_option(b"peer_timeout_ms", 3000)
    my_va = 0x7f2000000000
    ok = lib.amem_add_alloc_info(my_va, 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x111, owner_slot, OWNER_HANDLE, None,
                                 B.CALLER_P2P_PEER)
    bad = lib.amem_add_alloc_info(my_va + (1 << 30), 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x112, owner_slot, 0xBAD, None,
                                  B.CALLER_P2P_PEER)
    nobody = lib.amem_add_alloc_info(my_va + (2 << 30), 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x113, 6, OWNER_HANDLE, None,
                                     B.CALLER_P2P_PEER)
    to_parent.send(("result", lib.amem_get_slot(), ok, bad, nobody, sorted(H.region_table(lib, 0))))
    assert from_parent.recv() == "exit"
    lib.amem_shutdown()


def test_register_peer_across_processes():
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        gid = 0x5000 + os.getpid() % 4096
        o_out, o_in = ctx.Pipe(), ctx.Pipe()
        owner = ctx.Process(target=_owner, args=(ipc_dir, gid, o_out[1], o_in[0]))
        owner.start()
        tag, owner_slot = o_out[0].recv()
        assert tag == "slot" and 0 <= owner_slot < 8
        i_out, i_in = ctx.Pipe(), ctx.Pipe()
        imp = ctx.Process(target=_importer, args=(ipc_dir, gid, owner_slot, i_out[1], i_in[0]))
        imp.start()
        assert i_out[0].poll(60)
        tag, imp_slot, ok, bad, nobody, imp_table = i_out[0].recv()
        assert imp_slot not in (-1, owner_slot)            # slots are claimed first-free
        assert ok == 0                                     # owner knew the handle
        assert bad == 1 and nobody == 1                    # unknown handle / no such owner: dropped
        assert imp_table == [0x7f2000000000]               # only the good import stays in scope
        o_in[1].send("check")
        tag, has_peer, peers = o_out[0].recv()
        assert has_peer == 1 and peers[imp_slot] == 0x7f2000000000
        assert sum(1 for p in peers if p) == 1
        i_in[1].send("exit")
        o_in[1].send("exit")
        imp.join(30)
        owner.join(30)
        assert imp.exitcode == 0 and owner.exitcode == 0
        assert not [f for f in os.listdir(ipc_dir) if f.endswith(".sock")]   # sockets removed on shutdown


def _late_importer(ipc_dir, gid, owner_slot, to_parent, from_parent):
    import time
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid))
    from asystem_amem_amd import binding as B
    lib = B.load()
    lib.amem_set_option(b"peer_timeout_ms", 30000)
    my_va = 0x7f3000000000
    first = lib.amem_add_alloc_info(my_va, 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x211, owner_slot, OWNER_HANDLE, None,
                                    B.CALLER_P2P_PEER)
    to_parent.send(("first", first))
    assert from_parent.recv() == "owner is dead"
    t0 = time.perf_counter()
    second = lib.amem_add_alloc_info(my_va + (1 << 30), 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x212, owner_slot, OWNER_HANDLE,
                                     None, B.CALLER_P2P_PEER)
    # the first failure dropped the connection; this one has to find out from the stale socket file
    third = lib.amem_add_alloc_info(my_va + (2 << 30), 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x213, owner_slot, OWNER_HANDLE,
                                    None, B.CALLER_P2P_PEER)
    to_parent.send(("second", second, third, time.perf_counter() - t0))
    assert from_parent.recv() == "exit"
    lib.amem_shutdown()


def test_a_peer_that_died_is_noticed_at_once():
    """Failure detection the reference lacks (its connect loop retries for a fixed time and then aborts the
    process, gmm_client_impl.cpp:288-347): a slot's lock dies with its holder, so a request to a peer
    whose process was killed fails within a moment instead of waiting out the 30 s timeout."""
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        gid = 0x6000 + os.getpid() % 4096
        o_out, o_in = ctx.Pipe(), ctx.Pipe()
        owner = ctx.Process(target=_owner, args=(ipc_dir, gid, o_out[1], o_in[0]))
        owner.start()
        tag, owner_slot = o_out[0].recv()
        i_out, i_in = ctx.Pipe(), ctx.Pipe()
        imp = ctx.Process(target=_late_importer, args=(ipc_dir, gid, owner_slot, i_out[1], i_in[0]))
        imp.start()
        assert i_out[0].poll(60) and i_out[0].recv() == ("first", 0)
        owner.kill()                                       # this very process, by its pid; no clean-up runs
        owner.join(30)
        i_in[1].send("owner is dead")
        assert i_out[0].poll(60)
        tag, second, third, seconds = i_out[0].recv()
        assert tag == "second" and second == 1 and third == 1 and seconds < 2.0
        i_in[1].send("exit")
        imp.join(30)
        assert imp.exitcode == 0


def _several_ranks(ipc_dir, gid, to_parent):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid))
    from asystem_amem_amd import binding as B, harness as H
    lib = B.load()
    out = {}
    owned = [(OWNER_VA + (k << 30), OWNER_HANDLE + k) for k in range(4)]
    for va, h in owned:
        assert lib.amem_add_alloc_info(va, 4 * MiB, B.TYPE_LOCAL, 0, h, -1, 0, None, B.CALLER_P2P) == 0
    first = lib.amem_get_slot()
    extra = [lib.amem_ipc_claim_slot() for _ in range(3)]
    out["slots"] = [first] + extra
    out["sockets"] = sorted(f for f in os.listdir(ipc_dir) if f.endswith(".sock"))
    out["foreign"] = lib.amem_ipc_act_as((max(out["slots"]) + 1) % 8 if len(set(out["slots"])) < 8 else 0)
    # same-process rule of the reference while loopback is off: a rank does not register with a rank of its own process
    assert lib.amem_ipc_act_as(extra[0]) == 0
    out["refused"] = lib.amem_add_alloc_info(0x7e0000000000, 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x900, first, owned[0][1],
                                             None, B.CALLER_P2P_PEER)
    assert lib.amem_set_option(b"peer_loopback", 1) == 0
    want = {}
    for r, slot in enumerate(extra):
        assert lib.amem_ipc_act_as(slot) == 0
        for k, (va, h) in enumerate(owned):
            my_va = 0x7e1000000000 + (r << 36) + (k << 30)
            assert lib.amem_add_alloc_info(my_va, 4 * MiB, B.TYPE_PEER_POSIX, 0, 0x1000 + 16 * r + k, first, h, None,
                                           B.CALLER_P2P_PEER) == 0
            want.setdefault(va, {})[slot] = my_va
    assert lib.amem_ipc_act_as(-1) == 0
    tab = H.region_table(lib, 0)
    out["table_size"] = len(tab)
    out["peers_ok"] = all(tab[va]["has_peer"] == 1 and
                          {s: p for s, p in enumerate(tab[va]["peers"]) if p} == want[va] for va, _ in owned)
    assert lib.amem_set_option(b"peer_loopback", 0) == 0
    lib.amem_shutdown()
    out["sockets_after"] = [f for f in os.listdir(ipc_dir) if f.endswith(".sock")]
    to_parent.send(out)


def test_several_ranks_in_one_process_each_hold_a_slot():
    """A process claims three more slots; each has its own lock, socket and service thread, and regions
    imported on behalf of each of them are recorded by the owner under that slot: the layout of benchmark
    configuration 5 (every region imported by three peers) inside one process. Registry only, no GPU."""
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        out_r, out_w = ctx.Pipe(duplex=False)
        p = ctx.Process(target=_several_ranks, args=(ipc_dir, 0x7000 + os.getpid() % 4096, out_w))
        p.start()
        assert out_r.poll(60)
        out = out_r.recv()
        p.join(30)
        assert p.exitcode == 0
        assert len(set(out["slots"])) == 4 and all(0 <= s < 8 for s in out["slots"])
        assert len(out["sockets"]) == 4
        assert out["foreign"] == 1                         # cannot act as a slot the process does not hold
        assert out["refused"] == 1
        assert out["table_size"] == 4 + 12 and out["peers_ok"]
        assert out["sockets_after"] == []


def _service_under_garbage(ipc_dir, gid, to_parent, from_parent):
    os.environ.update(AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=ipc_dir, AMEM_GROUPID=str(gid))
    from asystem_amem_amd import binding as B, harness as H
    lib = B.load()
    assert lib.amem_add_alloc_info(OWNER_VA, 4 * MiB, B.TYPE_LOCAL, 0, OWNER_HANDLE, -1, 0, None, B.CALLER_P2P) == 0
    to_parent.send(("slot", lib.amem_get_slot()))
    assert from_parent.recv() == "check"
    t = H.region_table(lib, 0)[OWNER_VA]
    to_parent.send(("table", t["has_peer"], [p for p in t["peers"] if p], len(H.region_table(lib, 0))))
    assert from_parent.recv() == "exit"
    lib.amem_shutdown()


def test_service_survives_malformed_and_abandoned_requests():
    """Host-forced failures of the transport (the reference's worker asserts or spins on them,
    gmm_worker_impl.cpp:288-431): a client that sends bytes that are no request, one that sends an unknown
    operation, one that connects and goes away without a word. The service drops or answers each and keeps
    serving: a well-formed registration afterwards still reaches the registry, and nothing else changed it."""
    import socket
    import struct
    ctx = mp.get_context("spawn")
    with tempfile.TemporaryDirectory() as ipc_dir:
        gid = 0x7100 + os.getpid() % 2048
        o_out, o_in = ctx.Pipe(), ctx.Pipe()
        owner = ctx.Process(target=_service_under_garbage, args=(ipc_dir, gid, o_out[1], o_in[0]))
        owner.start()
        try:
            assert o_out[0].poll(60)
            tag, slot = o_out[0].recv()
            path = os.path.join(ipc_dir, "amem_worker_%x_%d.sock" % (gid, slot))
            # wire format of a request: magic "AMEM", op, sender slot, pid (4 x 32 bit), two 64-bit operands
            def request(magic, op, sender, src, tgt):
                return struct.pack("<IiiiQQ", magic, op, sender, os.getpid(), src, tgt)
            MAGIC, REGISTER = 0x414D454D, 16
            s1 = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM); s1.connect(path)
            s1.sendall(b"\x00" * 32)                                   # right length, wrong magic: dropped
            s1.settimeout(5)
            assert s1.recv(4) == b""                                   # the service closed the connection
            s1.close()
            s2 = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM); s2.connect(path)
            s2.close()                                                 # connected and left
            s3 = socket.socket(socket.AF_UNIX, socket.SOCK_STREAM); s3.connect(path)
            s3.settimeout(5)
            s3.sendall(request(MAGIC, 99, 5, 0, 0))                    # unknown operation: answered with an error
            assert struct.unpack("<i", s3.recv(4))[0] == 1
            s3.sendall(request(MAGIC, REGISTER, 5, 0xDEAD, 0x7f5000000000))   # unknown handle: error, connection stays
            assert struct.unpack("<i", s3.recv(4))[0] == 1
            s3.sendall(request(MAGIC, REGISTER, 9, OWNER_HANDLE, 0x7f5000000000))   # slot out of range: error
            assert struct.unpack("<i", s3.recv(4))[0] == 1
            s3.sendall(request(MAGIC, REGISTER, 5, OWNER_HANDLE, 0x7f5000000000))   # and a good one on the same connection
            assert struct.unpack("<i", s3.recv(4))[0] == 0
            s3.close()
            o_in[1].send("check")
            assert o_out[0].poll(30)
            tag, has_peer, peers, nregions = o_out[0].recv()
            assert has_peer == 1 and peers == [0x7f5000000000] and nregions == 1
            o_in[1].send("exit")
            owner.join(30)
            assert owner.exitcode == 0
        finally:
            if owner.is_alive():
                owner.kill()
