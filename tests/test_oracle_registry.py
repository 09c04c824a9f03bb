"""Pins the oracle's registry against what the reference's source fixes: return codes,
state machine and counter arithmetic read off amem_nccl_plugin/amem_nccl.cpp, and the two
samples of output the reference publishes (README ncclMemStats sample, run_result log line).
Each expectation below is written from the cited lines, not from the oracle's code."""
import json
import os

import oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
MiB = 1 << 20
LOCAL, PEER = 0, 3
ST_ALLOC, ST_HOLE = 1, 3


def add(orc, ctx, va, size=2 * MiB, type_=LOCAL, handle=None, peer_dev=-1, peer_handle=0, user=0, caller=1):
    return orc.oracle_add_alloc_info(ctx, va, size, type_, 0, handle if handle is not None else va + 1, peer_dev,
                                     peer_handle, user, caller)


def test_add_new_and_reregister(fresh_orc):
    orc = fresh_orc
    # amem_nccl.cpp:142-148: new VA -> state ALLOC, allocBytes[caller] += size, handle indexed (:264)
    assert add(orc, 0, 0x10000000, 4 * MiB, caller=1, handle=0xAAA, user=0x77) == 0
    t = O.region_table(orc, 0)[0x10000000]
    assert (t["state"], t["alloc_sz"], t["tags"], t["handle"], t["user_info"], t["refcount"], t["has_peer"]) == \
        (ST_ALLOC, 4 * MiB, 1, 0xAAA, 0x77, 0, 0)
    assert t["pid"] == os.getpid() and t["peers"] == [0] * 8 and t["cpu_addr"] == 0
    c = O.counters(orc, 0)
    assert c["alloc_bytes"][1] == 4 * MiB and c["smoke_log"] == 1
    assert orc.oracle_handle_lookup(0, 0, 0xAAA) == 0x10000000
    # :179-191: same VA again overwrites type/state/size/handle/userInfo/tags, no new byte accounting
    assert add(orc, 0, 0x10000000, 8 * MiB, caller=3, handle=0xBBB, user=0x99) == 0
    t = O.region_table(orc, 0)[0x10000000]
    assert (t["alloc_sz"], t["tags"], t["handle"], t["user_info"]) == (8 * MiB, 3, 0xBBB, 0x99)
    c = O.counters(orc, 0)
    assert c["alloc_bytes"][1] == 4 * MiB and c["alloc_bytes"][3] == 0 and c["region_count"] == 1
    # emplace keeps the old key too (:264): both handles now resolve
    assert orc.oracle_handle_lookup(0, 0, 0xBBB) == 0x10000000


def test_group_id_only_before_first_alloc(fresh_orc):
    orc = fresh_orc
    assert orc.oracle_set_group_id(0, 170) == 0 and orc.oracle_get_group_id(0) == 170  # :686-688
    add(orc, 0, 0x10000000)
    assert orc.oracle_set_group_id(0, 200) == 1 and orc.oracle_get_group_id(0) == 170  # :689-692


def test_disabled_is_a_no_op(fresh_orc):
    orc = fresh_orc
    orc.oracle_ctx_enable(0, 0)  # :107-109, :417, :454, :470, :580
    assert add(orc, 0, 0x10000000) == 0
    assert orc.oracle_region_count(0, 0) == 0
    assert orc.oracle_check_paused(0) == 0 and orc.oracle_mem_pause(0) == 0 and orc.oracle_mem_resume(0) == 0


def test_del_accounting(fresh_orc):
    orc = fresh_orc
    add(orc, 0, 0x10000000, 4 * MiB, caller=7, handle=0xA)
    add(orc, 0, 0x20000000, 2 * MiB, caller=99, handle=0xB)  # caller >= 16: not counted on add (:146)
    assert O.counters(orc, 0)["alloc_bytes"][7] == 4 * MiB
    assert orc.oracle_del_alloc_info(0, 0x10000000, 0xA, 0) == 0
    c = O.counters(orc, 0)
    assert c["alloc_bytes"][7] == 0 and c["del_bytes"] == 0
    assert orc.oracle_handle_lookup(0, 0, 0xA) == 0  # :445
    assert orc.oracle_del_alloc_info(0, 0x20000000, 0xB, 0) == 0
    assert O.counters(orc, 0)["del_bytes"] == 2 * MiB  # :438-440: tags >= 16 goes to delBytes
    assert orc.oracle_del_alloc_info(0, 0, 0, 0) == 0  # :421
    assert orc.oracle_del_alloc_info(0, 0x30000000, 0, 0) == 0  # unknown VA: still 0


def test_refcount_and_peer_info(fresh_orc):
    orc = fresh_orc
    add(orc, 0, 0x10000000, handle=0xA)
    assert orc.oracle_add_refcount(0, 0x10000000, 2) == 0 and orc.oracle_add_refcount(0, 0x10000000, 1) == 0
    assert orc.oracle_add_refcount(0, 0x99000000, 1) == 1  # :350-353
    assert O.region_table(orc, 0)[0x10000000]["refcount"] == 3
    assert orc.oracle_add_peer_info(0, 0x10000000, 0x7000, 5) == 0  # :367-372
    assert orc.oracle_add_peer_info(0, 0x99000000, 0x7000, 5) == 1
    assert orc.oracle_register_peer_info(0, 0xA, 0x8000, 2) == 0  # :305-315
    assert orc.oracle_register_peer_info(0, 0xDEAD, 0x8000, 2) == 1  # :323-326
    t = O.region_table(orc, 0)[0x10000000]
    assert t["has_peer"] == 1 and t["peers"][5] == 0x7000 and t["peers"][2] == 0x8000


def test_peer_add_registers_with_owner_or_is_dropped(fresh_orc):
    orc = fresh_orc
    add(orc, 0, 0x10000000, handle=0xA)                       # owner = context 0
    # importer = context 1 names owner slot 0 and the owner's handle (:195-207)
    assert add(orc, 1, 0x50000000, type_=PEER, handle=0xF1, peer_dev=0, peer_handle=0xA, caller=7) == 0
    assert O.region_table(orc, 0)[0x10000000]["peers"][1] == 0x50000000
    t = O.region_table(orc, 1)[0x50000000]
    assert t["type"] == PEER and t["mc_handle"] == 0xA and t["oos_flag"] == 0
    assert orc.oracle_handle_lookup(1, 0, 0xF1) == 0          # peers are not indexed by handle (:258-265)
    # owner does not know the handle -> RPC returns 1 -> importer erases its entry (:209-220), bytes stay counted
    assert add(orc, 1, 0x60000000, type_=PEER, handle=0xF2, peer_dev=0, peer_handle=0xBAD, caller=7) == 1
    assert 0x60000000 not in O.region_table(orc, 1)
    assert O.counters(orc, 1)["alloc_bytes"][7] == 4 * MiB
    # same process as owner: register_peer refuses (gmm_client_impl.cpp:482-484) -> dropped
    assert add(orc, 0, 0x70000000, type_=PEER, handle=0xF3, peer_dev=0, peer_handle=0xA, caller=7) == 1
    assert 0x70000000 not in O.region_table(orc, 0)
    # owner unknown (-1) and not detectable: erased, returns 1 (:245-256)
    assert add(orc, 1, 0x80000000, type_=PEER, handle=0xF4, peer_dev=-1, peer_handle=0xA, caller=9) == 1
    assert 0x80000000 not in O.region_table(orc, 1)


def test_memstats_total_matches_readme_sample(fresh_orc):
    orc = fresh_orc
    g = json.load(open(os.path.join(HERE, "golden", "memstats_readme.json")))
    va = 0x10000000
    for caller, nbytes in g["caller_bytes"].items():
        # split each caller's bytes over a few registrations, as NCCL would
        parts = [nbytes // 3, nbytes // 3, nbytes - 2 * (nbytes // 3)]
        for p in parts:
            assert add(orc, 0, va, p, caller=int(caller)) == 0
            va += 0x10000000
    c = O.counters(orc, 0)
    for caller, nbytes in g["caller_bytes"].items():
        assert c["alloc_bytes"][int(caller)] == nbytes
    total = orc.oracle_mem_stats_total(0)
    assert total == g["total_bytes"] and total >> 20 == g["total_mb"]
