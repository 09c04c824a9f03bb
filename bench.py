#!/usr/bin/env python3
"""Benchmark of the pause/resume path on one MI355X.

A step is one pause + resume cycle of the training-rank footprint: the shortest prefix of
the 2,560 log-uniform [2, 64) MiB draws (seed 2) that reaches 10 GiB — 572 regions,
10.02 GiB — with 30 % all-zero 64 KiB chunks, and writes to 1 % of the chunks between
cycles. The footprint is resident in HBM before the clock starts; the clock covers the
two calls amem_mem_pause() and amem_mem_resume() and nothing else.

Prints one JSON line:
  value      2 * F / (t_pause + t_resume), GB/s (1e9), F = registered footprint bytes
  pause_leg_frac_of_link / resume_leg_frac_of_link   bytes that crossed the host link in the leg over
             (leg time x measured hipMemcpy rate): the figures the 80 % target is about;
             both_legs_frac_of_link is the same for the whole cycle (bytes of both legs over both times)
  roofline   the on-device scan kernel (zero flags + checksums) against HBM peak
  link       each leg against the measured hipMemcpy rate of the host link
  link_kernels  the two kernels that take nearly all GPU time, gather-pack and scatter-unpack against pinned
             host memory: bytes per leg, device time, GB/s, fraction of the measured link rate (the gather
             kernel is narrowed on purpose while the copy runs ahead of the unmaps: launches_narrowed)
  first_cycle  times and phases of the very first cycle (pinned pool and engine tables are created in it)
  unmap      what the unmapping thread spends per region (the sum bounds the pause), what one hipMemUnmap costs
             on this machine with nothing else running (idle_us, probed before and after the timed cycles), the floor
             regions x idle_us + scan + plan that no pause of this footprint can beat, and pause_over_floor
  other_configs  configurations 1, 2 and 4 timed the same way for a few cycles each after the headline
  host       where the pinned slabs sit (NUMA node) beside the GPU's own node
  pack_unpack_in_hbm  the pack and unpack kernels with both sides in HBM, against HBM peak
  reference_structure_on_gpu  the reference's loop structure in HIP calls on the same footprint
  cpu_baseline  the reference's serial per-region memcpy path (oracle/) on this box's host cores,
                same footprint
"""
import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
PHASES = ("pause_sync_ms", "pause_scan_ms", "pause_plan_ms", "pause_pool_ms", "pause_scratch_ms", "pause_copy_ms",
          "pause_unmap_ms", "resume_plan_ms", "resume_map_ms", "resume_copy_ms", "resume_peer_ms", "resume_scratch_ms",
          "k1_ms", "k2_ms", "k3_ms")


def cpu_baseline(threads_all, gib):
    """The oracle's restatement of amem_memPause/amem_memResume on host memory, on the footprint the
    GPU run uses (capped at the 10 GiB headline prefix): one thread as the reference runs it, then
    all cores. The reference's structure copies every byte of every region, zero or not."""
    import numpy as np

    import oracle as O
    from asystem_amem_amd.footprint import Footprint

    orc = O.load()
    orc.oracle_reset()
    budget = int(min(gib, 10.0) * (1 << 30)) if gib > 0 else 10 << 30
    fp = Footprint(3, 2, byte_budget=budget, threads=threads_all)
    vas = []
    for i, sz in enumerate(fp.sizes):
        va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert orc.oracle_vmm_alloc(int(sz), C.byref(va), C.byref(h), C.byref(asz)) == 0
        np.frombuffer((C.c_uint8 * int(sz)).from_address(va.value), dtype=np.uint8)[:] = fp.region_bytes(i)
        assert orc.oracle_add_alloc_info(0, va.value, asz.value, 0, 0, h.value, -1, 0, 0, 1) == 0
        vas.append((va.value, asz.value))
    out = {}
    for threads in (1, threads_all):
        orc.oracle_mem_pause_mt(0, threads)  # warm cycle: host buffers are created here
        orc.oracle_mem_resume_mt(0, threads)
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            orc.oracle_mem_pause_mt(0, threads)
            orc.oracle_mem_resume_mt(0, threads)
            times.append(time.perf_counter() - t0)
        out[threads] = 2 * fp.total_bytes / statistics.median(times) / 1e9
    bad = 0
    for i, (va, asz) in enumerate(vas):
        buf = np.frombuffer((C.c_uint8 * int(fp.sizes[i])).from_address(va), dtype=np.uint8)
        bad += fp.check_region(i, buf)
        orc.oracle_del_alloc_info(0, va, 0, 0)
        orc.oracle_vmm_free(va, asz, 0)
    assert bad == 0, "oracle cycle is not bit-exact"
    return {"value": round(out[1], 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "the same footprint as the GPU run (config 3 prefix, %d regions, %.2f GiB) in the oracle's "
                      "host-memory VMM stand-in, p50 of 5 cycles after a warm one" % (len(fp.sizes), fp.total_bytes / 2**30),
            "all_cores": {"value": round(out[threads_all], 3), "cores": threads_all}}


def numa_placement(lib, slab_addr):
    """NUMA node of one pinned slab page beside the GPU's node (sysfs). The reference places its host buffers
    on the GPU's node by hand with an explicit fallback (amem_nccl.h:251-267); here the runtime places them."""
    out = {"nodes_online": None, "gpu_numa_node": None, "slab_numa_node": None}
    try:
        out["nodes_online"] = open("/sys/devices/system/node/online").read().strip()
    except OSError:
        pass
    bdf = C.create_string_buffer(32)
    if lib.amem_device_pci_bus_id(bdf, 32) == 0:
        try:
            out["gpu_pci"] = bdf.value.decode().lower()
            out["gpu_numa_node"] = int(open("/sys/bus/pci/devices/%s/numa_node" % out["gpu_pci"]).read())
        except (OSError, ValueError):
            pass
    if slab_addr:
        try:
            libc = C.CDLL(None, use_errno=True)
            page = C.c_void_p(slab_addr & ~4095)
            status = C.c_int(-999)
            # move_pages(pid 0, one page, no target nodes) only reports where the page is (syscall 279 on x86-64)
            rc = libc.syscall(279, 0, C.c_ulong(1), C.byref(page), None, C.byref(status), 0)
            if rc == 0 and status.value >= 0:
                out["slab_numa_node"] = status.value
            else:
                out["slab_numa_node_unknown"] = ("move_pages rc %d status %d errno %d: the kernel does not report a node for "
                                                 "this kind of mapping" % (rc, status.value, C.get_errno()))
        except Exception as e:  # noqa: BLE001 - a diagnostic must not break the benchmark
            out["slab_numa_node_unknown"] = repr(e)
    if out["nodes_online"] is not None and "-" not in out["nodes_online"] and "," not in out["nodes_online"]:
        out["note"] = "this machine has a single NUMA node: placement cannot be wrong"
    return out


def suballocation_kernels(lib, B, regs, pg):
    """Configuration 4's 100,000 sub-allocations as a descriptor list: gathered out of their granules into one
    device buffer and scattered back by the pack/unpack kernel (device memory on both sides), through the C ABI."""
    g = pg.GRANULE
    n = len(pg.starts)
    sizes = pg.sub.sizes.astype(np.uint64)
    descs = np.empty((n, 3), dtype=np.uint64)
    descs[:, 0] = regs.va[(pg.starts // g).astype(np.int64)] + (pg.starts % g).astype(np.uint64)
    descs[:, 1] = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.uint64)
    descs[:, 2] = sizes
    S = int(sizes.sum())
    sva, sh, sasz = C.c_uint64(), C.c_uint64(), C.c_uint64()
    if lib.amem_vmm_alloc(S, 0, C.byref(sva), C.byref(sh), C.byref(sasz)) != 0:
        return None
    dptr = descs.ctypes.data_as(C.POINTER(B.CopyDesc))
    gms, sms, ms = [], [], C.c_float()
    for _ in range(4):
        assert lib.amem_gather_pack(dptr, n, C.c_void_p(sva.value), S, 0, C.byref(ms)) == 0
        gms.append(ms.value)
        assert lib.amem_scatter_unpack(dptr, n, C.c_void_p(sva.value), S, 0, C.byref(ms)) == 0
        sms.append(ms.value)
    lib.amem_vmm_free(sva.value, sasz.value, sh.value)
    gm, sm = statistics.median(gms[1:]), statistics.median(sms[1:])
    return {"descriptors": n, "packed_bytes": S,
            "gather_pack": {"ms": round(gm, 3), "GBps": round(2 * S / gm / 1e6, 1), "frac_of_hbm_peak": round(2 * S / gm / 1e6 / HBM_PEAK_GBPS, 4)},
            "scatter_unpack": {"ms": round(sm, 3), "GBps": round(2 * S / sm / 1e6, 1), "frac_of_hbm_peak": round(2 * S / sm / 1e6 / HBM_PEAK_GBPS, 4)},
            "what": "move_pieces_hbm over one descriptor per sub-allocation (4-64 KiB each, 2*S bytes per launch: S read + S "
                    "written), p50 of 3 launches after a warm one; the granules' bytes are checked afterwards with the rest"}


def time_config(lib, B, H, fp, warmup, steps, d2h, h2d, extra=None):
    """One footprint through `warmup` untimed and `steps` timed pause/resume cycles, with the correctness gate."""
    regs = H.Regions(lib, fp)
    F = int(regs.alloc.sum())
    va_before, table_before = regs.va.copy(), regs.table()
    pause_s, resume_s, stats = [], [], []
    for step in range(warmup + steps):
        if hasattr(fp, "mutate"):
            regs.write_chunks(fp.mutate(1000 + step))
        t0 = time.perf_counter()
        rc1 = lib.amem_mem_pause(0, 0)
        t1 = time.perf_counter()
        rc2 = lib.amem_mem_resume(0, 0)
        t2 = time.perf_counter()
        assert rc1 == 0 and rc2 == 0, (rc1, rc2)
        if step >= warmup:
            pause_s.append(t1 - t0); resume_s.append(t2 - t1); stats.append(H.cycle_stats(lib))
    more = extra(regs, fp) if extra else None
    bad = regs.mismatched_bytes()
    tdiff = [d for d in H.compare_tables(table_before, regs.table()) if d[1] != "handle_gen"]
    ok = bad == 0 and bool((regs.va == va_before).all()) and not tdiff
    n = len(fp.sizes)
    regs.free()
    lib.amem_pool_trim()
    pp, pr = statistics.median(pause_s), statistics.median(resume_s)
    parked = statistics.mean(s["parked_bytes"] for s in stats)
    return {"regions": n, "footprint_bytes": F, "parked_bytes_per_leg": int(parked), "cycles_timed": steps,
            "p50_pause_s": round(pp, 5), "p50_resume_s": round(pr, 5),
            "effective_GBps": round(2 * F / (pp + pr) / 1e9, 2),
            "pause_leg_frac_of_link": round(parked / pp / 1e9 / d2h, 4),
            "resume_leg_frac_of_link": round(parked / pr / 1e9 / h2d, 4),
            "pause_us_per_region": round(pp * 1e6 / n, 1), "resume_us_per_region": round(pr * 1e6 / n, 1),
            "unmap_us_each_p50": round(statistics.median(s["pause_unmap_ms"] for s in stats) * 1e3 / n, 1),
            "bit_exact": ok, **({"suballocation_kernels": more} if more else {})}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--gib", type=float, default=10.0, help="footprint budget in GiB (headline: 10)")
    ap.add_argument("--config", type=int, default=3, choices=[1, 2, 3, 4],
                    help="benchmark configuration: 3 (default) is the one the metric is quoted on; 1, 2 and 4 "
                         "time the other single-process footprints the same way")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-reference-structure", action="store_true")
    ap.add_argument("--no-hbm-kernels", action="store_true", help="skip the pack/unpack-in-HBM measurement")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the short runs of configurations 1, 2 and 4")
    ap.add_argument("--pause-path", type=int, default=None)
    ap.add_argument("--opt", action="append", default=[], help="engine tunable, name=value (see amem_set_option)")
    ap.add_argument("--calib", action="store_true",
                    help="also run the plain 1 GiB copy kernel once, so that a counter profile of this command "
                         "holds a kernel of known HBM traffic (1 GiB read + 1 GiB written)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the pause/resume engine has no multi-GPU path "
                 "(each GPU would run its own independent engine); run with --gpus 1")

    from asystem_amem_amd import binding as B
    from asystem_amem_amd import harness as H
    from asystem_amem_amd.footprint import Footprint

    H.enable_env()
    import __graft_entry__
    __graft_entry__.ensure_built()      # loads what is built; compiles only if a library is missing
    lib = B.load()
    if lib.amem_device_count() < 1:
        sys.exit("bench.py needs a GPU")
    if args.pause_path is not None:
        lib.amem_set_option(b"pause_path", args.pause_path)
    for kv in args.opt:
        k, v = kv.split("=")
        assert lib.amem_set_option(k.encode(), int(v)) == 0, kv
    host_cpus = os.cpu_count() or 1
    host_threads = min(16, host_cpus)     # a GPU box gives one GPU's job a 16-core share whatever it reports

    d2h, h2d = C.c_double(), C.c_double()
    assert lib.amem_probe_link(1 << 30, 3, C.byref(d2h), C.byref(h2d)) == 0

    if args.calib:
        ms = C.c_float()
        assert lib.amem_calib_copy(1 << 30, 3, C.byref(ms)) == 0

    # What one hipMemUnmap costs here with nothing running: 64 mappings of 2 MiB, accessible, device idle.
    idle_p50, idle_mean, map_mean = C.c_double(), C.c_double(), C.c_double()
    assert lib.amem_probe_unmap(64, 2 << 20, C.byref(idle_p50), C.byref(idle_mean), C.byref(map_mean)) == 0
    assert lib.amem_probe_unmap(64, 2 << 20, C.byref(idle_p50), C.byref(idle_mean), C.byref(map_mean)) == 0  # (second pass: warm)

    if args.config == 3:
        fp = Footprint(3, 2, byte_budget=int(args.gib * (1 << 30)), threads=host_threads)
        workload = ("config 3 headline: training-rank footprint, %d regions log-uniform [2,64) MiB, %.2f GiB, 30%% zero "
                    "64 KiB chunks, seed 2, 1%% of chunks rewritten between cycles")
    elif args.config == 2:
        fp = Footprint(2, 1, threads=host_threads)
        workload = ("config 2: inference-rank footprint, %d regions (128x4 + 96x2 + 32x16 MiB), %.2f GiB, 50%% zero "
                    "64 KiB chunks, seed 1, 1%% of chunks rewritten between cycles")
    elif args.config == 1:
        fp = Footprint(1, 0, threads=host_threads)
        workload = "config 1: %d regions of 2 MiB x U{1..16}, %.2f GiB, no zero chunks, seed 0, 1%% of chunks rewritten between cycles"
    else:
        from asystem_amem_amd.footprint import PackedGranules
        fp = PackedGranules(3, 100000, threads=host_threads)
        workload = ("config 4: 100,000 sub-allocations of 4-64 KiB (seed 3) packed into %d granules of 2 MiB, %.2f GiB, "
                    "every granule one tracked region")
    regs = H.Regions(lib, fp)
    F = int(regs.alloc.sum())
    va_before = regs.va.copy()
    table_before = regs.table()

    cycle_no = [0]

    def run_cycles(warmup, steps):
        pause_s, resume_s, stats, first = [], [], [], None
        for step in range(warmup + steps):
            if hasattr(fp, "mutate"):
                touched = fp.mutate(cycle_no[0])  # writes between cycles, outside the clock
                regs.write_chunks(touched)
            cycle_no[0] += 1
            t0 = time.perf_counter()
            rc1 = lib.amem_mem_pause(0, 0)
            t1 = time.perf_counter()
            rc2 = lib.amem_mem_resume(0, 0)
            t2 = time.perf_counter()
            assert rc1 == 0 and rc2 == 0, (rc1, rc2)
            if step >= warmup:
                pause_s.append(t1 - t0)
                resume_s.append(t2 - t1)
                stats.append(H.cycle_stats(lib))
            elif step == 0:
                first = (t1 - t0, t2 - t1, H.cycle_stats(lib))
        return pause_s, resume_s, stats, first

    pause_s, resume_s, stats, first = run_cycles(args.warmup, args.steps)

    # The reference's own structure expressed in HIP calls (one waited-for whole-region copy per
    # region each way, no scan, no elision), on the same footprint, for comparison only.
    ref_struct = None
    if not args.no_reference_structure and args.config == 3:
        path_was = lib.amem_get_option(b"pause_path")
        assert lib.amem_set_option(b"pause_path", 4) == 0
        rp, rr, _, _ = run_cycles(1, 5)
        assert lib.amem_set_option(b"pause_path", path_was) == 0
        ref_struct = {"value": round(2 * F / statistics.median(a + b for a, b in zip(rp, rr)) / 1e9, 3), "unit": "GB/s",
                      "p50_pause_s": round(statistics.median(rp), 4), "p50_resume_s": round(statistics.median(rr), 4),
                      "what": "amem_memPause/amem_memResume loop structure of the reference (amem_nccl.cpp:502-558, "
                              ":604-630) written with hipMemcpyAsync + sync per region on this GPU; p50 of 5 cycles"}

    # The gather kernel at its full width: the default pause narrows it on purpose while it is ahead of the
    # unmaps, which lowers its own rate and shortens the pause. Four extra cycles with the narrowing off show
    # what the kernel does when left alone, and what the pause then costs (outside the timed region).
    full_width = None
    if args.config == 3 and lib.amem_get_option(b"pause_adaptive") == 1 and lib.amem_get_option(b"pause_path") in (2, 3):
        assert lib.amem_set_option(b"pause_adaptive", 0) == 0
        fp_s, _, fst, _ = run_cycles(1, 4)
        assert lib.amem_set_option(b"pause_adaptive", 1) == 0
        fk2 = statistics.median(s_["k2_ms"] for s_ in fst)
        fkb = statistics.mean(s_["kernel_bytes"] for s_ in fst)
        full_width = {"device_ms_per_pause": round(fk2, 3), "GBps": round(fkb / fk2 / 1e6, 2),
                      "frac_of_measured_d2h": round(fkb / fk2 / 1e6 / d2h.value, 4),
                      "p50_pause_s": round(statistics.median(fp_s), 4),
                      "unmap_us_each_p50": round(statistics.median(s_["pause_unmap_ms"] for s_ in fst) * 1e3 / len(fp.sizes), 1),
                      "what": "the same kernel with every launch 8 workgroups wide (pause_adaptive=0), p50 of 4 cycles after "
                              "the timed ones: the kernel itself is faster, each unmap beside it costs more, the pause is longer"}

    # The pack and unpack kernels on their own against the HBM roofline: the footprint's non-zero runs
    # gathered into one device buffer and scattered back (S read + S written each way), through the C ABI.
    hbm_kernels = None
    descs, S = H.nonzero_runs(fp, regs.va) if args.config == 3 else (None, 0)
    sva, sh, sasz = C.c_uint64(), C.c_uint64(), C.c_uint64()
    if S and not args.no_hbm_kernels and lib.amem_vmm_alloc(S, 0, C.byref(sva), C.byref(sh), C.byref(sasz)) == 0:
        dptr = descs.ctypes.data_as(C.POINTER(B.CopyDesc))
        gms, sms, ms = [], [], C.c_float()
        for _ in range(4):
            assert lib.amem_gather_pack(dptr, len(descs), C.c_void_p(sva.value), S, 0, C.byref(ms)) == 0
            gms.append(ms.value)
            assert lib.amem_scatter_unpack(dptr, len(descs), C.c_void_p(sva.value), S, 0, C.byref(ms)) == 0
            sms.append(ms.value)
        lib.amem_vmm_free(sva.value, sasz.value, sh.value)
        g, s_ = statistics.median(gms[1:]), statistics.median(sms[1:])
        hbm_kernels = {"packed_bytes": S, "descriptors": len(descs),
                       "gather_pack": {"ms": round(g, 3), "GBps": round(2 * S / g / 1e6, 1),
                                       "frac_of_hbm_peak": round(2 * S / g / 1e6 / HBM_PEAK_GBPS, 4)},
                       "scatter_unpack": {"ms": round(s_, 3), "GBps": round(2 * S / s_ / 1e6, 1),
                                          "frac_of_hbm_peak": round(2 * S / s_ / 1e6 / HBM_PEAK_GBPS, 4)},
                       "what": "the pack/unpack kernel in its device-memory shape (move_pieces_hbm: 4 KiB per 128-lane "
                               "workgroup) with a device-side buffer: 2*S bytes (S read + S written) per launch, "
                               "p50 of 3 launches after a warm one; the bytes are checked afterwards with the rest"}

    # the same probe again after the timed cycles: the cost of the call drifts on these machines
    idle_after = C.c_double()
    assert lib.amem_probe_unmap(64, 2 << 20, C.byref(idle_after), None, None) == 0
    slab_addr = next((t["cpu_addr"] for t in regs.table().values() if t["cpu_addr"]), 0)
    numa = numa_placement(lib, slab_addr)

    # correctness gate, outside the clock: bytes, addresses, table
    bad = regs.mismatched_bytes()
    same_va = bool((regs.va == va_before).all())
    table_after = regs.table()
    tdiff = [d for d in H.compare_tables(table_before, table_after) if d[1] != "handle_gen"]
    ctr = H.counters(lib)
    ok = bad == 0 and same_va and not tdiff and ctr["offload_cnt"] == 0 and ctr["pause_cnt"] == ctr["resume_cnt"]

    total = sum(pause_s) + sum(resume_s)
    K = len(pause_s)
    p50_pause, p50_resume = statistics.median(pause_s), statistics.median(resume_s)
    parked = statistics.mean(s["parked_bytes"] for s in stats)
    k1_ms = sum(s["k1_ms"] for s in stats) / max(1, sum(s["k1_launches"] for s in stats))
    k1_achieved = F / (k1_ms * 1e-3) / 1e9
    # HBM traffic of the scan kernel is not something this run can measure (it takes two rocprofv3 --pmc
    # runs of this very command); the figure of the committed counter profile is passed on, labelled,
    # when it was taken on the same footprint.
    traffic, traffic_from = None, None
    tpath = os.path.join(ROOT, "profiles", "scan_chunks_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            t = json.load(f)
        if t.get("footprint_bytes") == F:
            traffic = t.get("hbm_bytes_per_launch")
            traffic_from = "profiles/scan_chunks_traffic.json (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of this command; not measured by this run)"
    k2_ms = statistics.median(s["k2_ms"] for s in stats)
    k3_ms = statistics.median(s["k3_ms"] for s in stats)
    kbytes = statistics.mean(s["kernel_bytes"] for s in stats)
    PCIE_GEN5_X16 = 63.0
    idle_us = min(idle_p50.value, idle_after.value)
    pause_floor = (len(fp.sizes) * idle_us * 1e-6 +
                   statistics.median(s["pause_scan_ms"] + s["pause_plan_ms"] + s["pause_sync_ms"] for s in stats) * 1e-3)
    pause_frac = parked / p50_pause / 1e9 / d2h.value
    resume_frac = parked / p50_resume / 1e9 / h2d.value
    out = {
        "metric": "pause+resume GB/s and p50 latency (s), 10 GiB footprint, 1 MI355X",
        "value": round(2 * F * K / total / 1e9, 3),
        "unit": "GB/s",
        "pause_leg_frac_of_link": round(pause_frac, 4),
        "resume_leg_frac_of_link": round(resume_frac, 4),
        "both_legs_frac_of_link": round(2 * parked / (p50_pause + p50_resume) / 1e9 / ((d2h.value + h2d.value) / 2), 4),
        "leg_frac_target": 0.8,
        "legs_meeting_target": [n for n, f in (("pause", pause_frac), ("resume", resume_frac)) if f >= 0.8],
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": round(total / K * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": workload % (len(fp.sizes), F / 2**30),
                   "footprint_bytes": F, "regions": len(fp.sizes), "parked_bytes_per_leg": int(parked)},
        "p50_pause_s": round(p50_pause, 4),
        "p50_resume_s": round(p50_resume, 4),
        "p50_cycle_s": round(statistics.median(a + b for a, b in zip(pause_s, resume_s)), 4),
        "max_pause_s": round(max(pause_s), 4), "max_resume_s": round(max(resume_s), 4),
        "first_cycle_s": {"pause": round(first[0], 4), "resume": round(first[1], 4)} if args.warmup else None,
        "first_cycle": {"pause_s": round(first[0], 4), "resume_s": round(first[1], 4),
                        "phases_ms": {k: round(first[2][k], 3) for k in PHASES},
                        "slab_bytes": first[2]["slab_bytes"],
                        "what": "the process's first pause grows the pinned pool from nothing (pause_pool_ms) and creates "
                                "the engine's tables and events (pause_scratch_ms, resume_scratch_ms); later cycles reuse both"}
        if args.warmup else None,
        "pause_GBps": round(F / p50_pause / 1e9, 3),
        "resume_GBps": round(F / p50_resume / 1e9, 3),
        "bit_exact": ok,
        "roofline": {"kernel": "scan_chunks (zero flags + checksums)", "bound": "hbm",
                     "achieved": round(k1_achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(k1_achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_from": traffic_from,
                     "avg_launch_ms": round(k1_ms, 4), "algorithmic_bytes_per_launch": F,
                     "why_this_kernel": "the one kernel of a cycle that is bound by HBM; the two kernels that take over 99 % "
                                        "of a cycle's GPU time move bytes over the host link, which is neither an HBM nor an MFMA "
                                        "roofline: they are under link_kernels, against the measured link rate"},
        "link": {"measured_d2h_GBps": round(d2h.value, 2), "measured_h2d_GBps": round(h2d.value, 2),
                 "pause_leg_frac": round(pause_frac, 4),
                 "resume_leg_frac": round(resume_frac, 4),
                 "pause_copy_phase_frac": round(parked / (statistics.median(s["pause_copy_ms"] for s in stats) * 1e-3)
                                                / 1e9 / d2h.value, 4),
                 "resume_copy_phase_frac": round(parked / (statistics.median(s["resume_copy_ms"] for s in stats) * 1e-3)
                                                 / 1e9 / h2d.value, 4)},
        "link_kernels": {
            "move_tiles<0> (gather-pack into pinned host memory, 4 to 8 workgroups on one XCD, unmaps running beside it)": {
                "bound": "host link D2H", "bytes_per_pause": int(kbytes), "launches_per_pause": int(statistics.median(s["k2_launches"] for s in stats)),
                "launches_narrowed": int(statistics.median(s["pause_narrow_launches"] for s in stats)),
                "device_ms_per_pause": round(k2_ms, 3), "GBps": round(kbytes / k2_ms / 1e6, 2) if k2_ms else None,
                "frac_of_measured_d2h": round(kbytes / k2_ms / 1e6 / d2h.value, 4) if k2_ms else None,
                "frac_of_pcie_gen5_x16": round(kbytes / k2_ms / 1e6 / PCIE_GEN5_X16, 4) if k2_ms else None},
            "move_tiles<1> (scatter-unpack + zero fill from pinned host memory, 96 workgroups)": {
                "bound": "host link H2D", "bytes_per_resume": int(parked), "launches_per_resume": int(statistics.median(s["k3_launches"] for s in stats)),
                "device_ms_per_resume": round(k3_ms, 3), "GBps": round(parked / k3_ms / 1e6, 2) if k3_ms else None,
                "frac_of_measured_h2d": round(parked / k3_ms / 1e6 / h2d.value, 4) if k3_ms else None,
                "frac_of_pcie_gen5_x16": round(parked / k3_ms / 1e6 / PCIE_GEN5_X16, 4) if k3_ms else None},
            "gather_at_full_width": full_width,
            "what": "device time from HIP events on the launch stream (first launch to last, the sum over a leg's launches); "
                    "these two kernels are over 99 % of the GPU time of a cycle, the scan kernel of `roofline` under 1 %"},
        "unmap": {"regions": len(fp.sizes), "us_each_p50": round(statistics.median(s["pause_unmap_ms"] for s in stats)
                                                                   * 1e3 / max(len(fp.sizes), 1), 1),
                  "idle_us": round(idle_us, 1), "idle_us_before": round(idle_p50.value, 1), "idle_us_after": round(idle_after.value, 1),
                  "create_map_access_us": round(map_mean.value, 1),
                  "pause_floor_s": round(pause_floor, 4), "pause_over_floor": round(p50_pause / pause_floor, 3),
                  "what": "us_each_p50: time the unmapping thread spends per region (hipMemUnmap beside the gather kernel); "
                          "the sum bounds the pause. idle_us: one hipMemUnmap of an accessible 2 MiB mapping with nothing else "
                          "running, p50 of 64, probed before and after the timed cycles (the lower of the two). pause_floor_s = regions x idle_us + scan + "
                          "plan + sync: every mapping has to be unmapped inside the pause and the runtime serialises the calls. "
                          "pause_over_floor = p50_pause_s / pause_floor_s"},
        "phases_ms_p50": {k: round(statistics.median(s[k] for s in stats), 3) for k in PHASES},
        "host": dict({"cpus_reported": host_cpus, "threads_used": host_threads},
                     **{k: v for k, v in numa.items()}),
    }
    if hbm_kernels:
        out["pack_unpack_in_hbm"] = hbm_kernels
    if ref_struct:
        out["reference_structure_on_gpu"] = ref_struct
        out["speedup_vs_reference_structure"] = round(out["value"] / ref_struct["value"], 3)
    regs.free()
    lib.amem_pool_trim()
    if not args.no_other_configs and args.config == 3:
        from asystem_amem_amd.footprint import PackedGranules
        others = {}
        for name, make in (("config_1", lambda: Footprint(1, 0, threads=host_threads)),
                           ("config_2", lambda: Footprint(2, 1, threads=host_threads)),
                           ("config_4", lambda: PackedGranules(3, 100000, threads=host_threads))):
            extra = (lambda r, f: suballocation_kernels(lib, B, r, f)) if name == "config_4" else None
            others[name] = time_config(lib, B, H, make(), 1, 5, d2h.value, h2d.value, extra)
            ok = ok and others[name]["bit_exact"]
        others["what"] = ("the other single-process configurations of the benchmark, 5 timed cycles each after a warm one, "
                          "1 % of chunks rewritten between cycles where the footprint has a generator for it: config 1 = 64 "
                          "regions of 2 MiB x U{1..16}, no zero chunks, seed 0; config 2 = inference rank, 128x4 + 96x2 + 32x16 "
                          "MiB, 50 % zero chunks, seed 1; config 4 = 100,000 sub-allocations of 4-64 KiB packed into 2 MiB "
                          "granules, every granule one region, seed 3. Pause time follows the number of regions (one "
                          "hipMemUnmap each), not the bytes")
        out["other_configs"] = others
        out["bit_exact"] = ok
    if not args.no_cpu_baseline and args.config == 3:
        out["cpu_baseline"] = cpu_baseline(host_threads, args.gib)
        out["cpu_baseline"]["host_cpus_reported"] = host_cpus
    print(json.dumps(out), flush=True)
    if not ok:
        sys.exit("bench.py: correctness gate failed (mismatched bytes %d, same_va %s, table diffs %s)" %
                 (bad, same_va, tdiff[:3]))


if __name__ == "__main__":
    main()
