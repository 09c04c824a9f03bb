#!/usr/bin/env python3
"""Benchmark of the pause/resume path on one MI355X.

A step is one pause + resume cycle of the training-rank footprint: the shortest prefix of
the 2,560 log-uniform [2, 64) MiB draws (seed 2) that reaches 10 GiB — 572 regions,
10.02 GiB — with 30 % all-zero 64 KiB chunks, and writes to 1 % of the chunks between
cycles. The footprint is resident in HBM before the clock starts; the clock covers the
two calls amem_mem_pause() and amem_mem_resume() and nothing else.

Prints one JSON line:
  value      2 * F / (t_pause + t_resume), GB/s (1e9), F = registered footprint bytes
  roofline   the on-device scan kernel (zero flags + checksums) against HBM peak
  link       each leg against the measured hipMemcpy rate of the host link
  unmap      what the unmapping thread spends per region (the sum bounds the pause)
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

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--gib", type=float, default=10.0, help="footprint budget in GiB (headline: 10)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-reference-structure", action="store_true")
    ap.add_argument("--no-hbm-kernels", action="store_true", help="skip the pack/unpack-in-HBM measurement")
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
    host_threads = min(16, os.cpu_count() or 1)

    d2h, h2d = C.c_double(), C.c_double()
    assert lib.amem_probe_link(1 << 30, 3, C.byref(d2h), C.byref(h2d)) == 0

    if args.calib:
        ms = C.c_float()
        assert lib.amem_calib_copy(1 << 30, 3, C.byref(ms)) == 0

    fp = Footprint(3, 2, byte_budget=int(args.gib * (1 << 30)), threads=host_threads)
    regs = H.Regions(lib, fp)
    F = int(regs.alloc.sum())
    va_before = regs.va.copy()
    table_before = regs.table()

    cycle_no = [0]

    def run_cycles(warmup, steps):
        pause_s, resume_s, stats, first = [], [], [], None
        for step in range(warmup + steps):
            touched = fp.mutate(cycle_no[0])  # writes between cycles, outside the clock
            cycle_no[0] += 1
            regs.write_chunks(touched)
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
                first = (t1 - t0, t2 - t1)
        return pause_s, resume_s, stats, first

    pause_s, resume_s, stats, first = run_cycles(args.warmup, args.steps)

    # The reference's own structure expressed in HIP calls (one waited-for whole-region copy per
    # region each way, no scan, no elision), on the same footprint, for comparison only.
    ref_struct = None
    if not args.no_reference_structure:
        path_was = lib.amem_get_option(b"pause_path")
        assert lib.amem_set_option(b"pause_path", 4) == 0
        rp, rr, _, _ = run_cycles(1, 5)
        assert lib.amem_set_option(b"pause_path", path_was) == 0
        ref_struct = {"value": round(2 * F / statistics.median(a + b for a, b in zip(rp, rr)) / 1e9, 3), "unit": "GB/s",
                      "p50_pause_s": round(statistics.median(rp), 4), "p50_resume_s": round(statistics.median(rr), 4),
                      "what": "amem_memPause/amem_memResume loop structure of the reference (amem_nccl.cpp:502-558, "
                              ":604-630) written with hipMemcpyAsync + sync per region on this GPU; p50 of 5 cycles"}

    # The pack and unpack kernels on their own against the HBM roofline: the footprint's non-zero runs
    # gathered into one device buffer and scattered back (S read + S written each way), through the C ABI.
    hbm_kernels = None
    descs, S = H.nonzero_runs(fp, regs.va)
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
                       "what": "move_tiles with a device-side buffer: 2*S bytes (S read + S written) per launch, "
                               "p50 of 3 launches after a warm one; the bytes are checked afterwards with the rest"}

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
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "scan_chunks_traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            t = json.load(f)
        if t.get("footprint_bytes") == F:
            traffic = t.get("hbm_bytes_per_launch")
    out = {
        "metric": "pause+resume GB/s and p50 latency (s), 10 GiB footprint, 1 MI355X",
        "value": round(2 * F * K / total / 1e9, 3),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": round(total / K * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "config 3 headline: training-rank footprint, %d regions log-uniform [2,64) MiB, "
                               "%.2f GiB, 30%% zero 64 KiB chunks, seed 2, 1%% of chunks rewritten between cycles"
                               % (len(fp.sizes), F / 2**30),
                   "footprint_bytes": F, "regions": len(fp.sizes), "parked_bytes_per_leg": int(parked)},
        "p50_pause_s": round(p50_pause, 4),
        "p50_resume_s": round(p50_resume, 4),
        "p50_cycle_s": round(statistics.median(a + b for a, b in zip(pause_s, resume_s)), 4),
        "first_cycle_s": {"pause": round(first[0], 4), "resume": round(first[1], 4)} if args.warmup else None,
        "pause_GBps": round(F / p50_pause / 1e9, 3),
        "resume_GBps": round(F / p50_resume / 1e9, 3),
        "bit_exact": ok,
        "roofline": {"kernel": "scan_chunks (zero flags + checksums)", "bound": "hbm",
                     "achieved": round(k1_achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(k1_achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "avg_launch_ms": round(k1_ms, 4), "algorithmic_bytes_per_launch": F},
        "link": {"measured_d2h_GBps": round(d2h.value, 2), "measured_h2d_GBps": round(h2d.value, 2),
                 "pause_leg_frac": round(parked / p50_pause / 1e9 / d2h.value, 4),
                 "resume_leg_frac": round(parked / p50_resume / 1e9 / h2d.value, 4),
                 "pause_copy_phase_frac": round(parked / (statistics.median(s["pause_copy_ms"] for s in stats) * 1e-3)
                                                / 1e9 / d2h.value, 4),
                 "resume_copy_phase_frac": round(parked / (statistics.median(s["resume_copy_ms"] for s in stats) * 1e-3)
                                                 / 1e9 / h2d.value, 4)},
        "unmap": {"regions": len(fp.sizes), "us_each_p50": round(statistics.median(s["pause_unmap_ms"] for s in stats)
                                                                   * 1e3 / max(len(fp.sizes), 1), 1),
                  "what": "time the unmapping thread spends per region (hipMemUnmap beside the gather kernel); "
                          "the sum bounds the pause"},
        "phases_ms_p50": {k: round(statistics.median(s[k] for s in stats), 3) for k in (
            "pause_scan_ms", "pause_plan_ms", "pause_copy_ms", "pause_unmap_ms", "resume_map_ms", "resume_copy_ms",
            "k1_ms", "k2_ms", "k3_ms")},
    }
    if hbm_kernels:
        out["pack_unpack_in_hbm"] = hbm_kernels
    if ref_struct:
        out["reference_structure_on_gpu"] = ref_struct
        out["speedup_vs_reference_structure"] = round(out["value"] / ref_struct["value"], 3)
    regs.free()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(host_threads, args.gib)
    print(json.dumps(out), flush=True)
    if not ok:
        sys.exit("bench.py: correctness gate failed (mismatched bytes %d, same_va %s, table diffs %s)" %
                 (bad, same_va, tdiff[:3]))


if __name__ == "__main__":
    main()
