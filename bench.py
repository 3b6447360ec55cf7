#!/usr/bin/env python3
"""Benchmark of the alltoallv hot path on one MI355X.

A "step" is one complete collective call (planning kernels + every data-moving launch +
stream synchronisation) over one synthetic batch that is already resident in HBM.  Default
workload: benchmark configuration 4 — TTPL_BT_alltoallv, P = 1024 virtual ranks, 32 per node, r = 32,
1-byte elements, counts ~ Normal(4096, 1024) clipped to [0, 16384].

Prints ONE JSON line: effective GB/s (payload bytes / time), the HBM roofline of the copy
kernel (algorithmic bytes = one read + one write per hop, timed with HIP events on the
communicator's stream) and a CPU baseline measured on this box's host cores.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import subprocess
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from rbruck_alltoallv_amd import workloads as W  # noqa: E402

HBM_PEAK_GBPS = 8000.0
METRIC = "effective alltoallv GB/s + % HBM peak, P=64..1024 virtual ranks, 1 GPU"
# the sources the copy kernels are built from: a counter profile under profiles/ is only quoted while they are unchanged
KERNEL_SOURCES = ("vc_copy.hip", "vc_plan.hip", "vc_plan_math.h", "vc_common.h", "vc_scan.h", "vc_dispatch.h")


def kernel_sources_sha() -> str:
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "rbruck_alltoallv_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic(kernel: str, workload_name: str):
    """HBM bytes per launch of `kernel` on `workload_name` as rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE measured them (each
    scaled by what the same counter reads for a plain copy of known size), read from the committed summary
    profiles/<kernel>_<workload>_pmc_fetch_write.txt.  Counters cannot be read from inside this process, so this is the
    figure of the profiled run of the same command; None when there is no summary or when the kernel sources have
    changed since (the summary names the hash they had)."""
    path = os.path.join(ROOT, "profiles", f"{kernel}_{workload_name}_pmc_fetch_write.txt")
    if not os.path.exists(path):
        return None, None
    traffic = sha = None
    for line in open(path):
        w = line.split()
        if len(w) == 2 and w[0] == "traffic_bytes_per_launch":
            traffic = int(w[1])
        if len(w) == 2 and w[0] == "kernel_sources_sha256":
            sha = w[1]
    if traffic is None or sha != kernel_sources_sha():
        return None, os.path.basename(path) + " (stale: kernel sources changed since)" if traffic is not None else None
    return traffic, os.path.basename(path)


def workload(name: str, seed: int):
    """(counts, esz, function name, tunables, hop matrix) of one of the five benchmark configurations, or of one of the reference's
    own communication-pattern matrices (ML<P>: inputs/<P>proc, 1-byte elements, twophase_rbruck_alltoallv as in
    examples/MLinputs_example.cpp:96)."""
    if name.startswith("ML"):
        P = int(name[2:])
        counts = W.counts_from_npz(os.path.join(ROOT, "tests", "golden", "inputs", f"global_comm_pattern_{P}proc.npz"))
        r = min(32, P)
        return counts, 1, "twophase_rbruck_alltoallv", dict(r=r), W.hops_flat(P, r)
    if name.startswith("S"):
        # configuration 4's shape with short blocks, S<bytes>: counts uniform in 0..bytes (what the Bruck family exists for)
        counts = W.counts_uniform_random(1024, int(name[1:]), seed)
        return counts, 1, "TTPL_BT_alltoallv_s1", dict(n=32, r=32, bblock=0), W.hops_twolayer(1024, 32, 32)
    if name.startswith("U"):
        # equal blocks of U<bytes> bytes at configuration 4's shape: separates the cost of variable, unaligned blocks
        counts = np.full((1024, 1024), int(name[1:]), dtype=np.int32)
        return counts, 1, "TTPL_BT_alltoallv", dict(n=32, r=32, bblock=0), W.hops_twolayer(1024, 32, 32)
    if name.startswith("C4m"):
        # configuration 4 with every count rounded to a multiple of C4m<bytes>: sources and destinations then share their
        # phase modulo that many bytes, which prices the byte phases of the real configuration
        m = int(name[3:])
        counts = ((W.config_counts("C4", seed)[0] + m // 2) // m * m).astype(np.int32)
        return counts, 1, "TTPL_BT_alltoallv", dict(n=32, r=32, bblock=0), W.hops_twolayer(1024, 32, 32)
    counts, esz, tun = W.config_counts(name, seed)
    P = counts.shape[0]
    if name == "C4":
        return counts, esz, "TTPL_BT_alltoallv", dict(n=32, r=32, bblock=0), W.hops_twolayer(P, 32, 32)
    if name == "C5":
        return counts, esz, "tuna_algorithm", dict(r=32, b=0), W.hops_flat(P, 32)
    if name == "C3":
        return counts, esz, "twophase_rbruck_alltoallv", dict(r=16), W.hops_flat(P, 16)
    if name == "C2":
        return counts, esz, "twophase_rbruck_alltoallv", dict(r=tun["r"]), W.hops_flat(P, tun["r"])
    raise SystemExit(f"unknown workload {name}")


def call(api, func, tun, dp, send, recv):
    if func == "TTPL_BT_alltoallv":
        return api.TTPL_BT_alltoallv(tun["n"], tun["r"], tun["bblock"], dp, send, recv)
    if func == "TTPL_BT_alltoallv_s1":
        return api.TTPL_BT_alltoallv_s1(tun["n"], tun["r"], tun["bblock"], dp, send, recv)
    if func == "TTPL_rbruck_alltoallv":
        return api.TTPL_rbruck_alltoallv(tun["n"], tun["r"], dp, send, recv)
    if func == "tuna_algorithm":
        return api.tuna_algorithm(tun["r"], tun["b"], dp, send, recv)
    if func == "twophase_rbruck_alltoallv":
        return api.twophase_rbruck_alltoallv(tun["r"], dp, send, recv)
    if func == "twophase_rbruck_alltoallv_om":
        return api.twophase_rbruck_alltoallv_om(tun["r"], dp, send, recv)
    raise SystemExit(func)


def short_block_context(api, torch) -> dict:
    """Context beside the metric: blocking calls at the other end of the metric's range of rank counts and at the block sizes
    the Bruck family exists for (short ones), microseconds per call by wall clock.  `default` is the library's default
    mode after its first call on the communicator, `through_list` forces the work-item list (vc_comm_set_forwarding 2)."""
    out = {}
    for key, P, hi, what, fn in (
            ("P64_blocks_0_4096B_twophase_r2", 64, 4096, "benchmark configuration 2", lambda dp, s, d: api.twophase_rbruck_alltoallv(2, dp, s, d)),
            ("P1024_blocks_0_512B_ttpl_n32_r32", 1024, 512, "configuration 4's shape with short blocks", lambda dp, s, d: api.TTPL_BT_alltoallv_s1(32, 32, 0, dp, s, d)),
            ("P1024_blocks_0_16B_ttpl_n32_r32", 1024, 16, "configuration 4's shape with very short blocks", lambda dp, s, d: api.TTPL_BT_alltoallv_s1(32, 32, 0, dp, s, d))):
        prob = W.make_problem(W.counts_uniform_random(P, hi, seed=0), 1, 0, 0)
        dp = api.DeviceProblem(prob)
        send, recv = dp.new_send_arena(), dp.new_recv_arena()
        dp.fill_payload(0, 0, send)
        entry = {"workload": what, "payload_bytes": int(prob.payload_bytes)}
        for label, mode in (("default", 1), ("through_list", 2)):
            dp.comm.set_forwarding(mode)
            for _ in range(3):
                assert fn(dp, send, recv) == 0, dp.comm.error()
            reps = 200 if P <= 64 else 30
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                fn(dp, send, recv)
            entry[label + "_us_per_call"] = round((time.perf_counter() - t0) / reps * 1e6, 1)
            if mode == 1:
                st = dp.comm.last_stats()
                entry["default_kernel"] = kernel_name(st)
        entry["mismatched_bytes"] = int(dp.verify(send, recv))
        out[key] = entry
        dp.comm.free()
    return out


def cpu_sample(name: str, seed: int):
    """The bounded sample of workload `name` the CPU leg runs: (rank count, counts, element size, the reference driver's function
    name and arguments, this library's function name and tunables, what differs from the workload)."""
    sample_P = {"C4": 256, "C5": 512, "C3": 256, "C2": 64}[name]
    if name == "C4":
        return (sample_P, W.counts_normal(sample_P, 4096.0, 1024.0, 0, 16384, seed), 1, "ttpl", dict(r=32, b=0, n=32, bblock=0),
                "TTPL_BT_alltoallv", dict(n=32, r=32, bblock=0),
                "same count distribution at a quarter of the ranks (the box caps processes near 1000)")
    if name == "C5":
        return (sample_P, W.counts_fft_rows(sample_P, 32, 16384), 8, "tuna", dict(r=32, b=0, n=0, bblock=0),
                "tuna_algorithm", dict(r=32, b=0), "the configuration's rank count and pattern, blocks of 128 KiB instead of 1 MiB")
    if name == "C3":
        return (sample_P, W.counts_zipf(sample_P, 65536, 1.2, 5, seed), 4, "twophase", dict(r=16, b=0, n=0, bblock=0),
                "twophase_rbruck_alltoallv", dict(r=16), "the configuration itself")
    return (sample_P, W.counts_uniform_random(sample_P, 4096, seed), 1, "twophase", dict(r=2, b=0, n=0, bblock=0),
            "twophase_rbruck_alltoallv", dict(r=2), "the configuration itself")


def cpu_reference_leg(name: str, seed: int, budget_s: float) -> dict:
    """The same algorithm on this box's host cores, on a bounded sample of the workload.  Runs BEFORE this process touches
    the GPU (it starts child processes and needs nothing from the device).

    Preferred: the real reference functions (oracle/_ref/ref_driver, built in the build container from the
    reference's own sources) under `mpiexec -n P`, timed the reference's way (MPI_Wtime around the call, maximum
    over ranks, examples/rbruckv_example.cpp:101-131).  Configurations 2, 3 and 5 run at their real rank counts (64, 256,
    512; configuration 5 with blocks of 128 KiB instead of 1 MiB, which bounds the time).  The box allows ~1000 processes,
    so configuration 4 (1024 ranks) keeps its shape at P = 256 ranks (8 nodes of 32).  Fallback: the single-threaded C
    restatement (oracle/), "port".  The per-rank digests of what the CPU side received are kept: same_run_parity()
    runs the GPU path on the same sample afterwards and compares.
    """
    from oracle import oracle_py as O
    if name not in ("C2", "C3", "C4", "C5"):
        return {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "not measured for this workload"}
    sample_P, counts, esz, func, args, gpu_func, gpu_tun, what = cpu_sample(name, seed)
    payload = int(counts.astype(np.int64).sum()) * esz
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except Exception:
        pass
    sample = f"{func} P={sample_P}, {what}, payload {payload / 1e6:.1f} MB"
    keep = {"_counts": counts, "_esz": esz, "_gpu_func": gpu_func, "_gpu_tun": gpu_tun, "_seed": seed}
    if os.path.exists(O.REF_DRIVER) and os.path.exists(O.MPIEXEC):
        try:
            with tempfile.TemporaryDirectory() as tmp:
                cf = os.path.join(tmp, "counts.bin")
                counts.astype("<i4").tofile(cf)
                out = os.path.join(tmp, "out")
                cmd = [O.MPIEXEC, "-n", str(sample_P), O.REF_DRIVER, func, cf, str(esz), str(args["r"]), str(args["b"]),
                       str(args["n"]), str(args["bblock"]), "0", "0", str(seed), "3", out]
                res = subprocess.run(cmd, capture_output=True, text=True, timeout=budget_s)
                if res.returncode == 0:
                    times = [float(x) for x in open(out + ".times").read().split()]
                    digests = open(out + ".digests").read().split()
                    t = float(np.median(times[1:])) if len(times) > 1 else times[0]
                    return {"value": payload / t / 1e9, "unit": "GB/s", "cores": cores, "kind": "reference",
                            "sample": sample + f"; mpiexec -n {sample_P} (MPICH 3.3.2) on {cores} cores, "
                                               f"{sample_P / cores:.0f}x oversubscribed, median of 2 after 1 warm-up, "
                                               f"max over ranks; result equal to MPI_Alltoallv",
                            "seconds": t, "_digests": digests, **keep}
        except (subprocess.TimeoutExpired, OSError, ValueError):
            pass
    prob = W.make_problem(counts, esz, 0, 0)
    send = np.zeros(prob.send_bytes, dtype=np.uint8)
    O.fill_payload(0, seed, prob, send)
    recv = np.zeros(prob.recv_bytes, dtype=np.uint8)
    fn = {"ttpl": lambda: O.TTPL_BT_alltoallv(32, 32, 0, prob, send, recv),
          "tuna": lambda: O.tuna_algorithm(32, 0, prob, send, recv),
          "twophase": lambda: O.twophase_rbruck_alltoallv(args["r"], prob, send, recv)}[func]
    fn()
    t0 = time.perf_counter()
    reps = 0
    while reps < 3 or time.perf_counter() - t0 < 2.0:
        assert fn() == 0
        reps += 1
        if time.perf_counter() - t0 > budget_s:
            break
    t = (time.perf_counter() - t0) / reps
    return {"value": payload / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": sample + f"; single-threaded C restatement of the reference algorithm, mean of {reps} calls",
            "seconds": t, "_digests": [f"{int(h):016x}" for h in O.digest_recv(prob, recv)], **keep}


def same_run_parity(cpu: dict, api) -> dict:
    """Runs this library's function on the very sample the CPU leg ran (same counts, seed, payload, function, tunables) and
    compares each virtual rank's FNV-1a digest of its receive blocks with what the CPU ranks received — the check the
    reference's drivers make inside their timed runs (examples/rbruckv_example.cpp:101-121).  Returns the public part of
    the CPU leg's record with `digests_equal` added."""
    from oracle import oracle_py as O
    pub = {k: v for k, v in cpu.items() if not k.startswith("_")}
    if "_digests" not in cpu:
        return pub
    prob = W.make_problem(cpu["_counts"], cpu["_esz"], 0, 0)
    dp = api.DeviceProblem(prob)
    send, recv = dp.new_send_arena(), dp.new_recv_arena(0xEE)
    dp.fill_payload(0, cpu["_seed"], send)
    rc = call(api, cpu["_gpu_func"], cpu["_gpu_tun"], dp, send, recv)
    assert rc == 0, dp.comm.error()
    got = [f"{int(h):016x}" for h in O.digest_recv(prob, recv.cpu().numpy())]
    pub["digests_equal"] = got == cpu["_digests"]
    pub["digests_compared"] = len(got)
    pub["gpu_execution_on_sample"] = EXECUTION_NAMES[int(dp.comm.last_stats().execution)]
    dp.comm.free()
    return pub


# vc_stats_t.execution of the timed calls (the library's default mode picks between the two forwarded kernels)
EXECUTION_NAMES = {0: "launch per digit phase",
                   1: "forwarded (one launch, blocks carried through all hops in registers)",
                   2: "forwarded, without a work-item list (every pair of ranks derives its block's route in the copy kernel; "
                      "one host synchronisation per call)",
                   3: "forwarded, without a work-item list, staging slots at a fixed stride (no planner: the one launch of the call "
                      "also adds up the tables' totals; one host synchronisation per call)"}
EXECUTION_KERNELS = {0: "vc_copy_items", 1: "vc_copy_chains", 2: "vc_copy_blocks", 3: "vc_copy_blocks"}


def kernel_name(st) -> str:
    """Name of the copy kernel the timed calls launched, from vc_stats_t.execution, .lanes_per_item and .host_waits (a
    list-driven call whose launches all went out before the host had seen the plan runs the instance of the kernel that
    checks the plan on the device: second template argument true)."""
    base, lanes = EXECUTION_KERNELS[int(st.execution)], int(st.lanes_per_item)
    enqueued = int(st.execution) == 1 and int(st.host_waits) == 1
    if lanes == 16:
        return base + "_quarter_kernel" + ("<true>" if enqueued else "<false>" if int(st.execution) == 1 else "")
    if lanes == 1:
        return base + "_batch_kernel"
    if int(st.execution) == 1:
        return base + "_kernel" + f"<{lanes}, {'true' if enqueued else 'false'}>"
    return base + "_kernel" + f"<{lanes}>"


def copy_ceiling(comm, torch, mib: int = 2048, reps: int = 4) -> dict:
    """What contiguous copies sustain on this GPU in this run: vc_calibration_copy (one read, one write: the mix of
    launch-per-digit execution) and vc_calibration_copy2 (one read, two writes: the mix of the forwarded kernel on two-hop
    routes), 16-byte non-temporal loads and stores, one vector per lane — the access pattern of the block movers without
    their scatter.  HIP events on the communicator's stream.  What the two-writes copy sustains depends on which
    allocations it runs on (up to 10 % inside one process), so four buffers take the three roles in turn and the
    ceiling is the best of all launches; the slowest placement's best is reported beside it."""
    nb = mib << 20
    bufs = [torch.zeros(nb, dtype=torch.uint8, device="cuda:0") for _ in range(4)]
    per_placement = {1: [], 2: []}
    for shift in range(4):
        a, b, b2 = (bufs[(shift + k) % 4] for k in range(3))
        best = {1: None, 2: None}
        for _ in range(reps + 1):
            for writes in (1, 2):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                if writes == 1:
                    comm._check(comm.lib.vc_calibration_copy(b.data_ptr(), a.data_ptr(), nb, comm.handle))
                else:
                    comm._check(comm.lib.vc_calibration_copy2(b.data_ptr(), b2.data_ptr(), a.data_ptr(), nb, comm.handle))
                e1.record()
                torch.cuda.synchronize()
                ms = e0.elapsed_time(e1)
                best[writes] = ms if best[writes] is None or ms < best[writes] else best[writes]
        for writes in (1, 2):
            per_placement[writes].append(best[writes])
    del bufs
    ms1, ms2 = min(per_placement[1]), min(per_placement[2])
    return {"GBps": round(2 * nb / (ms1 * 1e-3) / 1e9, 1), "ms": round(ms1, 4), "bytes_each_way": nb, "placements": 4,
            "one_read_one_write_GBps": round(2 * nb / (ms1 * 1e-3) / 1e9, 1),
            "one_read_two_writes_GBps": round(3 * nb / (ms2 * 1e-3) / 1e9, 1), "one_read_two_writes_ms": round(ms2, 4),
            "one_read_two_writes_GBps_slowest_placement": round(3 * nb / (max(per_placement[2]) * 1e-3) / 1e9, 1)}


def ceiling_for_mix(ceiling: dict, writes_per_read: float) -> float:
    """GB/s a contiguous copy with this many writes per read sustains: the two measured mixes, the time per byte read
    interpolated (extrapolated beyond two writes) linearly between them."""
    t1 = 2.0 / ceiling["one_read_one_write_GBps"]
    t2 = 3.0 / ceiling["one_read_two_writes_GBps"]
    t = t1 + (writes_per_read - 1.0) * (t2 - t1)
    return (1.0 + writes_per_read) / t


def physical_bytes(st) -> int:
    """Bytes the copy kernels of the last call had to move through HBM: one launch per digit reads and writes every hop;
    forwarded execution reads every block once and writes it once per hop."""
    return 2 * st.moved_bytes if st.execution == 0 else st.payload_bytes + st.moved_bytes


def other_configurations(api, torch, ceiling: dict, seed: int) -> dict:
    """The benchmark's other configurations beside the one `value` is quoted on, a few steps each in the default mode:
    configuration 2 at its three radices, configuration 3, configuration 5 at r = 32 (what src/tuna.cpp:67-165 times) and at
    r = 2.  Per entry: milliseconds per blocking call (wall clock), the copy kernels' bytes over their launch time (HIP
    events on the communicator's stream) against the HBM peak, the execution the library chose, staging memory, and the
    exact receiver-side check."""
    out = {}
    for key, name, radix, steps in (("C2_r2", "C2", 2, 50), ("C2_r4", "C2", 4, 50), ("C2_r8", "C2", 8, 50), ("C3_r16", "C3", 16, 10),
                                    ("C5_r32", "C5", 32, 5), ("C5_r2", "C5", 2, 5)):
        counts, esz, func, tun, _ = workload(name, seed)
        tun = dict(tun, r=radix)
        prob = W.make_problem(counts, esz, 0, 0)
        dp = api.DeviceProblem(prob)
        send, recv = dp.new_send_arena(), dp.new_recv_arena(0)
        dp.fill_payload(0, seed, send)
        for _ in range(3):
            assert call(api, func, tun, dp, send, recv) == 0, dp.comm.error()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            call(api, func, tun, dp, send, recv)
        torch.cuda.synchronize()
        call_s = (time.perf_counter() - t0) / steps
        untimed = dp.comm.last_stats()                  # how the calls behind ms_per_call ran
        # the same calls again with the library's events around every launch (they cost microseconds that matter at
        # configuration 2, so the wall-clock figure above is taken without them; with them on a list-driven call also
        # keeps the host's look at the plan in mid-call, so the events bracket the copy kernel alone)
        dp.comm.set_timing(True)
        kern_ms, phys = 0.0, 0
        for _ in range(steps):
            assert call(api, func, tun, dp, send, recv) == 0, dp.comm.error()
            st = dp.comm.last_stats()
            kern_ms += sum(st.launch_ms[k] for k in range(st.n_launches))
            phys += physical_bytes(st)
        st = dp.comm.last_stats()
        achieved = phys / (kern_ms * 1e-3) / 1e9 if kern_ms > 0 else 0.0
        mix = 1.0 if st.execution == 0 else st.moved_bytes / max(st.payload_bytes, 1)
        out[key] = {"workload": f"benchmark configuration {name[1:]}: {func}, P={prob.P}, r={radix}, {esz}-byte elements",
                    "payload_bytes": int(prob.payload_bytes), "ms_per_call": round(call_s * 1e3, 4),
                    "GBps_effective": round(prob.payload_bytes / call_s / 1e9, 1),
                    "kernel": kernel_name(untimed), "execution": EXECUTION_NAMES[int(untimed.execution)],
                    "launches_per_call": int(untimed.n_launches), "host_waits_per_call": int(untimed.host_waits),
                    "kernel_timed": kernel_name(st), "kernel_ms_per_call": round(kern_ms / steps, 4),
                    "kernel_GBps_physical": round(achieved, 1), "frac": round(achieved / HBM_PEAK_GBPS, 4),
                    "frac_of_copy_ceiling": round(achieved / ceiling_for_mix(ceiling, mix), 4),
                    "algorithmic_frac_whole_call": round(2 * st.moved_bytes / call_s / 1e9 / HBM_PEAK_GBPS, 4),
                    "staging_bytes": int(st.staging_bytes), "steps": steps,
                    "mismatched_bytes": int(dp.verify(send, recv))}
        dp.comm.free()
        del send, recv, dp
        torch.cuda.empty_cache()
    return out


def metadata_calls(api, torch, counts) -> dict:
    """The caller-side steps of the reference's drivers (examples/rbruckv_example.cpp:69-82) on configuration 4's tables:
    count-matrix exchange, the two displacement scans, the two scans of arena bases, the global maximum — microseconds per
    blocking call (each ends in a stream synchronisation), mean of 20, checked against numpy."""
    P = counts.shape[0]
    comm = api.VirtualComm(P)
    lib, h = comm.lib, comm.handle
    dev = "cuda:0"
    sc = torch.from_numpy(np.ascontiguousarray(counts)).to(dev)
    rc = torch.empty_like(sc)
    sd, rd = torch.empty_like(sc), torch.empty_like(sc)
    sext, rext = torch.empty(P, dtype=torch.int64, device=dev), torch.empty(P, dtype=torch.int64, device=dev)
    sbase, rbase = torch.empty(P, dtype=torch.int64, device=dev), torch.empty(P, dtype=torch.int64, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    mx = torch.empty(1, dtype=torch.int32, device=dev)
    steps = (("vc_alltoall_counts", lambda: lib.vc_alltoall_counts(sc.data_ptr(), rc.data_ptr(), h)),
             ("vc_displs_from_counts_send", lambda: lib.vc_displs_from_counts(sc.data_ptr(), sd.data_ptr(), sext.data_ptr(), h)),
             ("vc_displs_from_counts_recv", lambda: lib.vc_displs_from_counts(rc.data_ptr(), rd.data_ptr(), rext.data_ptr(), h)),
             ("vc_bases_from_extents_send", lambda: lib.vc_bases_from_extents(sext.data_ptr(), 1, 256, sbase.data_ptr(), total.data_ptr(), h)),
             ("vc_bases_from_extents_recv", lambda: lib.vc_bases_from_extents(rext.data_ptr(), 1, 256, rbase.data_ptr(), total.data_ptr(), h)),
             ("vc_allreduce_max_count", lambda: lib.vc_allreduce_max_count(sc.data_ptr(), mx.data_ptr(), h)))
    out, reps = {"P": P, "table_bytes": int(counts.nbytes)}, 20
    for name, fn in steps:
        assert fn() == 0, comm.error()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        out[name] = round((time.perf_counter() - t0) / reps * 1e6, 1)
    out["total"] = round(sum(v for k, v in out.items() if k.startswith("vc_")), 1)
    c64 = counts.astype(np.int64)
    ok = (np.array_equal(rc.cpu().numpy(), counts.T) and np.array_equal(sd.cpu().numpy(), np.cumsum(c64, axis=1) - c64)
          and np.array_equal(rd.cpu().numpy(), np.cumsum(c64.T, axis=1) - c64.T) and int(mx.item()) == int(counts.max())
          and np.array_equal(sext.cpu().numpy(), c64.sum(axis=1)))
    out["equal_to_numpy"] = bool(ok)
    comm.free()
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="C4")
    ap.add_argument("--forward", type=int, default=1, choices=(0, 1),
                    help="1 (the library's default): forwarded execution is the mode that is measured; 0: one launch per digit "
                         "phase (vc_comm_set_forwarding(comm, 0)); the other one is reported beside it")
    ap.add_argument("--func", default=None, help="override the function (e.g. TTPL_BT_alltoallv_s1)")
    ap.add_argument("--radix", type=int, default=0, help="override the radix r of the workload")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-context", action="store_true", help="skip the context figures beside the metric (plans, graph, the other "
                                                             "execution mode, comparator, short-block calls): for profiling runs")
    ap.add_argument("--cpu-budget", type=float, default=150.0)
    ap.add_argument("--only-metadata", action="store_true",
                    help="only the caller-side metadata steps on the workload's count table (for profiling their kernels); prints their record")
    ap.add_argument("--calibration-copy", type=int, default=0, metavar="MiB",
                    help="also run one plain copy of this many MiB before the timed region (for scaling rocprofv3 --pmc byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs the virtual communicator on ONE GPU; --gpus N with N > 1 is not supported")

    # the CPU leg starts child processes (mpiexec) and needs nothing from the GPU: it runs before anything here touches the device
    cpu = None if args.no_cpu_baseline or args.only_metadata else cpu_reference_leg(args.workload, args.seed, args.cpu_budget)

    import torch
    from rbruck_alltoallv_amd import api

    counts, esz, func, tun, hops = workload(args.workload, args.seed)
    if args.only_metadata:
        if args.calibration_copy:                          # the transfer of known size the byte counters are scaled against
            comm = api.VirtualComm(2)
            nb = args.calibration_copy << 20
            a = torch.zeros(nb, dtype=torch.uint8, device="cuda:0")
            b = torch.zeros(nb, dtype=torch.uint8, device="cuda:0")
            comm._check(comm.lib.vc_calibration_copy(b.data_ptr(), a.data_ptr(), nb, comm.handle))
            comm.free()
            del a, b
        print(json.dumps({"metadata_us": metadata_calls(api, torch, counts)}), flush=True)
        return
    if args.func:
        func = args.func
    if args.radix:
        tun["r"] = args.radix
    if args.func or args.radix:
        # the hop model follows the function that is actually called
        P_ = counts.shape[0]
        if func in ("twophase_rbruck_alltoallv", "twophase_rbruck_alltoallv_om", "tuna_algorithm"):
            tun.setdefault("b", 0)
            hops = W.hops_flat(P_, min(tun["r"], P_ - 1 if func == "tuna_algorithm" else P_))
        else:
            tun.setdefault("n", 32)
            tun.setdefault("bblock", 0)
            hops = W.hops_twolayer_bruck(P_, tun["n"], tun["r"]) if func == "TTPL_rbruck_alltoallv" else W.hops_twolayer(P_, tun["n"], tun["r"])
    prob = W.make_problem(counts, esz, 0, 0)
    S = prob.payload_bytes
    A = W.algorithmic_bytes(counts, esz, hops)

    dp = api.DeviceProblem(prob)
    send = dp.new_send_arena()
    recv = dp.new_recv_arena(0)
    dp.fill_payload(0, args.seed, send)
    dp.comm.set_timing(True)

    if args.calibration_copy:
        nb = args.calibration_copy << 20
        a = torch.zeros(nb, dtype=torch.uint8, device="cuda:0")
        b = torch.zeros(nb, dtype=torch.uint8, device="cuda:0")
        dp.comm._check(dp.comm.lib.vc_calibration_copy(b.data_ptr(), a.data_ptr(), nb, dp.comm.handle))
        del a, b
    ceiling = copy_ceiling(dp.comm, torch)

    def timed_calls(warmup, steps):
        """`steps` blocking calls; per-launch times from the library's HIP events on the communicator's stream."""
        for _ in range(warmup):
            rc = call(api, func, tun, dp, send, recv)
            assert rc == 0, dp.comm.error()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        kern_ms, phys_bytes, alg_bytes, nkern, plan_ms = 0.0, 0, 0, 0, 0.0
        per_launch_ms = None
        every = []                                      # the statistics of every call; added up after the timed region
        for _ in range(steps):
            rc = call(api, func, tun, dp, send, recv)
            assert rc == 0, dp.comm.error()
            every.append(dp.comm.last_stats())
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        for st in every:
            for k in range(st.n_launches):
                kern_ms += st.launch_ms[k]
                nkern += 1
            phys_bytes += physical_bytes(st)
            alg_bytes += 2 * st.moved_bytes
            plan_ms += st.plan_ms
            if st.n_launches <= 16:
                now = [st.launch_ms[k] for k in range(st.n_launches)]
                per_launch_ms = now if per_launch_ms is None else [a + b for a, b in zip(per_launch_ms, now)]
        st = dp.comm.last_stats()
        assert 2 * st.moved_bytes == A, (st.moved_bytes, A)
        assert st.payload_bytes == S
        return dict(elapsed=elapsed, steps=steps, kern_ms=kern_ms, phys_bytes=phys_bytes, alg_bytes=alg_bytes, nkern=nkern,
                    plan_ms=plan_ms, per_launch_ms=per_launch_ms, st=st)

    def roofline_of(t) -> dict:
        """The HBM roofline of the copy kernel(s) of one execution mode.  `achieved` counts the bytes the kernels had to
        move (physical_bytes) over their launch time and is what `frac` is a fraction of; `algorithmic_*` counts one read
        and one write per hop whether or not the execution re-reads between hops."""
        st, nk = t["st"], max(t["nkern"], 1)
        secs = t["kern_ms"] * 1e-3
        kern = kernel_name(st)
        achieved = t["phys_bytes"] / secs / 1e9 if secs > 0 else 0.0
        alg = t["alg_bytes"] / secs / 1e9 if secs > 0 else 0.0
        quoted = not (args.radix or args.seed or args.func)
        # the contiguous copy with this execution's mix of reads and writes: one write per read when every hop is a launch
        # of its own, (bytes of all hops) / payload writes per read when the blocks are forwarded
        mix = 1.0 if st.execution == 0 else st.moved_bytes / max(st.payload_bytes, 1)
        like = ceiling_for_mix(ceiling, mix)
        traffic, source = profiled_traffic(kern.split("<")[0], args.workload) if quoted else (None, None)
        r = {"bound": "hbm", "kernel": kern, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
             "frac": round(achieved / HBM_PEAK_GBPS, 4), "frac_physical": round(achieved / HBM_PEAK_GBPS, 4),
             "physical_bytes_per_launch": int(t["phys_bytes"] / nk),
             "algorithmic_GBps": round(alg, 1), "algorithmic_frac": round(alg / HBM_PEAK_GBPS, 4),
             "algorithmic_bytes_per_launch": int(t["alg_bytes"] / nk),
             "copy_ceiling_writes_per_read": round(mix, 3), "copy_ceiling_GBps": round(like, 1),
             "frac_of_copy_ceiling": round(achieved / like, 4),
             "traffic": traffic, "traffic_source": source,
             "avg_launch_ms": round(t["kern_ms"] / nk, 4), "launches_per_call": int(st.n_launches),
             "per_launch": None if t["per_launch_ms"] is None else [
                 {"ms": round(m / t["steps"], 4),
                  "GBps": round((2 * st.launch_bytes[k] if st.execution == 0 else st.payload_bytes + st.launch_bytes[k])
                                / (m / t["steps"]) / 1e6, 1) if m > 0 else 0.0}
                 for k, m in enumerate(t["per_launch_ms"])]}
        if traffic and secs > 0:
            # measured HBM bytes per launch over the same launch duration: what the memory system sustained
            r["traffic_GBps"] = round(traffic / (secs / nk) / 1e9, 1)
            r["traffic_over_physical"] = round(traffic / (t["phys_bytes"] / nk), 4)
        return r

    def plan_timing(steps):
        """The same collective as a persistent plan (planned once, executed many times), and that plan in a HIP graph."""
        plan_kw = {"n": tun.get("n", 0), "r": tun.get("r", 2), "batch": tun.get("b", tun.get("bblock", 0))}
        plan = api.Plan(func, dp, recv, **plan_kw)
        if plan.rc != 0:
            return None
        assert plan.execute(send, recv) == 0, dp.comm.error()
        torch.cuda.synchronize()
        p0 = time.perf_counter()
        for _ in range(steps):
            assert plan.execute(send, recv) == 0
        torch.cuda.synchronize()
        plan_s = (time.perf_counter() - p0) / steps
        plan_bad = dp.verify(send, recv, packed_recv=packed)
        info = {"ms_per_call": round(plan_s * 1e3, 4), "GBps_effective": round(S / plan_s / 1e9, 1),
                "mismatched_bytes": int(plan_bad)}
        # ... and its launches captured once into a HIP graph (what a launch-bound inner loop would replay)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            dp.comm.use_current_stream()
            assert plan.execute_async(send, recv) == 0, dp.comm.error()
        dp.comm.use_current_stream()
        graph.replay()
        torch.cuda.synchronize()
        g0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
            torch.cuda.synchronize()
        graph_s = (time.perf_counter() - g0) / steps
        info["graph_replay_ms_per_call"] = round(graph_s * 1e3, 4)
        info["graph_mismatched_bytes"] = int(dp.verify(send, recv, packed_recv=packed))
        del graph
        plan.free()
        return info

    packed = func == "TTPL_BT_alltoallv"
    dp.comm.set_forwarding(bool(args.forward))
    t = timed_calls(args.warmup, args.steps)
    st = t["st"]
    elapsed = t["elapsed"]
    bad = dp.verify(send, recv, packed_recv=packed)
    call_s = elapsed / args.steps
    ms_per_step = call_s * 1e3
    phys_call = physical_bytes(st)

    out = {
        "metric": METRIC, "value": round(S / call_s / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": (f"benchmark configuration 4 with counts rounded to multiples of {args.workload[3:]} bytes" if args.workload.startswith("C4m") else
                                f"benchmark configuration {args.workload[1:]}" if args.workload[0] == "C" else
                                f"equal blocks of {args.workload[1:]} bytes" if args.workload[0] == "U" else
                                f"blocks uniform in 0..{args.workload[1:]} bytes" if args.workload[0] == "S" else
                                f"reference input matrix inputs/{prob.P}proc") + f": {func}, P={prob.P} virtual ranks, "
                               + ", ".join(f"{k}={v}" for k, v in tun.items()) + f", {esz}-byte elements",
                   "payload_bytes": S, "algorithmic_bytes": A, "physical_bytes": int(phys_call),
                   "launches_per_step": int(st.n_launches), "staging_bytes": int(st.staging_bytes)},
        # whole call (planning kernels, host synchronisations, copy launches) against the HBM peak: bytes the call had to
        # move, bytes of one read + one write per hop (the algorithm's), bytes of a one-pass gather
        "whole_call_hbm_frac": {"physical": round(phys_call / call_s / 1e9 / HBM_PEAK_GBPS, 4),
                                "algorithmic": round(A / call_s / 1e9 / HBM_PEAK_GBPS, 4),
                                "one_pass_floor": round(2 * S / call_s / 1e9 / HBM_PEAK_GBPS, 4)},
        "plan_ms_per_step": round(t["plan_ms"] / args.steps, 4),
        "mismatched_bytes": int(bad),
        "execution": EXECUTION_NAMES[int(st.execution)],
        "host_waits_per_call": int(st.host_waits),
        "kernel_sources_sha256": kernel_sources_sha(),
        "copy_ceiling": ceiling,
    }
    if not args.no_context:
        # Extra information; `value` stays the full call.
        out["persistent_plan"] = plan_timing(args.steps)

        # The other way of executing the same call (launch per digit phase <-> forwarded), on fewer steps.
        dp.comm.set_forwarding(not args.forward)
        o_steps = max(3, min(args.steps, 10))
        o = timed_calls(2, o_steps)
        o_bad = dp.verify(send, recv, packed_recv=packed)
        o_plan = plan_timing(o_steps)
        o_call = o["elapsed"] / o_steps
        out["other_execution_mode"] = {
            "mode": EXECUTION_NAMES[int(o["st"].execution)],
            "ms_per_call": round(o_call * 1e3, 4), "GBps_effective": round(S / o_call / 1e9, 1),
            "whole_call_hbm_frac": {"physical": round(physical_bytes(o["st"]) / o_call / 1e9 / HBM_PEAK_GBPS, 4),
                                    "algorithmic": round(A / o_call / 1e9 / HBM_PEAK_GBPS, 4)},
            "mismatched_bytes": int(o_bad),
            "plan_ms_per_call": None if o_plan is None else o_plan["ms_per_call"],
            "plan_graph_replay_ms": None if o_plan is None else o_plan["graph_replay_ms_per_call"],
            "roofline": roofline_of(o)}
        dp.comm.set_forwarding(bool(args.forward))

        # The linear comparator the reference drivers time beside the Bruck variants (examples/twophaseLayer_example.cpp:99-113
        # times MPI_Alltoallv): on one GPU it is a single pass over the payload.  Context only, not the metric.
        dp.comm.set_timing(False)
        comp_steps = max(3, min(args.steps, 10))
        assert api.spreadout_alltoallv(dp, send, recv) == 0, dp.comm.error()
        torch.cuda.synchronize()
        c0 = time.perf_counter()
        for _ in range(comp_steps):
            assert api.spreadout_alltoallv(dp, send, recv) == 0
        torch.cuda.synchronize()
        comp_s = (time.perf_counter() - c0) / comp_steps
        comp_bad = dp.verify(send, recv, packed_recv=False)
        out["one_pass_comparator"] = {"func": "spreadout_alltoallv", "ms_per_call": round(comp_s * 1e3, 4),
                                      "GBps_effective": round(S / comp_s / 1e9, 1),
                                      "hbm_frac": round(2 * S / comp_s / 1e9 / HBM_PEAK_GBPS, 4), "mismatched_bytes": int(comp_bad)}
        if args.workload == "C4" and args.func is None:
            out["short_block_calls"] = short_block_context(api, torch)
    out["roofline"] = roofline_of(t)
    dp.comm.free()
    del send, recv, dp
    torch.cuda.empty_cache()
    if not args.no_context and args.workload == "C4" and args.func is None and not args.radix:
        out["configs"] = other_configurations(api, torch, ceiling, args.seed)
        out["metadata_us"] = metadata_calls(api, torch, counts)
    if cpu is not None:
        out["cpu_baseline"] = same_run_parity(cpu, api)
    print(json.dumps(out), flush=True)
    if bad:
        raise SystemExit(f"bench.py: {bad} bytes differ from the alltoallv definition")
    if cpu is not None and out["cpu_baseline"].get("digests_equal") is False:
        raise SystemExit("bench.py: the digests of the GPU's receive blocks differ from those of the CPU run on the same sample")
    wrong = [k for k, v in out.get("configs", {}).items() if v["mismatched_bytes"]]
    if wrong:
        raise SystemExit(f"bench.py: configurations {wrong} differ from the alltoallv definition")


if __name__ == "__main__":
    main()
