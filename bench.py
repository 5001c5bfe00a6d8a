#!/usr/bin/env python3
"""Benchmark of the single-shot all-reduce data path on one MI355X.

A "step" is one all-reduce over the virtual ranks' buffers (already resident in
HBM).  Default workload: 8 virtual ranks, `bisect`, 16,777,216 binary16 values
(32 MiB) per rank, N(0, 0.02) inputs — the bandwidth-bound headline
configuration.  Prints ONE JSON line; see --help for the other modes.

Algorithmic bytes per step: B = N*S (every rank's input read once) + N*S (the sum
written once to every rank's output) = 2*N*S.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM-side bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (each scaled by the same counter's reading for a plain copy of known size).
# (workload, transport) -> (bytes, the summary under profiles/ that derives the
# figure; a CPU test checks that the file states this very number).
MEASURED_TRAFFIC_BYTES = {
    ("cfg3", "direct"): (536914021, "direct_allreduce_bisect_8x32MiB_hbm_traffic.md"),
    ("cfg4", "direct"): (167799218, "direct_allreduce_bisect_8x32MiB_hbm_traffic.md"),
    ("cfg5_32MiB", "wire"): (1498284599, "wire_allreduce_flag_words_8x32MiB.md"),
    ("cfg3", "wire"): (1501431833, "wire_allreduce_flag_words_8x32MiB.md"),
}


def measured_traffic(name, transport):
    algo = WORKLOADS[name][1]
    if transport == "static":
        return None
    if transport == "default":
        transport = "wire" if algo == "parallel" else "direct"
    return MEASURED_TRAFFIC_BYTES.get((name, transport), (None, None))[0]

# Element type of the run (--dtype): 0 = binary16, 1 = bfloat16.  Buffers are
# 2-byte elements either way; only the adds and the generated bit patterns differ.
DTYPE = 0
DTYPE_NAMES = {0: "f16", 1: "bf16"}

WORKLOADS = {
    # name: (nranks, algo, nelems per rank, dist, p0, p1, seed)
    "cfg1": (2, "simple", 16384, 0, -1.0, 1.0, 1000),
    "cfg2": (8, "small", 524288, 1, 0.0, 1.0, 2000),
    "cfg3": (8, "bisect", 16777216, 1, 0.0, 0.02, 3000),
    "cfg4": (4, "allgather_simple", 4194304, 0, -2.0, 2.0, 4000),
    # the 16-rank instantiation of bisect (allreduce.cpp:1020), same 256 MiB of inputs as cfg3
    "bisect16": (16, "bisect", 8388608, 1, 0.0, 0.02, 6000),
    # one point of the size sweep: its named protocol (message passing) at 32 MiB per rank
    "cfg5_32MiB": (8, "parallel", 16777216, 1, 0.0, 1.0, 5000),
    # the hot kernel at other shapes (profile runs; inputs repeat a 16 Mi-element draw)
    "bisect_8x64MiB": (8, "bisect", 1 << 25, 1, 0.0, 0.02, 7000),
    "bisect_8x128MiB": (8, "bisect", 1 << 26, 1, 0.0, 0.02, 7100),
    "bisect_8x256MiB": (8, "bisect", 1 << 27, 1, 0.0, 0.02, 7200),
    "bisect_4x64MiB": (4, "bisect", 1 << 25, 1, 0.0, 0.02, 7300),
    "simple_2x128MiB": (2, "simple", 1 << 26, 1, 0.0, 0.02, 7400),
}

# Fixed size of the kernel-time sample behind `roofline`, whatever --steps says.
KERNEL_SAMPLE_LAUNCHES = 200
KERNEL_SAMPLE_MIN_PAIRS = 20
# p50 kernel execution time of cfg2 in a rocprofv3 kernel trace (microseconds), and the
# summary under profiles/ that states it; printed beside the in-process figures.
CFG2_KERNEL_TRACE = (4.20, "direct_allreduce_small_8x1MiB_kernel_trace.md")

# --transport: how the virtual ranks exchange data (0 = the protocol's default).
TRANSPORT = 0
# --transport static: vr_allreduce_static (wire transport through the library's fixed scratch region)
STATIC = False


def describe(name):
    n, algo, ne, dist, p0, p1, _ = WORKLOADS[name]
    d = ("N(%g,%g)" % (p0, p1)) if dist == 1 else ("U[%g,%g)" % (p0, p1))
    return "%s: %d virtual ranks, %s, %d %s/rank (%.3g MiB), %s" % (
        name, n, algo, ne, "bfloat16" if DTYPE else "binary16", ne * 2 / 2**20, d)


def algorithmic_bytes(name):
    n, algo, ne, *_ = WORKLOADS[name]
    s = ne * 2
    if algo.startswith("allgather"):
        return n * s + n * n * s
    return 2 * n * s


def setup(vr, binding, name, inplace, nsets=1):
    """Context + `nsets` independent sets of per-rank device buffers holding the
    same seeded inputs.  Rotating through several sets defeats the 256 MiB
    memory-side cache, so that every step really streams from and to HBM."""
    n, algo, ne, dist, p0, p1, seed = WORKLOADS[name]
    ctx = vr.VirtualRanks(n)
    ctx.set_dtype(DTYPE)
    draw = min(ne, 1 << 24)         # larger inputs repeat a 16 Mi-element draw (generation time)
    host = [binding.generate(draw, seed + r, dist, p0, p1, dtype=DTYPE) for r in range(n)]
    if draw < ne:
        host = [np.tile(a, ne // draw) for a in host]
    sets = []
    for _ in range(nsets):
        ins = [binding.DeviceBuffer(ne * 2) for _ in range(n)]
        for b, a in zip(ins, host):
            b.upload(a)
        if algo.startswith("allgather"):
            outs = [binding.DeviceBuffer(n * ne * 2) for _ in range(n)]
        elif inplace:
            outs = None
        else:
            outs = [binding.DeviceBuffer(ne * 2) for _ in range(n)]
        sets.append((ins, outs))
    return ctx, host, sets


def launch(ctx, name, ins, outs):
    n, algo, ne, *_ = WORKLOADS[name]
    if algo.startswith("allgather"):
        ctx.allgather(algo, [b.ptr for b in ins], [b.ptr for b in outs], ne, transport=TRANSPORT)
    elif STATIC:
        # the allocation-free entry point: message passing through the library's fixed region
        ctx.allreduce_static(algo, [b.ptr for b in ins], ne, outs=[b.ptr for b in outs] if outs else None)
    else:
        ctx.allreduce(algo, [b.ptr for b in ins], ne, outs=[b.ptr for b in outs] if outs else None,
                      transport=TRANSPORT)


def time_kernels(binding, ctx, name, sets, iters, group=1):
    """Kernel times (ms per launch) from HIP event pairs recorded on the launch
    stream, rotating through the buffer sets.  With group > 1 each pair brackets
    `group` back-to-back launches and the result is their mean, which amortises
    the ~2 us the event commands themselves add."""
    npairs = (iters + group - 1) // group
    timer = binding.EventTimer(npairs)
    k = 0
    for p in range(npairs):
        timer.start(p)
        for _ in range(group):
            launch(ctx, name, *sets[k % len(sets)])
            k += 1
        timer.stop(p)
    ctx.sync()
    out = timer.elapsed_ms(npairs) / group
    timer.close()
    return out


def kernel_sample(binding, ctx, name, sets, group):
    """The kernel-time sample the roofline figure rests on: always at least
    KERNEL_SAMPLE_LAUNCHES launches in at least KERNEL_SAMPLE_MIN_PAIRS event pairs on
    the launch stream, independent of --steps."""
    group = max(1, min(group, KERNEL_SAMPLE_LAUNCHES // KERNEL_SAMPLE_MIN_PAIRS))
    kms = time_kernels(binding, ctx, name, sets, KERNEL_SAMPLE_LAUNCHES, group=group)
    return kms, {"kernel_us_avg": round(float(kms.mean()) * 1e3, 3),
                 "kernel_us_min": round(float(kms.min()) * 1e3, 3),
                 "kernel_us_p50": round(float(np.median(kms)) * 1e3, 3),
                 "kernel_us_p99": round(float(np.percentile(kms, 99)) * 1e3, 3),
                 "n_pairs": int(len(kms)), "launches_per_pair": group,
                 "launches": int(len(kms)) * group}


def in_place_cold(binding, ctx, name, sets, host, rounds=10):
    """The reference's in-place semantics (parallel_transmit.hpp:125-130) on buffers no
    cache holds: each round restores every set's work buffers from the inputs with
    a device copy (outside the timing), then times one in-place launch per set
    inside one event pair.  The work buffers are the out-of-place sets' outputs."""
    n, algo, ne, *_ = WORKLOADS[name]
    timer = binding.EventTimer(rounds)
    for p in range(rounds):
        for ins, outs in sets:
            for src, dst in zip(ins, outs):
                ctx.stream_probe(0, dst.ptr, src.ptr, ne * 2)
        timer.start(p)
        for ins, outs in sets:
            launch(ctx, name, outs, None)
        timer.stop(p)
    ctx.sync()
    ms = timer.elapsed_ms(rounds) / len(sets)
    timer.close()
    return ms[1:] if rounds > 2 else ms


def memory_clock():
    """The memory clock levels the driver reports (sysfs, `*` marks the current
    one), sampled while the GPU is still warm from the timed region."""
    import glob
    found = {}
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_mclk")):
        try:
            lines = [l.strip() for l in open(path).read().splitlines() if l.strip()]
        except OSError:
            continue
        found[path.split("/")[4]] = {"levels": [l.rstrip(" *") for l in lines],
                                     "current": [l.rstrip(" *") for l in lines if l.endswith("*")]}
    return found or None


def launch_plan(binding, algo, n, ne, args):
    """The launch the library picks for the timed workload on the direct transport
    (vr_direct_launch_plan), with the --tune overrides of this run beside it."""
    if args.transport not in ("default", "direct") or algo == "parallel":
        return None
    plan = binding.direct_launch_plan(algo, n, ne, bool(args.inplace))
    if args.tune:
        plan["overridden_by_--tune"] = list(args.tune)
    return plan


def device_state():
    """Clock levels in use, power and temperatures as sysfs shows them right after the timed
    region: boxes of one pool differ by a few per cent in every kernel, and this is what
    can be read about why."""
    import glob
    found = {}
    for dev in sorted(glob.glob("/sys/class/drm/card*/device")):
        st = {}
        for clk in ("sclk", "mclk", "fclk", "socclk"):
            try:
                cur = [l.strip().rstrip(" *") for l in open("%s/pp_dpm_%s" % (dev, clk)) if l.strip().endswith("*")]
            except OSError:
                continue
            if cur:
                st[clk] = cur[0].split(":", 1)[-1].strip()
        for hw in glob.glob(dev + "/hwmon/hwmon*"):
            for key, fname, scale in (("power_cap_W", "power1_cap", 1e-6), ("power_W", "power1_average", 1e-6),
                                      ("power_W", "power1_input", 1e-6), ("temp_edge_C", "temp1_input", 1e-3),
                                      ("temp_junction_C", "temp2_input", 1e-3), ("temp_memory_C", "temp3_input", 1e-3)):
                try:
                    st.setdefault(key, round(int(open("%s/%s" % (hw, fname)).read()) * scale, 1))
                except (OSError, ValueError):
                    pass
        if st:
            found[dev.split("/")[4]] = st
    return found or None


def multi_stream_copy(binding, ctx, name, sets, iters, group):
    """The all-reduce kernel itself with the adds removed (N read streams, N write
    streams, same grid, addressing and cache policies), on the same rotating
    buffer sets: the ceiling of this access shape."""
    n, algo, ne, *_ = WORKLOADS[name]
    npairs = (iters + group - 1) // group
    timer = binding.EventTimer(npairs)
    k = 0
    for p in range(npairs):
        timer.start(p)
        for _ in range(group):
            ins, outs = sets[k % len(sets)]
            ctx.stream_probe_multi([b.ptr for b in outs], [b.ptr for b in ins], ne * 2)
            k += 1
        timer.stop(p)
    ctx.sync()
    ms = timer.elapsed_ms(npairs) / group
    timer.close()
    return float(ms.mean())


def hbm_ceilings(binding, ctx):
    """Plain streaming kernels over 2 GiB (nothing cache-resident): what this
    GPU's HBM delivers for pure reads, pure writes and a 1:1 copy."""
    nbytes = 512 << 20
    bufs = [binding.DeviceBuffer(nbytes) for _ in range(8)]
    for b in bufs:
        b.fill(0)
    out = {}
    for label, mode, moved in (("copy", 0, 2 * nbytes), ("read_only", 1, nbytes),
                               ("write_only", 2, nbytes)):
        timer = binding.EventTimer(24)
        for k in range(24):       # src/dst walk over all eight buffers
            timer.start(k)
            ctx.stream_probe(mode, bufs[(2 * k + 1) % 8].ptr, bufs[(2 * k) % 8].ptr, nbytes)
            timer.stop(k)
        ctx.sync()
        ms = timer.elapsed_ms()[8:]
        timer.close()
        out[label + "_GBps"] = round(moved / (float(np.median(ms)) * 1e-3) / 1e9, 1)
    for b in bufs:
        b.free()
    return out


def cpu_leg(name, gpu_results, budget_s):
    """The CPU side of the run, and the only place that touches the oracle: time
    its OpenMP loop for this workload on the host cores (a reported baseline),
    and use its output as the checker for what the GPU produced on the same
    inputs.  `gpu_results` maps a workload name to the per-rank output arrays of
    one GPU launch on fresh inputs."""
    from tests import oracle_lib
    o = oracle_lib.load()

    def reference(wname):
        n, algo, ne, dist, p0, p1, seed = WORKLOADS[wname]
        draw = min(ne, 1 << 24)                 # as setup(): larger inputs repeat a 16 Mi-element draw
        host = [o.generate_dt(DTYPE, draw, seed + r, dist, p0, p1) for r in range(n)]
        if draw < ne:
            host = [np.tile(a, ne // draw) for a in host]
        if algo.startswith("allgather"):
            return host, o.allgather
        if DTYPE == 0:                      # the oracle's vectorised binary16 loop
            return host, (o.bisect if algo == "bisect" else o.rotated)
        mode = oracle_lib.ORDER_BISECT if algo == "bisect" else oracle_lib.ORDER_ROTATED
        return host, (lambda ins: o.order_dt(DTYPE, mode, ins))

    mismatches = {}
    for wname, outs in gpu_results.items():
        host, fn = reference(wname)
        want = fn(host)
        mismatches[wname] = int(sum(o.count_mismatch_dt(DTYPE, g, want) for g in outs))

    host, fn = reference(name)
    n, algo, *_ = WORKLOADS[name]
    forms = [("device_order", fn)]
    if not algo.startswith("allgather"):
        # the reference's own host oracle: per element a chain over the ranks in rank
        # order (allreduce.cpp:18-27), OpenMP over elements
        if DTYPE == 0:
            forms.append(("reference_rank_order", o.rank_order))
        else:
            forms.append(("reference_rank_order", lambda ins: o.order_dt(DTYPE, oracle_lib.ORDER_RANK, ins)))
    env = os.environ.get("OMP_NUM_THREADS")
    all_threads = int(env) if env else min(os.cpu_count() or 1, 64)
    share = budget_s / (2 * len(forms))
    timing = {}
    for form, f in forms:
        for label, threads in (("all", all_threads), ("one", 1)):
            used = o.set_threads(threads)
            f(host)                                          # warm-up, page faults
            best, reps, t_start = 1e30, 0, time.perf_counter()
            while True:
                t0 = time.perf_counter()
                f(host)
                dt = time.perf_counter() - t0
                best, reps = min(best, dt), reps + 1
                elapsed = time.perf_counter() - t_start
                if (reps >= 5 and elapsed > share / 2) or elapsed > share:
                    break
            timing[(form, label)] = (algorithmic_bytes(name) / best / 1e9, used, reps, best)
    o.set_threads(all_threads)
    gb_all, cores, reps, best = timing[("device_order", "all")]
    orders = {form: {"GBps_all_threads": round(timing[(form, "all")][0], 3),
                     "GBps_one_thread": round(timing[(form, "one")][0], 3),
                     "ms_all_threads": round(timing[(form, "all")][3] * 1e3, 2)}
              for form, _ in forms}
    text = "%s full size, best of %d passes (%.1f ms); 1 thread: %.3f GB/s" % (
        name, reps, best * 1e3, timing[("device_order", "one")][0])
    if "reference_rank_order" in orders:
        text += "; the reference's rank-order host sum (allreduce.cpp:18-27): %.3f GB/s on %d threads, " \
                "%.3f GB/s on 1" % (orders["reference_rank_order"]["GBps_all_threads"], cores,
                                    orders["reference_rank_order"]["GBps_one_thread"])
    baseline = {"value": round(gb_all, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": text, "orders": orders}
    return baseline, mismatches


def sweep_rows(vr, binding, ctx, bufs, host, algo, tr, sizes, iters_for):
    """One protocol over the given per-rank sizes, in place on one buffer set (the
    reference's own run protocol, main.cpp:67-108): microseconds (median of
    per-launch HIP-event times) and algorithmic GB/s per size."""
    n = ctx.nranks
    rows = []
    for S in sizes:
        ne = S // 2
        for b in bufs:
            b.upload(host[:ne])
        ptrs = [b.ptr for b in bufs]
        ctx.time_allreduce(algo, ptrs, ne, 3, transport=tr)
        ms = ctx.time_allreduce(algo, ptrs, ne, iters_for(S, tr == vr.TRANSPORT_DIRECT), transport=tr)
        ctx.check()
        us = float(np.median(ms)) * 1e3
        rows.append({"bytes_per_rank": S, "us": round(us, 2),
                     "GBps": round(2 * n * S / (us * 1e-6) / 1e9, 1)})
    return rows


def sweep_inputs(binding, max_bytes):
    draw = min(max_bytes // 2, 1 << 24)
    host = binding.generate(draw, 5000, 1, 0.0, 1.0, dtype=DTYPE)
    return np.tile(host, (max_bytes // 2) // draw) if draw < max_bytes // 2 else host


def sweep(vr, binding, args):
    """The size sweep: 8 virtual ranks, per-rank sizes 4 KiB ... 256 MiB in powers of
    two, in place on one buffer set, N(0,1) inputs.  One line of JSON: GB/s and us per
    size for each protocol, and the sizes at which the fastest protocol changes."""
    n = 8
    ctx = vr.VirtualRanks(n)
    ctx.set_dtype(DTYPE)
    for kv in args.tune:
        k, v = kv.split("=")
        ctx.set_tuning(**{k: int(v)})
    max_bytes = 256 << 20
    host = sweep_inputs(binding, max_bytes)
    bufs = [binding.DeviceBuffer(max_bytes) for _ in range(n)]
    protos = [("small", vr.TRANSPORT_DIRECT), ("simple", vr.TRANSPORT_DIRECT),
              ("bisect", vr.TRANSPORT_DIRECT), ("parallel", vr.TRANSPORT_WIRE)]
    if args.sweep_wire:
        protos += [(a, vr.TRANSPORT_WIRE) for a in ("small", "simple", "bisect", "small_ring",
                                                     "simple_ring", "small_pcie", "simple_pcie")]
    curves = {}
    sizes = [1 << p for p in range(12, 29)]

    def iters_for(S, direct):
        return (200 if S <= (1 << 22) else 40) if direct else (30 if S <= (1 << 22) else 5)

    for algo, tr in protos:
        key = algo + ("@wire" if tr == vr.TRANSPORT_WIRE and algo != "parallel" else "")
        curves[key] = sweep_rows(vr, binding, ctx, bufs, host, algo, tr, sizes, iters_for)
    # The fastest protocol per size; a protocol only takes over when it is more
    # than 3 % faster than the incumbent, so that timer noise between kernels
    # that perform alike does not read as a crossover.
    def fastest_of(keys):
        best = []
        for i in range(len(sizes)):
            fastest = min(keys, key=lambda k: curves[k][i]["us"])
            if best and curves[best[-1]][i]["us"] <= 1.03 * curves[fastest][i]["us"]:
                fastest = best[-1]
            best.append(fastest)
        cross = [{"bytes_per_rank": sizes[i], "from": best[i - 1], "to": best[i]}
                 for i in range(1, len(sizes)) if best[i] != best[i - 1]]
        return best, cross

    best, crossovers = fastest_of(list(curves))
    # The same question inside the message-passing family, where the four protocols
    # are different kernels with different wire formats and flows (the form that
    # would run across GPUs): small = 8-byte messages, simple / parallel = 128 / 256-byte
    # messages over ParallelTransmit, bisect = pair exchange + 4-way exchange.
    wire_keys = [k for k in ("small@wire", "simple@wire", "bisect@wire", "parallel") if k in curves]
    wire_best, wire_cross = fastest_of(wire_keys) if len(wire_keys) > 1 else ([], [])
    print(json.dumps({"metric": "allreduce_GBps_vs_size_8vrank_fp16", "unit": "GB/s",
                      "note": "in place on one buffer set: sizes up to 16 MiB/rank are served by "
                              "the caches, 64 MiB/rank and above stream from HBM; times are HIP-event "
                              "times of single launches (~2 us of event overhead included)",
                      "curves": curves, "fastest": dict(zip(map(str, sizes), best)),
                      "crossovers": crossovers,
                      "fastest_message_passing": dict(zip(map(str, sizes), wire_best)),
                      "crossovers_message_passing": wire_cross}))


def latency_block(vr, binding, want_check, gpu_results, iters):
    """Second half of the metric: latency of the 1 MiB/rank `small` all-reduce (config 2),
    in place on cache-resident buffers, every figure taken inside the library (C side)."""
    c2, h2, s2 = setup(vr, binding, "cfg2", True, 1)
    n, algo, ne, *_ = WORKLOADS["cfg2"]
    ptrs = [b.ptr for b in s2[0][0]]
    launch(c2, "cfg2", *s2[0])
    c2.sync()
    if want_check:
        gpu_results["cfg2"] = [b.download(np.uint16, ne) for b in s2[0][0]]
    c2.time_allreduce_kernel(algo, ptrs, ne, 50, transport=TRANSPORT)                 # warm
    kern = c2.time_allreduce_kernel(algo, ptrs, ne, iters, transport=TRANSPORT) * 1e3  # kernel execution, us
    single = c2.time_allreduce(algo, ptrs, ne, iters, transport=TRANSPORT) * 1e3       # event pair per launch
    groups = max(10, iters // 20)
    b2b, host_c = c2.time_allreduce_grouped(algo, ptrs, ne, groups, 20, transport=TRANSPORT)
    b2b = b2b * 1e3
    # the same call through the Python binding (ctypes marshalling on top of the C call)
    t0 = time.perf_counter()
    for _ in range(iters):
        c2.allreduce(algo, ptrs, ne, transport=TRANSPORT)
    host_py = (time.perf_counter() - t0) / iters * 1e6
    c2.sync()
    p50 = float(np.percentile(kern, 50))
    out = {
        "workload": describe("cfg2") + ", in place", "iters": iters,
        "p50_us": round(p50, 3), "p99_us": round(float(np.percentile(kern, 99)), 3),
        "min_us": round(float(kern.min()), 3),
        "what": "kernel execution time per launch, from events attached to each kernel dispatch "
                "(its own begin / end timestamps: what a kernel trace shows and what the reference "
                "prints from its SYCL event, main.cpp:36-43); one launch at a time in the queue's order",
        "kernel_trace_p50_us": CFG2_KERNEL_TRACE[0], "kernel_trace_profile": CFG2_KERNEL_TRACE[1],
        "event_pair_per_launch": {"p50_us": round(float(np.percentile(single, 50)), 3),
                                  "p99_us": round(float(np.percentile(single, 99)), 3),
                                  "note": "hipEventRecord before and after each launch: adds the event "
                                          "commands' own time to the kernel's"},
        "back_to_back_us_per_launch": round(float(np.median(b2b)), 3),
        "host_call_us": {"c_abi": round(host_c, 3), "through_ctypes": round(host_py, 3),
                         "note": "host wall time for one vr_allreduce call to return (validation, launch "
                                 "heuristics, kernel enqueue), mean over back-to-back calls; c_abi is "
                                 "measured inside the library's own loop"},
        "bit_exact_vs_oracle": None,
        "GBps_at_p50": round(algorithmic_bytes("cfg2") / (p50 * 1e-6) / 1e9, 1),
    }
    return out


def allgather_block(vr, binding, want_check, gpu_results):
    """Config 4: 4 virtual ranks, all-gather of 8 MiB slices into 32 MiB outputs.  The
    headline figures rotate through 16 buffer sets: 512 MiB of inputs, twice the
    256 MiB memory-side cache, so that the reads come from HBM like the writes go to
    it (2.5 GiB touched).  With 4 sets the 128 MiB of inputs stay in that cache (the
    streaming stores do not displace them) and only the writes reach HBM: printed as
    `inputs_cache_resident`, not an HBM figure."""
    name = "cfg4"
    n, algo, ne, *_ = WORKLOADS[name]
    c4, h4, s4 = setup(vr, binding, name, False, 16)
    launch(c4, name, *s4[0])
    c4.sync()
    if want_check:
        gpu_results[name] = [b.download(np.uint16, n * ne) for b in s4[0][1]]
    time_kernels(binding, c4, name, s4, 16)
    kms, stats = kernel_sample(binding, c4, name, s4, 10)
    B = algorithmic_bytes(name)
    gb = B / (float(kms.mean()) * 1e-3) / 1e9
    out = {"workload": describe(name), "GBps": round(gb, 1), "frac_of_hbm_peak": round(gb / HBM_PEAK_GBPS, 4),
           "algorithmic_bytes_per_step": B, "traffic": measured_traffic(name, "default"),
           "buffer_sets_rotated": len(s4), "bit_exact_vs_oracle": None,
           "launch": binding.direct_launch_plan(WORKLOADS[name][1], WORKLOADS[name][0], WORKLOADS[name][2], False)}
    out.update(stats)
    time_kernels(binding, c4, name, s4[:4], 8)
    warm, wstats = kernel_sample(binding, c4, name, s4[:4], 10)
    wgb = B / (float(warm.mean()) * 1e-3) / 1e9
    out["inputs_cache_resident"] = {
        "GBps": round(wgb, 1), "kernel_us_avg": wstats["kernel_us_avg"], "buffer_sets_rotated": 4,
        "note": "4 sets: their 128 MiB of inputs fit the 256 MiB memory-side cache, so the reads "
                "(a fifth of the bytes) are served by it; not an HBM figure"}
    return out


def cfg5_block(vr, binding):
    """Config 5 at three sizes: its named protocol `parallel` (message passing through
    scratch) and the direct kernel (`simple`), in place on one buffer set as the
    reference's own run protocol has it (main.cpp:67-108)."""
    n = 8
    sizes = [1 << 20, 32 << 20, 256 << 20]
    ctx = vr.VirtualRanks(n)
    ctx.set_dtype(DTYPE)
    host = sweep_inputs(binding, sizes[-1])
    bufs = [binding.DeviceBuffer(sizes[-1]) for _ in range(n)]

    def iters_for(S, direct):
        return {1 << 20: 200, 32 << 20: 40, 256 << 20: 10}[S] if direct else {1 << 20: 40, 32 << 20: 10, 256 << 20: 4}[S]

    out = {"sizes_bytes_per_rank": sizes,
           "parallel": sweep_rows(vr, binding, ctx, bufs, host, "parallel", vr.TRANSPORT_WIRE, sizes, iters_for),
           "direct_simple": sweep_rows(vr, binding, ctx, bufs, host, "simple", vr.TRANSPORT_DIRECT, sizes, iters_for),
           "note": "8 virtual ranks, N(0,1), in place on one buffer set (1 MiB per rank is served by the "
                   "caches; 32 MiB per rank, a footprint of exactly the memory-side cache's size, and 256 MiB "
                   "per rank are launched as streaming); median of single-launch "
                   "HIP-event times; the full 17-point curves: bench.py --sweep"}
    for b in bufs:
        b.free()
    ctx.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg3", choices=sorted(WORKLOADS) + ["copy", "read_only", "write_only"],
                    help="'copy' runs only the plain streaming copy (512 MiB per launch), the "
                         "known-size kernel that hardware-counter readings are scaled by")
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"],
                    help="element type of the adds (the reference instantiates both)")
    ap.add_argument("--transport", default="default", choices=["default", "direct", "wire", "static"],
                    help="direct: one pass over HBM; wire: the reference's message passing through "
                         "scratch; default: wire for 'parallel', direct otherwise; static: the "
                         "allocation-free entry point (wire transport through the library's fixed region)")
    ap.add_argument("--inplace", action="store_true",
                    help="reference semantics: results overwrite the inputs (values saturate "
                         "after a few steps; traffic is identical)")
    ap.add_argument("--sets", type=int, default=None,
                    help="buffer sets the steps rotate through (1 = reuse one set, cache-warm); default 4, "
                         "2 from 64 MiB per rank on")
    ap.add_argument("--event-group", type=int, default=10,
                    help="launches bracketed by one HIP event pair when timing kernels")
    ap.add_argument("--only-headline", action="store_true",
                    help="run nothing but the headline workload (for profiler runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--latency-iters", type=int, default=1000)
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VAL")
    ap.add_argument("--sweep", action="store_true",
                    help="GB/s-vs-size curves of small / simple / bisect / parallel and their "
                         "crossover sizes instead of the headline measurement")
    ap.add_argument("--sweep-wire", action="store_true",
                    help="with --sweep: add every message-passing flow to the curves")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every virtual rank lives in one MI355X's HBM; "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import gpu_ipc_example_amd as vr
    from gpu_ipc_example_amd import binding

    global DTYPE, TRANSPORT, STATIC
    DTYPE = 1 if args.dtype == "bf16" else 0
    STATIC = args.transport == "static"
    TRANSPORT = {"default": vr.TRANSPORT_DEFAULT, "direct": vr.TRANSPORT_DIRECT,
                 "wire": vr.TRANSPORT_WIRE, "static": vr.TRANSPORT_WIRE}[args.transport]

    if args.sweep:
        sweep(vr, binding, args)
        return

    if args.workload in ("copy", "read_only", "write_only"):
        # the streaming yardsticks alone: 512 MiB per launch, source and destination walking
        # over eight buffers (4 GiB), median of single-launch HIP-event times
        mode = {"copy": 0, "read_only": 1, "write_only": 2}[args.workload]
        ctx = vr.VirtualRanks(8)
        for kv in args.tune:
            k, v = kv.split("=")
            ctx.set_tuning(**{k: int(v)})
        nbytes = 512 << 20
        bufs = [binding.DeviceBuffer(nbytes) for _ in range(8)]
        for b in bufs:
            b.fill(0)
        timer = binding.EventTimer(args.steps)
        for k in range(args.steps):
            timer.start(k)
            ctx.stream_probe(mode, bufs[(2 * k + 1) % 8].ptr, bufs[(2 * k) % 8].ptr, nbytes)
            timer.stop(k)
        ctx.sync()
        ms = timer.elapsed_ms()
        moved = 2 * nbytes if mode == 0 else nbytes
        print(json.dumps({"metric": "plain_%s_bandwidth" % args.workload, "unit": "GB/s",
                          "bytes_read": nbytes if mode != 2 else 0, "bytes_written": nbytes if mode != 1 else 0,
                          "launches": args.steps, "tune": args.tune,
                          "value": round(moved / (float(np.median(ms)) * 1e-3) / 1e9, 1)}))
        return

    name = args.workload
    n, algo, ne, *_ = WORKLOADS[name]
    B = algorithmic_bytes(name)
    nsets = args.sets if args.sets is not None else (4 if ne * 2 <= (32 << 20) or n * ne * 2 <= (256 << 20) else 2)
    if args.sets is None:
        # the inputs of all sets together are at least twice the 256 MiB memory-side cache
        # (streaming stores do not displace cached inputs, so the inputs alone must not fit it)
        nsets = min(64, max(nsets, -(-(512 << 20) // (n * ne * 2))))
    ctx, host, sets = setup(vr, binding, name, args.inplace, nsets)
    for kv in args.tune:
        k, v = kv.split("=")
        ctx.set_tuning(**{k: int(v)})

    # one launch of exactly this configuration on fresh inputs, kept for the checker
    want_check = not args.no_cpu and not args.only_headline
    gpu_results = {}
    launch(ctx, name, *sets[0])
    ctx.sync()
    if want_check:
        count = (n * ne) if algo.startswith("allgather") else ne
        gpu_results[name] = [b.download(np.uint16, count) for b in (sets[0][1] or sets[0][0])]
    if args.inplace:
        for b, a in zip(sets[0][0], host):
            b.upload(a)

    for i in range(args.warmup):
        launch(ctx, name, *sets[i % len(sets)])
    ctx.sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        launch(ctx, name, *sets[i % len(sets)])
    ctx.sync()
    wall = time.perf_counter() - t0
    ctx.check()            # outside the timed region: a wire-transport poll time-out voids the run
    ms_per_step = wall / args.steps * 1e3
    value = B / (wall / args.steps) / 1e9

    # kernel durations from HIP events on the launch stream: a sample of fixed size
    # (the --steps launches above are the wall-clock figure; this is the kernel figure)
    kms, kstats = kernel_sample(binding, ctx, name, sets, args.event_group)
    k_avg = float(kms.mean())
    achieved = B / (k_avg * 1e-3) / 1e9

    roofline = {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": measured_traffic(name, args.transport)}
    roofline.update(kstats)
    result = {
        "metric": ("allreduce_algorithmic_hbm_bandwidth_8vrank_%s_32MiB_per_rank"
                   % ("bf16" if DTYPE else "fp16"))
                  if name == "cfg3" else "algorithmic_hbm_bandwidth_" + name,
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": DTYPE_NAMES[DTYPE], "data": "synthetic",
        "config": {"workload": describe(name), "virtual_ranks": n, "protocol": algo,
                   "transport": args.transport,
                   "bytes_per_rank": ne * 2, "in_place": bool(args.inplace),
                   "algorithmic_bytes_per_step": B, "buffer_sets_rotated": len(sets),
                   "note": "steps rotate through %d buffer sets (%.0f MiB touched) so the 256 MiB "
                           "memory-side cache cannot serve them" % (
                               len(sets), len(sets) * (B if not args.inplace else B / 2) / 2**20)
                           if len(sets) > 1 else "every step reuses one buffer set (cache-warm)"},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "launch": launch_plan(binding, algo, n, ne, args),
        "memory_clock": memory_clock(),
        "device_state": device_state(),
        "bit_exact_vs_oracle": None,
        "roofline": roofline,
    }
    if not algo.startswith("allgather"):
        strict = (n + 1) * ne * 2
        result["strict_GBps_(N+1)S"] = round(strict / (k_avg * 1e-3) / 1e9, 2)

    reduces = not algo.startswith("allgather")
    if len(sets) > 1 and sets[0][1] is not None and reduces and not args.only_headline:
        # the reference's in-place semantics on the same cold sets
        ims = in_place_cold(binding, ctx, name, sets, host)
        result["in_place_cold"] = {
            "GBps": round(B / (float(ims.mean()) * 1e-3) / 1e9, 2),
            "kernel_us_avg": round(float(ims.mean()) * 1e3, 3), "kernel_us_min": round(float(ims.min()) * 1e3, 3),
            "frac": round(B / (float(ims.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "note": "results overwrite the inputs (parallel_transmit.hpp:125-130); %d sets restored from "
                    "the inputs by a device copy before every round, outside the timing; the library "
                    "sees %d MiB of in-place footprint and picks its launch policy from that" % (
                        len(sets), B // 2 >> 20)}

    if len(sets) > 1 and not args.only_headline:
        # the same launches on ONE buffer set, with cached instead of streaming loads
        # so that the inputs stay in the memory-side cache
        if not args.tune:
            ctx.set_tuning(nt_load=0, waves_per_cu=8, f16_wide=0)
        time_kernels(binding, ctx, name, sets[:1], 10)
        wms = time_kernels(binding, ctx, name, sets[:1], 50, group=10)
        if not args.tune:
            ctx.set_tuning(nt_load=-1, waves_per_cu=-1, f16_wide=-1)
        result["same_buffers_cache_warm"] = {
            "GBps": round(B / (float(wms.mean()) * 1e-3) / 1e9, 2),
            "kernel_us_avg": round(float(wms.mean()) * 1e3, 3),
            "note": "one buffer set, cached loads: inputs served by the Infinity Cache; "
                    "not an HBM figure"}

    if not args.only_headline and (name == "cfg3" or reduces):
        if name == "cfg3":
            result["latency_1MiB_per_rank"] = latency_block(vr, binding, want_check, gpu_results, args.latency_iters)
        result["hbm_ceilings"] = hbm_ceilings(binding, ctx)
        if sets[0][1] is not None and reduces and TRANSPORT != vr.TRANSPORT_WIRE and algo != "parallel":
            # the same kernel, grid and policies without the adds, on the same buffer sets
            time_kernels(binding, ctx, name, sets, 8)                      # back to steady state
            c_ms = multi_stream_copy(binding, ctx, name, sets, 100, 10)
            a_ms = float(time_kernels(binding, ctx, name, sets, 100, group=10).mean())
            result["hbm_ceilings"]["same_shape_no_adds"] = {
                "kernel_us_avg": round(c_ms * 1e3, 3), "GBps": round(B / (c_ms * 1e-3) / 1e9, 1),
                "allreduce_us_avg_same_run": round(a_ms * 1e3, 3),
                "note": "k_direct_allreduce with the adds removed: %d read + %d write streams, same "
                        "grid, buffer addressing and nt / nt sc1 policies, same rotating buffer sets" % (n, n)}
        if name == "cfg3":
            # free the headline's 2 GiB before the other configurations allocate theirs
            for ins, outs in sets:
                for b in ins + (outs or []):
                    b.free()
            result["cfg4_allgather"] = allgather_block(vr, binding, want_check, gpu_results)
            result["cfg5_sweep_points"] = cfg5_block(vr, binding)

    if want_check:
        result["cpu_baseline"], bad = cpu_leg(name, gpu_results, args.cpu_seconds)
        result["bit_exact_vs_oracle"] = bad[name] == 0
        result["mismatches"] = bad[name]
        if "cfg2" in bad and "latency_1MiB_per_rank" in result:
            result["latency_1MiB_per_rank"]["bit_exact_vs_oracle"] = bad["cfg2"] == 0
        if "cfg4" in bad and "cfg4_allgather" in result:
            result["cfg4_allgather"]["bit_exact_vs_oracle"] = bad["cfg4"] == 0
    print(json.dumps(result, default=float))


if __name__ == "__main__":
    main()
