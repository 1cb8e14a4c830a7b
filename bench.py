#!/usr/bin/env python3
"""Benchmark of the MI355X allreduce hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|3|4|5] [--no-others] [--all-configs] [--full]
    python bench.py --only-roofline [--config N]     the kernel leg alone (what the counter profiles run)
    python bench.py --whole-buffer                    adds roofline.whole_buffer_launch to the line
    python bench.py --sweep [--config N]              every kernel variant of the measurement library at the launch shape
    python bench.py --ceiling [--config N]            the best variant, the shipped kernel on a large launch, hipMemcpyAsync
    python bench.py --call-breakdown [--config N]     where the time of one blocking call goes, from the library's own trace

One "step" is one rank's complete allreduce schedule on the GPU -- one GPU's share of the
collective: every partial sum the rank receives is added to its own contribution (the result going
to a pool slot for forwarding, or to recvbuf), every finished chunk is gathered into recvbuf,
exactly as in the full world.  The other emulated ranks are replaced by a recording of
what they sent (made by first running the whole world once, all sendbufs resident in HBM), paced
the way the real dependency on upstream ranks paces them.  The headline `value` is the allreduce
algorithm bandwidth of that schedule, len * 4 B / time per step.  `extra.world_all_ranks_on_one_gpu`
gives the same figure when all N ranks' schedules are executed on the one GPU per step.  Default
workload: configs[1] of BASELINE.json (ring, 8 ranks, 256 MiB fp32 per rank, IBCOMM_CHUNKSIZE = 8 MiB).

Two more legs, both on rank 0 of a one-GPU run:
  roofline      the dominant kernel (the segment reduction, dst = a + b at 12 B per fp32 element)
                launched at the shape the schedule launches it, back to back on one stream, timed
                with HIP events recorded on that stream.
  cpu_baseline  the CPU oracle's restatement of the reference's AllreduceRing<float> (scalar loop,
                gcc -O2, one thread per emulated rank) on the same workload, timed on the host.
The oracle is used only as that baseline and as the checker of the final result.

The default run also carries, under `extra`:
  other_configs   configurations 4 and 3 (5 with --all-configs) measured the same way after the headline one: rank
                  and whole-world time per step, the kernel-landing variant, and the roofline leg of their dominant launch
  reference_api   the reference's own entry point and protocol: the example program built against the drop-in header,
                  one thread per rank in blocking AllreduceRingCuda calls, 3 warm-ups then timed calls, configurations 2 and 4
and under `roofline`, `in_schedule_*`: the kernels' own durations inside the rank's schedule, taken from the
library's trace of eagerly issued calls (each launch leaves its own begin and end timestamps there).

--sweep and --ceiling use libibcomm_hip_bench.so (allreduce-proto_amd/csrc/bench_variants.hip): alternative
forms of the kernel, built for measuring only; the default run loads it for `roofline.ceiling` (the best of
those forms at the launch shape, next to the shipped kernel).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E

# HBM bytes per launch of the reduction kernel from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE),
# each calibrated against a device copy of known size; the summaries with the commands are under
# profiles/.  Shapes that have not been measured report null.
MEASURED_TRAFFIC_BYTES = {
    # (launch shape, workgroup size, die-local tile order, sc1 stores) of the aligned kernel -> bytes;
    # all four from profiles/aligned_add_kernel_traffic_four_configs.md
    ("1 segments x 8388608 fp32", 128, 1, 1): 100676300,     # config 2
    ("2 segments x 25165824 fp32", 128, 1, 0): 603980781,    # config 3
    ("1 segments x 2097152 fp32", 256, 1, 1): 25179438,      # config 4
    ("1 segments x 16777216 fp32", 128, 1, 1): 201344831,    # config 5
}

CONFIGS = {
    # id: (algo name, ranks, elements per rank, IBCOMM_CHUNKSIZE, data)
    2: ("ring", 8, 67108864, 8388608, "normal"),
    3: ("rabenseifner", 16, 102760448, 4194304, "normal1e-2"),
    4: ("ring", 8, 16777216, 65536, "uniform"),
    5: ("ring", 32, 536870911, 16777216, "normal"),
}


def make_inputs(torch, world, n, kind, seed):
    out = []
    for r in range(world):
        g = torch.Generator(device="cuda").manual_seed(seed + r)
        if kind == "normal":
            t = torch.randn(n, device="cuda", generator=g)
        elif kind == "normal1e-2":
            t = torch.randn(n, device="cuda", generator=g) * 1e-2
        else:
            t = torch.rand(n, device="cuda", generator=g) * 2 - 1
        out.append(t)
    return out


def check_result(torch, O, H, algo, send, recv, chunk):
    """Bit-exact check of the last step's result: every rank on one chunk group with torch's fp32 adds
    in the reference's order, and rank 0's first and last chunk against the oracle on the host."""
    import numpy as np
    world, n = len(send), send[0].numel()
    rc, ranges = O.split_buffer(n, 4, world, chunk)
    assert rc == 0
    groups = O.rank_to_chunk(len(ranges), world)
    it = torch.int32
    if algo == H.RING:
        g = world // 2
        s, e = ranges[groups[g][0]][0], ranges[groups[g][-1]][1]
        acc = send[g][s:e].clone()
        for j in range(1, world):
            acc += send[(g + j) % world][s:e]
    else:
        s, e = ranges[groups[0][0]][0], ranges[groups[0][-1]][1]
        level = [t[s:e] for t in send]
        while len(level) > 1:
            level = [level[i] + level[i + 1] for i in range(0, len(level), 2)]
        acc = level[0]
    ok = all(torch.equal(recv[r][s:e].view(it), acc.view(it)) for r in range(world))
    owner = {c: gi for gi, cs in enumerate(groups) for c in cs}
    for c in (0, len(ranges) - 1):
        s, e = ranges[c]
        host = [t[s:e].cpu().numpy() for t in send]
        if algo == H.RING:
            rot = host[owner[c]:] + host[:owner[c]]
            want = rot[0].copy()
            for x in rot[1:]:
                O.lib().orc_reduce_inplace(O.F32, want.ctypes.data, x.ctypes.data, want.size)
        else:
            rc, want = O.closed_form_tree(host)
        ok = ok and np.array_equal(recv[0][s:e].cpu().numpy().view(np.uint32), want.view(np.uint32))
    return bool(ok)


def launch_tables(send, recv, seg_elems, k, staging=None):
    """Operand tables for launches of k segments x seg_elems.  The operands that are READ are distinct
    ranges of two ranks' sendbufs at the same offset, successive launches walking through all ranks'
    buffers (at least 2 GiB per pass), none of them ever written: nothing that is read comes out of a
    cache.  The operand that is WRITTEN goes where the schedule puts it: with `staging` (a device
    buffer of the size of a rank's staging working set) the launches cycle through that buffer, as a
    rank's reductions cycle through the few pool slots they stage their results in; without it dst
    walks through all ranks' recvbufs."""
    world = len(send)
    vp = C.c_void_p
    n = send[0].numel()
    per_buf = max(1, n // seg_elems)
    shapes = []
    # enough launches' worth of distinct operands that a pass over the tables reads at least 2 GiB
    tables = max(world * 2, -(-(2 << 30) // (8 * seg_elems * k)))
    stage_segments = max(1, staging.numel() // seg_elems) if staging is not None else 0
    for i in range(tables):
        dst, a, b = [], [], []
        for j in range(k):
            idx = (i * k + j)
            r = idx % world
            off = ((idx // world) % per_buf) * seg_elems * 4
            if staging is not None:
                dst.append(staging.data_ptr() + (idx % stage_segments) * seg_elems * 4)
            else:
                dst.append(recv[r].data_ptr() + off)
            a.append(send[r].data_ptr() + off)
            b.append(send[(r + world // 2) % world].data_ptr() + off)
        shapes.append(((vp * k)(*dst), (vp * k)(*a), (vp * k)(*b), (C.c_size_t * k)(*([seg_elems] * k))))
    return shapes


def time_launches(torch, stream, launch, launches, warm=5):
    """Average seconds per launch: HIP events recorded on the stream the launches go to."""
    with torch.cuda.stream(stream):
        for i in range(warm):
            launch(i)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(launches):
            launch(i)
        e1.record(stream)
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / launches


def roofline_leg(torch, H, send, recv, seg_elems, segs_per_launch, launches, staging=None):
    """Average duration of the dominant kernel at its in-schedule launch shape, HIP events on its own stream."""
    stream = torch.cuda.Stream()
    k = segs_per_launch
    shapes = launch_tables(send, recv, seg_elems, k, staging)
    L = H.lib()

    def launch(i):
        d, a, b, ln = shapes[i % len(shapes)]
        rc = L.ibcomm_hip_reduce_segments(H.F32, k, d, a, b, ln, stream.cuda_stream)
        assert rc == 0, H.last_error()

    avg_s = time_launches(torch, stream, launch, launches)
    algorithmic = 12.0 * seg_elems * k
    aligned, threads, die_local, through = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    d, a, b, ln = shapes[0]
    assert L.ibcomm_hip_describe_launch(H.F32, k, d, a, b, ln, C.byref(aligned), C.byref(threads), C.byref(die_local), C.byref(through)) == 0
    shape = "%d segments x %d fp32" % (k, seg_elems)
    return {
        "bound": "hbm",
        "achieved": round(algorithmic / avg_s * 1e-9, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(algorithmic / avg_s * 1e-9 / HBM_PEAK_GBPS, 4),
        # counter traffic is known for the kernel geometry it was collected on, and only for that
        "traffic": MEASURED_TRAFFIC_BYTES.get((shape, threads.value, die_local.value, through.value)) if aligned.value else None,
        "kernel": "ibcomm_hip::%s<float4, %d threads, add>, %s tile order, non-temporal loads, %s stores" % (
            ("Aligned" if aligned.value else "") + ("OneSegmentKernel" if k == 1 else "SegmentKernel"), threads.value,
            "die-local" if die_local.value else "plain", "agent-scope (sc1)" if through.value else "non-temporal"),
        "launch_shape": shape,
        "algorithmic_bytes_per_launch": int(algorithmic),
        "avg_launch_us": round(avg_s * 1e6, 2),
        "launches_timed": launches,
        "result_goes_to": ("a staging region of %d bytes, cycled through as a rank's reductions cycle through their pool slots"
                           % (staging.numel() * 4)) if staging is not None else "all ranks' recvbufs in turn",
    }


# ---- the measurement library: kernel variants -------------------------------------------------------

_bench_lib = None


def bench_lib():
    global _bench_lib
    if _bench_lib is None:
        path = os.path.join(ROOT, "allreduce-proto_amd", "libibcomm_hip_bench.so")
        if not os.path.exists(path):
            raise RuntimeError("%s is not built; run __graft_entry__.build()" % path)
        B = C.CDLL(path)
        vp, sz, i = C.c_void_p, C.c_size_t, C.c_int
        B.ibv_last_error.restype = C.c_char_p
        B.ibv_variant_name.restype = C.c_char_p
        B.ibv_variant_name.argtypes = [i]
        B.ibv_variant_accepts.argtypes = [i, sz]
        B.ibv_variant_launch.argtypes = [i, vp, vp, vp, sz, vp]
        _bench_lib = B
    return _bench_lib


def variant_times(torch, H, send, recv, total_elems, add, launches=60, passes=3, staging=None):
    """Every variant that takes `total_elems` fp32 in one segment, and the shipped kernel on the same
    operands: -> [(name, seconds per launch)], shipped kernel first.  Each figure is the median of
    `passes` HIP-event averages over `launches` back-to-back launches; the passes go round all variants,
    so that a drift of the device over the run touches all of them alike, and a best-of-many is not
    just the luckiest single measurement."""
    B = bench_lib()
    L = H.lib()
    stream = torch.cuda.Stream()
    shapes = launch_tables(send, recv, total_elems, 1, staging)

    def shipped(i):
        d, a, b, ln = shapes[i % len(shapes)]
        if add:
            rc = L.ibcomm_hip_reduce_segments(H.F32, 1, d, a, b, ln, stream.cuda_stream)
        else:
            rc = L.ibcomm_hip_copy_segments(H.F32, 1, d, a, ln, stream.cuda_stream)
        assert rc == 0, H.last_error()

    def variant(v):
        def launch(i):
            d, a, b, _ = shapes[i % len(shapes)]
            rc = B.ibv_variant_launch(v, d[0], a[0], b[0] if add else None, total_elems, stream.cuda_stream)
            assert rc == 0, B.ibv_last_error()
        return launch

    def off_grid(shift_d, shift_a, shift_b, elems):
        # the shipped kernel on operands moved off the 16-byte grid (bytes) and on a ragged length, inside the same ranges
        ln = (C.c_size_t * 1)(elems)
        moved = [((C.c_void_p * 1)(d[0] + shift_d), (C.c_void_p * 1)(a[0] + shift_a), (C.c_void_p * 1)(b[0] + shift_b)) for d, a, b, _ in shapes]

        def launch(i):
            d, a, b = moved[i % len(moved)]
            if add:
                rc = L.ibcomm_hip_reduce_segments(H.F32, 1, d, a, b, ln, stream.cuda_stream)
            else:
                rc = L.ibcomm_hip_copy_segments(H.F32, 1, d, a, ln, stream.cuda_stream)
            assert rc == 0, H.last_error()
        return launch

    name = "ibcomm_hip_reduce_segments" if add else "ibcomm_hip_copy_segments"
    runners = [("shipped kernel (%s)" % name, shipped),
               ("shipped kernel, all operands 4 bytes off the 16-byte grid, %d elements" % (total_elems - 4), off_grid(4, 4, 4, total_elems - 4)),
               ("shipped kernel, ragged length of %d elements" % (total_elems - 1), off_grid(0, 0, 0, total_elems - 1)),
               ("shipped kernel, operands at three different 16-byte phases (dst +0, a +4, b +8 bytes), %d elements" % (total_elems - 4),
                off_grid(0, 4, 8, total_elems - 4)),
               ("shipped kernel, 16 bytes off the 128-byte grid, %d elements" % (total_elems - 4), off_grid(16, 16, 16, total_elems - 4))]
    runners += [(B.ibv_variant_name(v).decode(), variant(v)) for v in range(B.ibv_variant_count()) if B.ibv_variant_accepts(v, total_elems)]
    samples = [[] for _ in runners]
    for _ in range(passes):
        for k, (_, fn) in enumerate(runners):
            samples[k].append(time_launches(torch, stream, fn, launches))
    return [(name, sorted(samples[k])[passes // 2]) for k, (name, _) in enumerate(runners)]


def ceiling_leg(torch, H, send, recv, seg_elems, segs_per_launch, shipped_us, full=False, staging=None):
    """How far the shipped kernel is from the best any measured form of the kernel reaches at this launch
    size ("the ceiling"), what the shipped kernel sustains once a launch is large, and the runtime's own
    device-to-device copy as a 1 read : 1 write datum."""
    total = seg_elems * segs_per_launch
    times = variant_times(torch, H, send, recv, total, add=True, staging=staging)
    others = [t for t in times if not t[0].startswith("shipped kernel")]
    best = min(others, key=lambda t: t[1])
    again = times[0][1]
    out = {
        "what": "best of %d other forms of dst = a + b (libibcomm_hip_bench.so) on %d fp32 in one segment, same operands, "
                "median of 3 HIP-event averages over 60 launches each" % (len(others), total),
        "best_variant": best[0],
        "best_variant_us": round(best[1] * 1e6, 2),
        "shipped_kernel_us_same_pass": round(again * 1e6, 2),
        "shipped_over_best": round(again / best[1], 4),
        "best_variant_frac_of_peak": round(12.0 * total / best[1] * 1e-9 / HBM_PEAK_GBPS, 4),
    }
    if full:
        n = send[0].numel()
        big = roofline_leg(torch, H, send, recv, n, 1, 40)
        out["shipped_kernel_large_launch"] = {k: big[k] for k in ("launch_shape", "avg_launch_us", "achieved", "frac")}
        stream = torch.cuda.Stream()
        world = len(send)

        def memcpy(i):
            with torch.cuda.stream(stream):
                recv[i % world].copy_(send[(i + 1) % world], non_blocking=True)

        t = time_launches(torch, stream, memcpy, 40)
        out["hipMemcpyAsync_device_to_device"] = {"bytes_moved": 8 * n, "us": round(t * 1e6, 2), "GBps_at_8B_per_element": round(8.0 * n / t * 1e-9, 1),
                                                  "frac_of_peak": round(8.0 * n / t * 1e-9 / HBM_PEAK_GBPS, 4)}
    return out


def cpu_baseline_leg(O, world, n, chunk, algo_name):
    """The oracle's CPU ring (AllreduceRing<float> restated) on the same workload, one thread per rank."""
    import numpy as np
    bufs = [np.random.default_rng(900 + r).standard_normal(n).astype(np.float32) for r in range(world)]
    algo = O.RING_CPU if algo_name == "ring" else O.RABEN_CPU
    recv = [np.empty_like(b) for b in bufs]
    times = []
    for i in range(16):  # 1 warm-up + 15 timed
        t0 = time.perf_counter()
        rc = O.allreduce_into(algo, bufs, recv, chunk if algo_name == "ring" else None)
        t1 = time.perf_counter()
        assert rc == 0
        if i:
            times.append(t1 - t0)
    del recv
    t = min(times)
    # The reference's own CPU-runnable case and timing protocol (examples/allreduce.cpp:28-29, 87-94, 107-118):
    # 4 ranks x 4,194,304 integer-valued floats, default chunking, 3 warm-ups then one timed run.
    n1 = 4 * 1024 * 1024
    bufs1 = [np.random.default_rng(r).integers(-1000, 1001, n1).astype(np.float32) for r in range(4)]
    recv1 = [np.empty_like(b) for b in bufs1]
    for i in range(4):
        t0 = time.perf_counter()
        rc = O.allreduce_into(O.RING_CPU, bufs1, recv1, None)
        t_cfg1 = time.perf_counter() - t0
        assert rc == 0
    exact = np.sum(np.stack(bufs1).astype(np.int64), axis=0)
    cfg1_ok = all(bool(np.array_equal(r.astype(np.int64), exact)) for r in recv1)
    single_n = 64 * 1024 * 1024  # 256 MiB per operand: memory-bound on any host
    single = O.lib().orc_time_reduce_f32(single_n, 3)
    import subprocess
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), "unknown")
    except OSError:
        pass
    try:
        gcc = subprocess.run(["gcc", "--version"], capture_output=True, text=True).stdout.splitlines()[0]
    except (OSError, IndexError):
        gcc = "unknown"
    return {
        "value": round(n * 4 / t * 1e-9, 3),
        "unit": "GB/s algbw",
        "cores": min(world, os.cpu_count() or 1),
        "kind": "port",
        "cpu_model": model,
        "logical_cpus": os.cpu_count() or 1,
        "pinning": "none (threads placed by the kernel's scheduler)",
        "compiler": "%s, -O2 (the reference's release flags), scalar loop not vectorised by this gcc" % gcc,
        "sample": "%s, %d ranks x %d fp32, IBCOMM_CHUNKSIZE=%s, whole workload, best of 15 after 1 warm-up, "
                  "one host thread per emulated rank on %d logical CPUs" % (algo_name, world, n, chunk, os.cpu_count() or 1),
        "seconds": round(t, 3),
        "seconds_median": round(sorted(times)[len(times) // 2], 3),
        "single_core_reduce_loop_GBps": round(12.0 * single_n / single * 1e-9, 2),
        "config1_ring_4x16MiB": {"seconds": round(t_cfg1, 4), "algbw_GBps": round(n1 * 4 / t_cfg1 * 1e-9, 3), "threads": 4,
                                 "protocol": "3 warm-ups + 1 timed run", "equals_exact_integer_sum": cfg1_ok},
    }


def print_variant_table(title, times, bytes_per_launch):
    print(title)
    print("%-100s %10s %10s %8s" % ("variant", "us/launch", "GB/s", "of peak"))
    for name, t in times:
        print("%-100s %10.2f %10.1f %8.4f" % (name, t * 1e6, bytes_per_launch / t * 1e-9, bytes_per_launch / t * 1e-9 / HBM_PEAK_GBPS), flush=True)


def call_breakdown(torch, H, w, rank, algo, send_ptr, out_ptr, n):
    """Where one blocking call of the rank's schedule spends its time, from the library's trace: the launches' own
    durations when the call is issued eagerly, and for graph replays the host spans "graph launched" and "waiting for
    the completion flag" next to the device's first-kernel-to-end duration."""
    import statistics as st
    import tempfile
    fn = H.lib().ibcomm_hip_replay_allreduce
    args = (w.comms[rank], C.c_int(algo), C.c_int(H.F32), C.c_void_p(send_ptr), C.c_void_p(out_ptr), C.c_size_t(n))

    def wall(calls):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(calls):
            assert fn(*args) == 0, H.last_error()
        return (time.perf_counter() - t0) / calls * 1e6

    def traced(calls):
        base = os.path.join(tempfile.mkdtemp(), "trace")
        os.environ["IBCOMM_TRACE_FILE"] = base
        w.set_trace(True)
        t = wall(calls)
        w.dump_trace()
        w.set_trace(False)
        lines = {name: [] for name in ("device-redu-kernel", "device-copy-kernel", "device-graph")}  # written only when device work was timed
        lines.update({ln.split(",")[0]: [float(x) for x in ln.split(",")[1:-1]] for ln in open("%s_%d.dat" % (base, rank)).read().splitlines()})
        return t, lines

    for _ in range(5):
        assert fn(*args) == 0, H.last_error()
    replayed = w.graph_counters()[2] > 0  # the per-message hipMemcpyAsync landing is never recorded as a graph
    if replayed:
        print("graph replay, trace off: %8.2f us per call (host wall clock, 50 calls)" % wall(50))
        t, lines = traced(50)
        spans = list(zip(lines["other"][0::2], lines["other"][1::2]))
        launch, wait = spans[0::2], spans[1::2]
        print("graph replay, trace on:  %8.2f us per call; per call, medians of %d replays:" % (t, len(lines["device-graph"]) // 2))
        print("    host, inside hipGraphLaunch (with the two timing events the trace adds)  %8.2f us" % (st.median(d for _, d in launch) * 1e3))
        print("    host, spinning on the completion flag                                    %8.2f us" % (st.median(d for _, d in wait) * 1e3))
        print("    device, event before the graph to event after it                         %8.2f us" % (st.median(lines["device-graph"][1::2]) * 1e3))
    else:
        print("this landing mode is not recorded as a graph: every call is issued eagerly")
    w.set_graph_mode(0)
    for _ in range(3):
        assert fn(*args) == 0, H.last_error()
    print("eager issue, trace off:  %8.2f us per call" % wall(30))
    t, lines = traced(30)
    red, cp = lines["device-redu-kernel"][1::2], lines["device-copy-kernel"][1::2]
    per_call_red, per_call_cp = len(red) // 30, len(cp) // 30
    print("eager issue, trace on:   %8.2f us per call; the launches' own durations (each leaves its begin and end timestamps in the trace):" % t)
    print("    %d reduction launches per call: median %.2f us, sum per call %.2f us" % (per_call_red, st.median(red) * 1e3, sum(red) / 30 * 1e3))
    print("    %d copy launches per call:      median %.2f us, sum per call %.2f us" % (per_call_cp, st.median(cp) * 1e3, sum(cp) / 30 * 1e3))
    issue = [lines[k][1::2] for k in ("issue-redu-kernel", "issue-copy-kernel", "issue-send", "received", "issue-recv", "reduced", "other")]
    print("    host time per call in the trace's categories (us): issue-redu-kernel %.1f, issue-copy-kernel %.1f, issue-send %.1f, "
          "received %.1f, issue-recv %.1f, reduced %.1f, other %.1f" % tuple(sum(v) / 30 * 1e3 for v in issue))
    w.set_graph_mode(1)


def same_bits(torch, got, want, what, chunk_elems):
    """Bit-exact comparison of two device tensors; a mismatch is described on stderr (how many elements, where)."""
    bad = got.view(torch.int32) != want.view(torch.int32)
    count = int(bad.sum())
    if count == 0:
        return True
    where = bad.nonzero().flatten()
    first, last = int(where[0]), int(where[-1])
    print("PARITY MISMATCH in %s: %d of %d elements differ, first %d (chunk %d), last %d (chunk %d); got %r want %r" % (
        what, count, got.numel(), first, first // chunk_elems, last, last // chunk_elems, float(got[first]), float(want[first])),
        file=sys.stderr, flush=True)
    return False


def timed(torch, H, call, steps, warm):
    for _ in range(warm):
        assert call() == 0, H.last_error()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        rc = call()
        assert rc == 0, H.last_error()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def device_bytes(s):
    return 12 * s["reduce_elements"] + 2 * s["landing_bytes"] + 2 * s["gather_bytes"]


def in_schedule_leg(torch, H, world, rank, algo, sp, rp, out_ptr, n, landing=None, fuse=None, calls=10):
    """The kernels' own durations inside the rank's schedule.  A world of its own whose ranks issue on ONE stream each and
    eagerly: the rank's launches then follow one another on an in-order stream exactly as the nodes of the recorded graph
    do in a replay, and with the library's trace on every launch leaves its own begin and end timestamps (the dispatch's,
    as a profiler reports them) in the trace's device lines.  -> per-position means over `calls` calls, reductions and
    gathers in the order launched."""
    import tempfile
    base = os.path.join(tempfile.mkdtemp(), "trace")
    saved = {k: os.environ.get(k) for k in ("IBCOMM_TRACE_FILE", "IBCOMM_NUM_CUDA_STREAM")}
    os.environ["IBCOMM_TRACE_FILE"] = base
    os.environ["IBCOMM_NUM_CUDA_STREAM"] = "1"
    try:
        with H.World(world) as w:
            if landing is not None:
                w.set_landing(landing)
            if fuse:
                w.set_max_fuse(fuse)
            w.set_graph_mode(0)
            assert w.record(rank, algo, H.F32, sp, rp, n) == 0, H.last_error()
            for _ in range(2):
                assert w.replay(rank, algo, H.F32, sp[rank], out_ptr, n) == 0, H.last_error()
            w.set_trace(True)
            for _ in range(calls):
                assert w.replay(rank, algo, H.F32, sp[rank], out_ptr, n) == 0, H.last_error()
            w.dump_trace()
            w.set_trace(False)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    lines = {name: [] for name in ("device-redu-kernel", "device-copy-kernel")}
    lines.update({ln.split(",")[0]: [float(x) for x in ln.split(",")[1:-1]] for ln in open("%s_%d.dat" % (base, rank)).read().splitlines()})

    def per_position(durations_ms):
        k = len(durations_ms) // calls
        if k == 0:
            return []
        return [round(sum(durations_ms[c * k + i] for c in range(calls)) / calls * 1e3, 2) for i in range(k)]

    return per_position(lines["device-redu-kernel"][1::2]), per_position(lines["device-copy-kernel"][1::2])


def measure_config(torch, H, O, cfg, args, steps, warm, full):
    """One configuration: the whole world once (recorded, checked), rank 0's schedule replayed and timed, the whole
    world timed, the kernel-landing variant, the roofline legs.  `full` adds the legs only the headline configuration
    carries (hipMemcpyAsync landing, the ceiling).  -> dict of everything measured."""
    algo_name, world, n, chunk, kind = CONFIGS[cfg]
    algo = H.RING if algo_name == "ring" else H.RABENSEIFNER
    os.environ["IBCOMM_CHUNKSIZE"] = str(chunk)
    if cfg == 4:
        os.environ.setdefault("IBCOMM_NUM_CUDA_STREAM", "64")
    landing_name = args.landing or os.environ.get("IBCOMM_HIP_LANDING", "staged")
    rank = 0
    send = make_inputs(torch, world, n, kind, 1234)
    recv = [torch.empty_like(t) for t in send]
    # The library's streams do not synchronise with torch's: the inputs must be complete (and torch's
    # allocator done recycling the generators' temporaries under these very addresses) before it runs.
    torch.cuda.synchronize()
    sp = [t.data_ptr() for t in send]
    rp = [t.data_ptr() for t in recv]
    res = {"cfg": cfg, "algo_name": algo_name, "world": world, "n": n, "chunk": chunk, "rank": rank, "landing": landing_name}

    w = H.World(world)
    keep_open = False
    try:
        if args.landing:
            w.set_landing({"memcpy": H.LAND_MEMCPY, "kernel": H.LAND_KERNEL, "direct": H.LAND_DIRECT, "staged": H.LAND_STAGED}[args.landing])
        if args.fuse:
            w.set_max_fuse(args.fuse)
        if args.no_graph:
            w.set_graph_mode(0)

        # 1. the whole world once, eagerly, recording what `rank` receives; its counters give the per-step work
        w.reset_stats()
        assert w.record(rank, algo, H.F32, sp, rp, n) == 0, H.last_error()
        torch.cuda.synchronize()
        st = [w.stats(r) for r in range(world)]
        parity = check_result(torch, O, H, algo, send, recv, chunk)
        if not parity:
            print("PARITY MISMATCH in config %d: the whole world's result differs from the oracle / from torch's adds in the reference's order" % cfg,
                  file=sys.stderr, flush=True)

        # 2. THE TIMED STEP: `rank`'s complete schedule on its own, peers replaced by the recording
        out = torch.empty_like(send[rank])
        torch.cuda.synchronize()
        w.reset_stats()
        assert w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n) == 0, H.last_error()
        st_rank = w.stats(rank)
        # Shape of the dominant reduction launch of the rank, as the engine issued it: one ring step
        # reduces one chunk group, the first Rabenseifner halving step half of all groups; chunks that
        # follow one another in all three operands share a kernel segment.
        leg_segments = max(1, st_rank["largest_reduce_kernel_segments"])
        seg_elems = st_rank["largest_reduce_elements"] // leg_segments
        # Where that launch's result goes in the schedule: into the pool slots the rank stages partial sums in,
        # a working set of `slots_high_water` chunks (taken from the full-world run).  If launches of the dominant
        # shape follow one another within a call (every ring step), their results cycle through that working set,
        # and the leg's results do the same.  If the shape occurs once per call (the first halving step), everything
        # else the rank writes in a call lies between two of its launches, and the leg's results cycle through a
        # region of that size instead: the distance after which a location is written again is what decides
        # whether the 256 MB memory-side cache still holds it.
        staging_elems = max(s["slots_high_water"] for s in st) * (chunk // 4)
        written_per_call = st_rank["reduce_elements"] + st_rank["gather_bytes"] // 4 + st_rank["landing_bytes"] // 4
        if st_rank["largest_reduce_launches"] < 2:
            staging_elems = max(staging_elems, written_per_call)
        staging = torch.empty(max(staging_elems, seg_elems * leg_segments), device="cuda")
        res.update(send=send, recv=recv, staging=staging, seg_elems=seg_elems, leg_segments=leg_segments, st=st, st_rank=st_rank, w=w,
                   algo=algo, sp=sp, rp=rp, out=out)
        if args.call_breakdown or args.sweep or args.ceiling or args.only_roofline:
            keep_open = True
            return res  # the caller runs its leg inside this world, then closes it

        # the C entry point with its arguments converted once, as any caller in a loop would hold them
        replay_fn = H.lib().ibcomm_hip_replay_allreduce
        replay_args = (w.comms[rank], C.c_int(algo), C.c_int(H.F32), C.c_void_p(sp[rank]), C.c_void_p(out.data_ptr()), C.c_size_t(n))
        res["sec_per_step"] = timed(torch, H, lambda: replay_fn(*replay_args), steps, warm)
        parity = same_bits(torch, out, recv[rank], "config %d, rank schedule replayed" % cfg, chunk // 4) and parity

        # ... and the device's own time for one replay: HIP events before and after the graph, from the library's trace
        if not args.no_graph:
            import tempfile
            base = os.path.join(tempfile.mkdtemp(), "replay")
            saved_base = os.environ.get("IBCOMM_TRACE_FILE")
            os.environ["IBCOMM_TRACE_FILE"] = base
            w.set_trace(True)
            for _ in range(20):
                assert replay_fn(*replay_args) == 0, H.last_error()
            w.dump_trace()
            w.set_trace(False)
            if saved_base is None:
                os.environ.pop("IBCOMM_TRACE_FILE", None)
            else:
                os.environ["IBCOMM_TRACE_FILE"] = saved_base
            spans = [ln for ln in open("%s_%d.dat" % (base, rank)).read().splitlines() if ln.startswith("device-graph,")]
            durations = sorted(float(x) for x in spans[0].split(",")[1:-1][1::2]) if spans else []
            if durations:
                res["replay_device_us"] = round(durations[len(durations) // 2] * 1e3, 2)

        # 3. for reference: all ranks' schedules executed on the one GPU per step
        res["world_sec"] = timed(torch, H, lambda: w.allreduce_ptrs(algo, H.F32, sp, rp, n), steps, warm)
        res["graph_counters"] = w.graph_counters()

        # 4. the kernels' own durations inside the schedule (a one-stream world of its own, eager issue, traced)
        if not args.no_graph:
            out.fill_(0)
            torch.cuda.synchronize()
            landing_code = {"memcpy": H.LAND_MEMCPY, "kernel": H.LAND_KERNEL, "direct": H.LAND_DIRECT, "staged": H.LAND_STAGED}[landing_name]
            res["in_schedule_reduce_us"], res["in_schedule_copy_us"] = in_schedule_leg(torch, H, world, rank, algo, sp, rp, out.data_ptr(), n,
                                                                                       landing_code, args.fuse)
            parity = same_bits(torch, out, recv[rank], "config %d, rank schedule issued eagerly on one stream with the trace on" % cfg, chunk // 4) and parity

        # 5. for reference: the same single-rank schedule when every message is first copied into a pool
        #    slot of the receiver by a copy kernel ("kernel" landing), unless that is the mode already measured
        res["copied"] = None
        if landing_name != "kernel":
            w.set_landing(H.LAND_KERNEL)
            out.fill_(0)
            torch.cuda.synchronize()
            copied_sec = timed(torch, H, lambda: w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n), steps, warm)
            copied_ok = same_bits(torch, out, recv[rank], "config %d, kernel landing" % cfg, chunk // 4)
            parity = parity and copied_ok
            res["copied"] = {"ms_per_step": round(copied_sec * 1e3, 4), "algbw_GBps": round(n * 4 / copied_sec * 1e-9, 2),
                             "parity_bit_exact": copied_ok}

        # 6. and the most literal form: every message lands in a pool slot through hipMemcpyAsync
        #    (always issued eagerly), unless that is the mode already measured
        res["memcpy_landing"] = None
        if full and landing_name != "memcpy":
            w.set_landing(H.LAND_MEMCPY)
            out.fill_(0)
            torch.cuda.synchronize()
            w.reset_stats()
            m_sec = timed(torch, H, lambda: w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n), min(steps, 10), 2)
            calls = w.stats(rank)["calls"]
            copies = (w.stats(rank)["landing_copies"] + w.stats(rank)["gather_copies"]) // max(1, calls)
            m_ok = same_bits(torch, out, recv[rank], "config %d, hipMemcpyAsync landing" % cfg, chunk // 4)
            parity = parity and m_ok
            res["memcpy_landing"] = {"ms_per_step": round(m_sec * 1e3, 4), "algbw_GBps": round(n * 4 / m_sec * 1e-9, 2),
                                     "hipMemcpyAsync_calls_per_step": copies, "parity_bit_exact": m_ok}
    finally:
        if not keep_open:
            w.close()
            res["w"] = None
    res["parity"] = parity

    # 7. the dominant kernel at its in-schedule launch shape
    if not args.no_roofline:
        leg = roofline_leg(torch, H, send, recv, seg_elems, leg_segments, 200, staging)
        # the same launches with the result walking through all ranks' recvbufs instead (2 GiB and more): what
        # the one reduction per schedule whose result stays in recvbuf sees
        far = roofline_leg(torch, H, send, recv, seg_elems, leg_segments, 200)
        leg["result_walking_through_all_recvbufs"] = {k: far[k] for k in ("avg_launch_us", "achieved", "frac")}
        if "in_schedule_reduce_us" in res and res["in_schedule_reduce_us"]:
            # mean over the rank's reduction launches of the dominant shape, as they ran inside the schedule
            dominant = [u for u in res["in_schedule_reduce_us"]]
            mean_us = sum(dominant) / len(dominant)
            alg = 12.0 * st_rank["reduce_elements"] / len(dominant)
            leg["in_schedule_what"] = ("each launch's own begin-to-end time (the dispatch's timestamps) with rank 0's schedule issued eagerly on one in-order "
                                       "stream, in the order a graph replay runs the same launches, the library's trace on, mean over 10 calls per position; "
                                       "the host issues slower than the device runs, so every launch finds the device idle: a launch on its own, without the "
                                       "kernel boundary that a chain adds (`roofline.avg_launch_us` is back to back and contains it)")
            leg["in_schedule_reduce_launches_us"] = res["in_schedule_reduce_us"]
            leg["in_schedule_mean_us"] = round(mean_us, 2)
            leg["in_schedule_frac"] = round(alg / (mean_us * 1e-6) * 1e-9 / HBM_PEAK_GBPS, 4)
            leg["in_schedule_gather_launches_us"] = res["in_schedule_copy_us"]
            if "replay_device_us" in res:
                # one replay of the schedule as one chain of launches on the device, completion node included; what it
                # takes beyond the sum of the launches' own durations is the kernel boundaries of the chain
                own = sum(res["in_schedule_reduce_us"]) + sum(res["in_schedule_copy_us"])
                launches = len(res["in_schedule_reduce_us"]) + len(res["in_schedule_copy_us"])
                leg["replay_device_us_per_call"] = res["replay_device_us"]
                leg["replay_launches_per_call"] = launches
                leg["replay_minus_launches_own_time_us_per_launch"] = round((res["replay_device_us"] - own) / max(1, launches), 2)
        leg["target_0p80_met"] = bool(leg["frac"] >= 0.80)
        if full:
            leg["ceiling"] = ceiling_leg(torch, H, send, recv, seg_elems, leg_segments, leg["avg_launch_us"], staging=staging)
            if args.whole_buffer:
                # the same kernel over one whole per-rank buffer: what it sustains once the launch is large.
                # Not part of the default run, so that a profile of the default run holds the dominant
                # shape only under this kernel's name.
                whole = roofline_leg(torch, H, send, recv, n, 1, 40)
                leg["whole_buffer_launch"] = {k: whole[k] for k in (
                    "launch_shape", "algorithmic_bytes_per_launch", "avg_launch_us", "achieved", "frac", "launches_timed")}
        res["roofline"] = leg
    for k in ("send", "recv", "staging", "out", "sp", "rp"):
        res.pop(k, None)
    del send, recv, staging, out
    torch.cuda.empty_cache()
    return res


def summary_of(res):
    """The figures of one configuration that the measured table is made of."""
    n, world = res["n"], res["world"]
    rank_bytes = device_bytes(res["st_rank"])
    world_bytes = sum(device_bytes(s) for s in res["st"])
    out = {
        "workload": "%s allreduce, %d emulated ranks, %d fp32 per rank, IBCOMM_CHUNKSIZE=%d" % (res["algo_name"], world, n, res["chunk"]),
        "rank_ms_per_step": round(res["sec_per_step"] * 1e3, 4),
        "rank_algbw_GBps": round(n * 4 / res["sec_per_step"] * 1e-9, 2),
        "rank_device_GBps": round(rank_bytes / res["sec_per_step"] * 1e-9, 1),
        "rank_frac_of_hbm_peak": round(rank_bytes / res["sec_per_step"] * 1e-9 / HBM_PEAK_GBPS, 4),
        "world_all_ranks_on_one_gpu_ms_per_step": round(res["world_sec"] * 1e3, 4),
        "world_all_ranks_on_one_gpu_algbw_GBps": round(n * 4 / res["world_sec"] * 1e-9, 2),
        "rank_with_copy_kernel_landing": res["copied"],
        "parity_bit_exact": res["parity"],
    }
    if "roofline" in res:
        leg = res["roofline"]
        out["roofline"] = {k: leg[k] for k in ("launch_shape", "kernel", "algorithmic_bytes_per_launch", "avg_launch_us", "achieved", "frac", "traffic",
                                               "result_walking_through_all_recvbufs", "target_0p80_met") if k in leg}
        for k in ("in_schedule_what", "in_schedule_mean_us", "in_schedule_frac", "in_schedule_reduce_launches_us", "in_schedule_gather_launches_us",
                  "replay_device_us_per_call", "replay_launches_per_call", "replay_minus_launches_own_time_us_per_launch"):
            if k in leg:
                out["roofline"][k] = leg[k]
    return out


def compact_leg(leg, top=True):
    """A roofline leg without its prose: the contract's keys first, then the figures the measured table is made of.
    `frac_into_recvbufs`: the same launches with the result walking through all recvbufs instead of the staging region;
    `in_schedule_mean_us` / `_frac`: mean of the reduction launches' own begin-to-end times, issued one at a time in the
    schedule's order (a replayed chain adds a kernel boundary per launch); `replay_device_us`: one replay of the rank's
    schedule on the device, HIP events around the graph."""
    out = {k: leg[k] for k in (("bound", "achieved", "peak", "unit", "frac", "traffic") if top else ("frac", "traffic")) if k in leg}
    out["launch_shape"] = leg["launch_shape"]
    if top:
        out["algorithmic_bytes_per_launch"] = leg["algorithmic_bytes_per_launch"]
    out["avg_launch_us"] = leg["avg_launch_us"]
    out["target_0p80_met"] = leg.get("target_0p80_met")
    out["frac_into_recvbufs"] = leg["result_walking_through_all_recvbufs"]["frac"]
    for k, short in (("in_schedule_mean_us", "in_schedule_mean_us"), ("in_schedule_frac", "in_schedule_frac"), ("replay_device_us_per_call", "replay_device_us")):
        if k in leg:
            out[short] = leg[k]
    if top and "in_schedule_mean_us" in leg:
        out["in_schedule_is"] = "each launch's own time, issued alone in schedule order; a chain adds a kernel boundary"
    return out


def compact_line(full):
    """The line that is printed by default: every figure, little prose.  (The driver that runs this benchmark keeps
    only the end of its output, a few thousand characters; --full prints everything, with descriptions.)"""
    full = dict(full)
    full["metric"] = "emulated allreduce algbw, fp32 (+ reduce-kernel HBM roofline)"
    line = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                                 "vs_baseline", "dtype", "data")}
    c = full["config"]
    line["config"] = {"workload": "BASELINE configs[%d]: %s, %d emulated ranks x %d fp32, IBCOMM_CHUNKSIZE=%d; step = rank %d's complete schedule "
                                  "on the GPU, peers replayed from a recording of the full world" % (
                                      full["_config_id"] - 1, c["algo"], c["ranks"], c["elements_per_rank"], c["chunk_bytes"], c["measured_rank"]),
                      "landing": c["landing"], "max_fuse": c["max_fuse"]}
    line["parity_bit_exact"] = full["parity_bit_exact"]  # every configuration and landing mode of the run
    e = full["extra"]

    def landing(d):
        return None if d is None else {k: d[k] for k in d if k != "parity_bit_exact"}

    x = {"busbw_GBps": e["busbw_GBps"], "rank_device_GBps": e["rank_device_GBps"], "rank_frac_of_hbm_peak": e["rank_frac_of_hbm_peak"],
         "rank_launches_per_step": e["rank_reduce_launches_per_step"] + e["rank_gather_launches_per_step"] + e["rank_landing_launches_per_step"],
         "world_all_ranks_on_one_gpu": {k: e["world_all_ranks_on_one_gpu"][k] for k in ("ms_per_step", "algbw_GBps", "frac_of_hbm_peak")},
         "rank_with_copy_kernel_landing": landing(e["rank_with_copy_kernel_landing"]),
         "rank_with_hipMemcpyAsync_landing": landing(e["rank_with_hipMemcpyAsync_landing"]),
         "issue": e["issue"], "graph_calls_eager_captured_replayed": e["graph_calls_eager_captured_replayed"],
         "pool_slots_high_water": e["pool_slots_high_water"]}
    if "other_configs" in e:
        x["other_configs"] = {}
        for name, o in e["other_configs"].items():
            y = {"workload": o["workload"].replace(" allreduce, ", " ").replace(" emulated ranks, ", " x ").replace(" per rank, IBCOMM_CHUNKSIZE=", ", chunk "),
                 "rank_ms_per_step": o["rank_ms_per_step"], "rank_algbw_GBps": o["rank_algbw_GBps"],
                 "rank_frac_of_hbm_peak": o["rank_frac_of_hbm_peak"], "world_ms_per_step": o["world_all_ranks_on_one_gpu_ms_per_step"],
                 "world_algbw_GBps": o["world_all_ranks_on_one_gpu_algbw_GBps"],
                 "kernel_landing_rank_algbw_GBps": (o["rank_with_copy_kernel_landing"] or {}).get("algbw_GBps")}
            if "roofline" in o:
                y["roofline"] = compact_leg(o["roofline"], top=False)
            x["other_configs"][name] = y
    if "reference_api" in e:
        x["reference_api"] = {"what": "8 rank threads in blocking IBVerbsCommunicator::AllreduceRingCuda<float> calls; 3 warm-ups, 10 timed; ms per allreduce"}
        for name, o in e["reference_api"].items():
            x["reference_api"][name] = o if "error" in o else {"first_timed_call": o["ms_per_allreduce_first_timed_call"], "median": o["ms_per_allreduce_median"],
                                                               "max": o["ms_per_allreduce_max"], "all_ranks_ok": o["all_ranks_report_ok"]}
    line["extra"] = x
    if "roofline" in full:
        r = full["roofline"]
        leg = compact_leg(r)
        leg["kernel"] = r["kernel"]
        if "ceiling" in r:
            leg["ceiling"] = {"best_of_57_other_forms_us": r["ceiling"]["best_variant_us"], "shipped_us_same_pass": r["ceiling"]["shipped_kernel_us_same_pass"],
                              "shipped_over_best": r["ceiling"]["shipped_over_best"]}
        if "whole_buffer_launch" in r:
            leg["whole_buffer_launch"] = r["whole_buffer_launch"]
        line["roofline"] = leg
    if "cpu_baseline" in full:
        b = full["cpu_baseline"]
        line["cpu_baseline"] = {"value": b["value"], "unit": b["unit"], "cores": b["cores"], "kind": b["kind"],
                                "sample": "same workload, whole; the oracle's restatement of AllreduceRing<float>, gcc -O2 scalar loop, one thread per rank, best of 15",
                                "seconds": b["seconds"], "cpu_model": b["cpu_model"], "logical_cpus": b["logical_cpus"],
                                "single_core_reduce_loop_GBps": b["single_core_reduce_loop_GBps"],
                                "config1_ring_4x16MiB": {k: b["config1_ring_4x16MiB"][k] for k in ("seconds", "algbw_GBps", "equals_exact_integer_sum")}}
    return line


def reference_api_leg(cfg, timed_runs=10):
    """The reference's own entry point and timing protocol: one IBVerbsCommunicator per rank, one host thread per rank,
    every rank in a blocking AllreduceRingCuda / AllreduceRabenseifnerCuda call; 3 warm-ups, then timed runs
    (examples/allreduce.cpp:28-29, 107-118, which times one).  Runs the example program built against the drop-in
    header in a process of its own."""
    import subprocess
    algo_name, world, n, chunk, _ = CONFIGS[cfg]
    exe = os.path.join(ROOT, "allreduce-proto_amd", "allreduce_example")
    if not os.path.exists(exe):
        return {"error": "%s is not built" % exe}
    env = dict(os.environ, IBCOMM_CHUNKSIZE=str(chunk))
    if cfg == 4:
        env.setdefault("IBCOMM_NUM_CUDA_STREAM", "64")
    p = subprocess.run([exe, str(world), algo_name, str(n), str(timed_runs)], env=env, capture_output=True, text=True, timeout=600)
    first, runs = None, []
    for ln in p.stdout.splitlines():
        if ln.startswith("elapsed time :"):
            first = float(ln.split(":")[1].split()[0])
        if ln.startswith("elapsed times of"):
            runs = [float(x) for x in ln.split(":")[1].split()]
    if p.returncode != 0 or first is None:
        return {"error": "exit status %d: %s" % (p.returncode, (p.stdout + p.stderr)[-300:])}
    runs = runs or [first]
    return {
        "workload": "%s, %d rank threads x %d fp32, IBCOMM_CHUNKSIZE=%d, integer-valued inputs as in the reference's example" % (algo_name, world, n, chunk),
        "entry_point": "IBVerbsCommunicator::Allreduce%sCuda<float>, one blocking call per rank thread" % ("Ring" if algo_name == "ring" else "Rabenseifner"),
        "protocol": "3 warm-ups, then %d timed calls; rank 0's wall clock around its own call" % len(runs),
        "ms_per_allreduce_first_timed_call": round(first * 1e3, 4),
        "ms_per_allreduce_median": round(sorted(runs)[len(runs) // 2] * 1e3, 4),
        "ms_per_allreduce_max": round(max(runs) * 1e3, 4),
        "algbw_GBps_median": round(n * 4 / sorted(runs)[len(runs) // 2] * 1e-9, 2),
        "all_ranks_report_ok": p.stdout.count(" OK") == world,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2, choices=sorted(CONFIGS))
    ap.add_argument("--landing", choices=["memcpy", "kernel", "direct", "staged"], default=None)
    ap.add_argument("--fuse", type=int, default=None)
    ap.add_argument("--no-graph", action="store_true", help="issue every step eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-roofline", action="store_true", help="skip the kernel roofline leg")
    ap.add_argument("--no-others", action="store_true",
                    help="skip extra.other_configs (configurations 4 and 3 measured after the headline one) and extra.reference_api")
    ap.add_argument("--full", action="store_true", help="print the line with every detail and description (several times longer)")
    ap.add_argument("--all-configs", action="store_true", help="extra.other_configs also holds configuration 5 (32 ranks x 2 GiB)")
    ap.add_argument("--only-roofline", action="store_true",
                    help="run only the kernel roofline leg at the workload's launch shape (for profiling the kernel alone)")
    ap.add_argument("--leg-shape", default=None, metavar="SEGMENTS,ELEMENTS,STAGING_ELEMENTS",
                    help="with --only-roofline: time exactly this launch shape (as printed by a plain --only-roofline run as "
                         "`leg_shape`) without running the collective first, so that a profile of the command holds the leg's launches only")
    ap.add_argument("--whole-buffer", action="store_true",
                    help="also time the reduction kernel over one whole per-rank buffer in a single segment "
                         "(roofline.whole_buffer_launch): what it sustains once a launch is large")
    ap.add_argument("--sweep", action="store_true",
                    help="time every kernel variant of the measurement library, adds and copies, at the workload's launch shape")
    ap.add_argument("--ceiling", action="store_true",
                    help="the best variant at the launch shape, the shipped kernel on a whole-buffer launch, and hipMemcpyAsync")
    ap.add_argument("--call-breakdown", action="store_true",
                    help="run the rank's schedule with the library's trace on, eagerly and as graph replays, and print host spans "
                         "and device durations per call")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py measures one GPU only: every emulated rank lives on the same MI355X and nothing in this build "
              "uses a second device; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py is a single-process, single-GPU benchmark; do not launch it under torchrun", file=sys.stderr)
        sys.exit(2)

    import torch
    import hip_lib as H
    import oracle_lib as O

    algo_name, world, n, chunk, kind = CONFIGS[args.config]
    torch.cuda.set_device(0)
    warm = max(args.warmup, 0 if args.no_graph else 2)  # the call shape is recorded on its second use

    if args.only_roofline and args.leg_shape:
        os.environ["IBCOMM_CHUNKSIZE"] = str(chunk)
        send = make_inputs(torch, world, n, kind, 1234)
        recv = [torch.empty_like(t) for t in send]
        k, elems, staging_elems = (int(x) for x in args.leg_shape.split(","))
        staging = torch.empty(max(staging_elems, k * elems), device="cuda")
        for _ in range(3):  # the copies of known size that calibrate hardware counters (see below)
            recv[0].copy_(send[0])
        torch.cuda.synchronize()
        print(json.dumps({"only_roofline": True, "config": args.config, "leg_shape": args.leg_shape,
                          "roofline": roofline_leg(torch, H, send, recv, elems, k, 200, staging)}))
        return

    res = measure_config(torch, H, O, args.config, args, args.steps, warm, full=True)
    if args.call_breakdown or args.sweep or args.ceiling or args.only_roofline:
        # legs that run inside the world measure_config left open
        w, send, recv, staging = res["w"], res["send"], res["recv"], res["staging"]
        seg_elems, leg_segments, rank = res["seg_elems"], res["leg_segments"], res["rank"]
        try:
            if args.call_breakdown:
                call_breakdown(torch, H, w, rank, res["algo"], res["sp"][rank], res["out"].data_ptr(), n)
            total = seg_elems * leg_segments
            if args.sweep:
                print_variant_table("dst = a + b, %d fp32 in one segment (12 B per element)" % total,
                                    variant_times(torch, H, send, recv, total, True, staging=staging), 12.0 * total)
                print()
                print_variant_table("dst = a (the gather and landing copies), %d fp32 in one segment (8 B per element)" % total,
                                    variant_times(torch, H, send, recv, total, False), 8.0 * total)
            if args.ceiling:
                leg = roofline_leg(torch, H, send, recv, seg_elems, leg_segments, 200, staging)
                print(json.dumps({"config": args.config, "roofline": leg,
                                  "ceiling": ceiling_leg(torch, H, send, recv, seg_elems, leg_segments, leg["avg_launch_us"], full=True,
                                                         staging=staging)}))
            if args.only_roofline:
                # a plain device copy of known size (n * 4 bytes read, n * 4 written), so that hardware
                # counters collected over this command can be calibrated against a known traffic
                for _ in range(3):
                    recv[0].copy_(send[0])
                torch.cuda.synchronize()
                print(json.dumps({"only_roofline": True, "config": args.config,
                                  "leg_shape": "%d,%d,%d" % (leg_segments, seg_elems, staging.numel()),
                                  "roofline": roofline_leg(torch, H, send, recv, seg_elems, leg_segments, 200, staging)}))
        finally:
            w.close()
        return

    st, st_rank, rank = res["st"], res["st_rank"], res["rank"]
    sec_per_step, world_sec = res["sec_per_step"], res["world_sec"]
    parity = res["parity"]
    rank_bytes = device_bytes(st_rank)
    world_bytes = sum(device_bytes(s) for s in st)
    chunks_per_launch = round(st_rank["reduce_segments"] / max(1, st_rank["reduce_launches"]), 2)
    segs_per_launch = round(st_rank["reduce_kernel_segments"] / max(1, st_rank["reduce_launches"]), 2)
    graph_counters = res["graph_counters"]

    algbw = n * 4 / sec_per_step * 1e-9
    world_algbw = n * 4 / world_sec * 1e-9
    line = {
        "metric": "emulated allreduce algbw (GB/s) with reduce-kernel HBM roofline, fp32",
        "value": round(algbw, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": warm,
        "ms_per_step": round(sec_per_step * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[%d]: %s allreduce, %d emulated ranks, %d fp32 (%.0f MiB) per rank, IBCOMM_CHUNKSIZE=%d; "
                        "one step = rank %d's complete schedule on the GPU (its reductions and gathers, plus landing copies in the modes that make them), the "
                        "other ranks' messages replayed from a recording of the full world" % (
                            args.config - 1, algo_name, world, n, n * 4 / 2**20, chunk, rank),
            "algo": algo_name, "ranks": world, "elements_per_rank": n, "chunk_bytes": chunk, "measured_rank": rank,
            "landing": res["landing"],
            "max_fuse": args.fuse or int(os.environ.get("IBCOMM_HIP_MAX_FUSE", "64")),
        },
        "parity_bit_exact": parity,
        "extra": {
            "busbw_GBps": round(algbw * 2 * (world - 1) / world, 2),
            "rank_device_traffic_GB_per_step": round(rank_bytes * 1e-9, 3),
            "rank_device_GBps": round(rank_bytes / sec_per_step * 1e-9, 1),
            "rank_frac_of_hbm_peak": round(rank_bytes / sec_per_step * 1e-9 / HBM_PEAK_GBPS, 4),
            "rank_reduce_launches_per_step": st_rank["reduce_launches"],
            "rank_mean_chunks_per_launch": chunks_per_launch,
            "rank_mean_kernel_segments_per_launch": segs_per_launch,
            "rank_reduce_elements_per_step": st_rank["reduce_elements"],
            "rank_landing_launches_per_step": st_rank["landing_copies"],
            "rank_gather_launches_per_step": st_rank["gather_copies"],
            "world_all_ranks_on_one_gpu": {
                "ms_per_step": round(world_sec * 1e3, 4),
                "algbw_GBps": round(world_algbw, 2),
                "device_traffic_GB_per_step": round(world_bytes * 1e-9, 3),
                "device_GBps": round(world_bytes / world_sec * 1e-9, 1),
                "frac_of_hbm_peak": round(world_bytes / world_sec * 1e-9 / HBM_PEAK_GBPS, 4),
            },
            "rank_with_copy_kernel_landing": res["copied"],
            "rank_with_hipMemcpyAsync_landing": res["memcpy_landing"],
            "north_star_landing_mode": "memcpy (rank_with_hipMemcpyAsync_landing is that mode's figure; `value` is the '%s' mode)" % res["landing"],
            "streams_per_rank": st[0]["streams_created"],
            "issue": "hip graph replay" if graph_counters[2] > 0 else "eager",
            "graph_calls_eager_captured_replayed": list(graph_counters),
            "pool_slots_high_water": max(s["slots_high_water"] for s in st),
        },
    }
    if "roofline" in res:
        line["roofline"] = res["roofline"]
    if not args.no_others:
        # the other configurations, each to the same parity check, and the reference's own blocking per-rank entry point
        others = {}
        for cfg in [c for c in (4, 3) + ((5,) if args.all_configs else ()) if c != args.config]:
            r = measure_config(torch, H, O, cfg, args, args.steps, warm, full=False)
            others["config_%d" % cfg] = summary_of(r)
            parity = parity and r["parity"]
        line["extra"]["other_configs"] = others
        line["extra"]["reference_api"] = {"config_%d" % cfg: reference_api_leg(cfg) for cfg in (2, 4)}
        line["parity_bit_exact"] = parity
    if not args.no_cpu:
        torch.cuda.empty_cache()
        line["cpu_baseline"] = cpu_baseline_leg(O, world, n, chunk, algo_name)
        # the like-for-like GPU figure for that baseline: all N ranks' schedules on the one GPU per step
        line["cpu_baseline"]["gpu_all_ranks_on_one_gpu_algbw_GBps"] = round(world_algbw, 2)
    line["_config_id"] = args.config
    out = line if args.full else compact_line(line)
    out.pop("_config_id", None)
    print(json.dumps(out, separators=(",", ":")) if not args.full else json.dumps(out))
    if not parity:
        sys.exit(1)


if __name__ == "__main__":
    main()
