#!/usr/bin/env python3
"""Benchmark of the MI355X allreduce hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|3|4|5]
    python bench.py --only-roofline [--config N]     the kernel leg alone (what the counter profiles run)
    python bench.py --whole-buffer                    adds roofline.whole_buffer_launch to the line
    python bench.py --sweep [--config N]              the kernel leg per kernel variant and launch setting

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
    "1 segments x 8388608 fp32": 100681210,     # config 2, profiles/segment_kernel_add_ring8_256MiB.md
    "2 segments x 25165824 fp32": 603978883,    # config 3, profiles/segment_kernel_add_traffic_rabenseifner16_ring8_64KiB_ring32_2GiB.md
    "1 segments x 2097152 fp32": 25180425,      # config 4, same file
    "1 segments x 16777216 fp32": 201346522,    # config 5, same file
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


def roofline_leg(torch, H, send, recv, seg_elems, segs_per_launch, launches):
    """Average duration of the dominant kernel at its in-schedule launch shape, HIP events on its own stream."""
    world = len(send)
    stream = torch.cuda.Stream()
    k = segs_per_launch
    vp = C.c_void_p
    n = send[0].numel()
    per_buf = max(1, n // seg_elems)
    # Every operand of every segment is a distinct range, and successive launches walk through
    # all ranks' buffers (several GiB), so nothing is served from a cache: dst and a come from
    # rank r's recvbuf / sendbuf, b from another rank's recvbuf at the same offset.
    shapes = []
    for i in range(world * 2):
        dst, a, b = [], [], []
        for j in range(k):
            idx = (i * k + j)
            r = idx % world
            off = ((idx // world) % per_buf) * seg_elems * 4
            dst.append(recv[r].data_ptr() + off)
            a.append(send[r].data_ptr() + off)
            b.append(recv[(r + world // 2) % world].data_ptr() + off)
        shapes.append(((vp * k)(*dst), (vp * k)(*a), (vp * k)(*b), (C.c_size_t * k)(*([seg_elems] * k))))
    L = H.lib()

    def launch(i):
        d, a, b, ln = shapes[i % len(shapes)]
        rc = L.ibcomm_hip_reduce_segments(H.F32, k, d, a, b, ln, stream.cuda_stream)
        assert rc == 0, H.last_error()

    with torch.cuda.stream(stream):
        for i in range(5):
            launch(i)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(launches):
            launch(i)
        e1.record(stream)
    e1.synchronize()
    avg_s = e0.elapsed_time(e1) * 1e-3 / launches
    algorithmic = 12.0 * seg_elems * k
    return {
        "bound": "hbm",
        "achieved": round(algorithmic / avg_s * 1e-9, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(algorithmic / avg_s * 1e-9 / HBM_PEAK_GBPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get("%d segments x %d fp32" % (k, seg_elems)),
        "kernel": "ibcomm_hip::AlignedSegmentKernel<float, float4, threads and tile order by launch size, nontemporal, add>",
        "launch_shape": "%d segments x %d fp32" % (k, seg_elems),
        "algorithmic_bytes_per_launch": int(algorithmic),
        "avg_launch_us": round(avg_s * 1e6, 2),
        "launches_timed": launches,
    }


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
    return {
        "value": round(n * 4 / t * 1e-9, 3),
        "unit": "GB/s algbw",
        "cores": min(world, os.cpu_count() or 1),
        "kind": "port",
        "sample": "%s, %d ranks x %d fp32, IBCOMM_CHUNKSIZE=%s, whole workload, best of 15 after 1 warm-up, "
                  "one host thread per emulated rank on %d logical CPUs" % (algo_name, world, n, chunk, os.cpu_count() or 1),
        "seconds": round(t, 3),
        "seconds_median": round(sorted(times)[len(times) // 2], 3),
        "single_core_reduce_loop_GBps": round(12.0 * single_n / single * 1e-9, 2),
        "config1_ring_4x16MiB": {"seconds": round(t_cfg1, 4), "algbw_GBps": round(n1 * 4 / t_cfg1 * 1e-9, 3), "threads": 4,
                                 "protocol": "3 warm-ups + 1 timed run", "equals_exact_integer_sum": cfg1_ok},
    }


SWEEP = [
    # (label, environment of the child).  Any tuning variable routes the launch to the general kernel.
    ("aligned kernel (default)", {}),
    ("general kernel, 256 threads x 1 vector", {"IBCOMM_HIP_NO_ALIGNED_KERNEL": "1"}),
    ("general, 256 x 2", {"IBCOMM_HIP_UNROLL": "2"}),
    ("general, 256 x 4", {"IBCOMM_HIP_UNROLL": "4"}),
    ("general, 1024 x 1", {"IBCOMM_HIP_THREADS": "1024"}),
    ("general, 1024 x 2", {"IBCOMM_HIP_THREADS": "1024", "IBCOMM_HIP_UNROLL": "2"}),
    ("general, 256 x 1, at most 2048 workgroups (grid-stride)", {"IBCOMM_HIP_MAX_BLOCKS": "2048"}),
    ("general, 256 x 2, at most 2048 workgroups", {"IBCOMM_HIP_MAX_BLOCKS": "2048", "IBCOMM_HIP_UNROLL": "2"}),
    ("general, 256 x 4, at most 1024 workgroups", {"IBCOMM_HIP_MAX_BLOCKS": "1024", "IBCOMM_HIP_UNROLL": "4"}),
    ("aligned, 256 threads, plain tile order", {"IBCOMM_HIP_XCD_RUN_MAX_BLOCKS": "0", "IBCOMM_HIP_WG128_MIN_BLOCKS": "2000000000"}),
    ("aligned, 256 threads, die-local tile order", {"IBCOMM_HIP_XCD_RUN_MAX_BLOCKS": "2000000000", "IBCOMM_HIP_WG128_MIN_BLOCKS": "2000000000"}),
    ("aligned, 128 threads, plain tile order", {"IBCOMM_HIP_XCD_RUN_MAX_BLOCKS": "0", "IBCOMM_HIP_WG128_MIN_BLOCKS": "0"}),
    ("aligned, 128 threads, die-local tile order", {"IBCOMM_HIP_XCD_RUN_MAX_BLOCKS": "2000000000", "IBCOMM_HIP_WG128_MIN_BLOCKS": "0"}),
    ("aligned, ordinary loads and stores", {"IBCOMM_HIP_NONTEMPORAL": "0"}),
    ("aligned, non-temporal loads only", {"IBCOMM_HIP_NONTEMPORAL": "3"}),
    ("aligned, non-temporal stores only", {"IBCOMM_HIP_NONTEMPORAL": "4"}),
]


def sweep(config):
    """One child process per variant; nothing here touches the GPU itself."""
    import subprocess
    print("%-58s %-28s %10s %10s %8s" % ("variant", "launch shape", "us/launch", "GB/s", "of peak"))
    for label, env in SWEEP:
        child = subprocess.run([sys.executable, os.path.abspath(__file__), "--only-roofline", "--config", str(config)],
                               env={**os.environ, **env}, capture_output=True, text=True)
        lines = [ln for ln in child.stdout.splitlines() if ln.startswith("{")]
        if child.returncode != 0 or not lines:
            print("%-58s failed (exit %d): %s" % (label, child.returncode, child.stderr.strip().splitlines()[-1:] or ""))
            continue
        r = json.loads(lines[-1])["roofline"]
        print("%-58s %-28s %10.2f %10.1f %8.4f" % (label, r["launch_shape"], r["avg_launch_us"], r["achieved"], r["frac"]), flush=True)


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
    ap.add_argument("--only-roofline", action="store_true",
                    help="run only the kernel roofline leg at the workload's launch shape (for profiling the kernel alone)")
    ap.add_argument("--whole-buffer", action="store_true",
                    help="also time the reduction kernel over one whole per-rank buffer in a single segment "
                         "(roofline.whole_buffer_launch): what it sustains once a launch is large")
    ap.add_argument("--sweep", action="store_true",
                    help="run the roofline leg once per kernel variant and launch setting (each in a child process, "
                         "because the library reads its tuning variables once) and print one line per variant")
    args = ap.parse_args()

    if args.sweep:
        sweep(args.config)
        return
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
    algo = H.RING if algo_name == "ring" else H.RABENSEIFNER
    torch.cuda.set_device(0)
    os.environ["IBCOMM_CHUNKSIZE"] = str(chunk)
    if args.config == 4:
        os.environ.setdefault("IBCOMM_NUM_CUDA_STREAM", "64")

    send = make_inputs(torch, world, n, kind, 1234)
    recv = [torch.empty_like(t) for t in send]
    sp = [t.data_ptr() for t in send]
    rp = [t.data_ptr() for t in recv]

    def timed(call, steps, warm):
        for _ in range(warm):
            assert call() == 0, H.last_error()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            rc = call()
            assert rc == 0, H.last_error()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    rank = 0
    with H.World(world) as w:
        if args.landing:
            w.set_landing({"memcpy": H.LAND_MEMCPY, "kernel": H.LAND_KERNEL, "direct": H.LAND_DIRECT, "staged": H.LAND_STAGED}[args.landing])
        if args.fuse:
            w.set_max_fuse(args.fuse)
        if args.no_graph:
            w.set_graph_mode(0)
        warm = max(args.warmup, 0 if args.no_graph else 2)  # the call shape is recorded on its second use

        # 1. the whole world once, eagerly, recording what `rank` receives; its counters give the per-step work
        w.reset_stats()
        assert w.record(rank, algo, H.F32, sp, rp, n) == 0, H.last_error()
        torch.cuda.synchronize()
        st = [w.stats(r) for r in range(world)]
        parity = check_result(torch, O, H, algo, send, recv, chunk)

        # 2. THE TIMED STEP: `rank`'s complete schedule on its own, peers replaced by the recording
        out = torch.empty_like(send[rank])
        w.reset_stats()
        assert w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n) == 0, H.last_error()
        st_rank = w.stats(rank)
        # Shape of the dominant reduction launch of the rank, as the engine issued it: one ring step
        # reduces one chunk group, the first Rabenseifner halving step half of all groups; chunks that
        # follow one another in all three operands share a kernel segment.
        leg_segments = max(1, st_rank["largest_reduce_kernel_segments"])
        seg_elems = st_rank["largest_reduce_elements"] // leg_segments

        if args.only_roofline:
            # a plain device copy of known size (n * 4 bytes read, n * 4 written), so that hardware
            # counters collected over this command can be calibrated against a known traffic
            for _ in range(3):
                recv[0].copy_(send[0])
            torch.cuda.synchronize()
            print(json.dumps({"only_roofline": True, "config": args.config,
                              "roofline": roofline_leg(torch, H, send, recv, seg_elems, leg_segments, 200)}))
            return
        sec_per_step = timed(lambda: w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n), args.steps, warm)
        parity = parity and bool(torch.equal(out.view(torch.int32), recv[rank].view(torch.int32)))
        del out

        # 3. for reference: all ranks' schedules executed on the one GPU per step
        world_sec = timed(lambda: w.allreduce_ptrs(algo, H.F32, sp, rp, n), args.steps, warm)
        graph_counters = w.graph_counters()

        # 4. for reference: the same single-rank schedule when every message is first copied into a pool
        #    slot of the receiver by a copy kernel ("kernel" landing), unless that is the mode already measured
        copied = None
        if (args.landing or os.environ.get("IBCOMM_HIP_LANDING", "staged")) != "kernel":
            w.set_landing(H.LAND_KERNEL)
            out = torch.empty_like(send[rank])
            copied_sec = timed(lambda: w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n), args.steps, warm)
            copied_ok = bool(torch.equal(out.view(torch.int32), recv[rank].view(torch.int32)))
            parity = parity and copied_ok
            copied = {"ms_per_step": round(copied_sec * 1e3, 4), "algbw_GBps": round(n * 4 / copied_sec * 1e-9, 2),
                      "parity_bit_exact": copied_ok}
            del out

        # 5. and the most literal form: every message lands in a pool slot through its own hipMemcpyAsync
        #    (always issued eagerly), unless that is the mode already measured
        memcpy_landing = None
        if (args.landing or os.environ.get("IBCOMM_HIP_LANDING", "staged")) != "memcpy":
            w.set_landing(H.LAND_MEMCPY)
            out = torch.empty_like(send[rank])
            m_sec = timed(lambda: w.replay(rank, algo, H.F32, sp[rank], out.data_ptr(), n), min(args.steps, 10), 2)
            m_ok = bool(torch.equal(out.view(torch.int32), recv[rank].view(torch.int32)))
            parity = parity and m_ok
            memcpy_landing = {"ms_per_step": round(m_sec * 1e3, 4), "algbw_GBps": round(n * 4 / m_sec * 1e-9, 2),
                              "parity_bit_exact": m_ok}
            del out

    def device_bytes(s):
        return 12 * s["reduce_elements"] + 2 * s["landing_bytes"] + 2 * s["gather_bytes"]

    rank_bytes = device_bytes(st_rank)
    world_bytes = sum(device_bytes(s) for s in st)
    chunks_per_launch = round(st_rank["reduce_segments"] / max(1, st_rank["reduce_launches"]), 2)
    segs_per_launch = round(st_rank["reduce_kernel_segments"] / max(1, st_rank["reduce_launches"]), 2)

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
            "landing": args.landing or os.environ.get("IBCOMM_HIP_LANDING", "staged"),
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
            "rank_with_copy_kernel_landing": copied,
            "rank_with_hipMemcpyAsync_landing": memcpy_landing,
            "streams_per_rank": st[0]["streams_created"],
            "issue": "hip graph replay" if graph_counters[2] > 0 else "eager",
            "graph_calls_eager_captured_replayed": list(graph_counters),
            "pool_slots_high_water": max(s["slots_high_water"] for s in st),
        },
    }
    if not args.no_roofline:
        line["roofline"] = roofline_leg(torch, H, send, recv, seg_elems, leg_segments, 200)
        if args.whole_buffer:
            # the same kernel over one whole per-rank buffer: what it sustains once the launch is large.
            # Not part of the default run, so that a profile of the default run holds the dominant
            # shape only under this kernel's name.
            whole = roofline_leg(torch, H, send, recv, n, 1, 40)
            line["roofline"]["whole_buffer_launch"] = {k: whole[k] for k in (
                "launch_shape", "algorithmic_bytes_per_launch", "avg_launch_us", "achieved", "frac", "launches_timed")}
    del recv
    if not args.no_cpu:
        del send
        torch.cuda.empty_cache()
        line["cpu_baseline"] = cpu_baseline_leg(O, world, n, chunk, algo_name)
    print(json.dumps(line))
    if not parity:
        sys.exit(1)


if __name__ == "__main__":
    main()
