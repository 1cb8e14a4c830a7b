"""ctypes view of tests/support/libibcomm_sim.so: the allreduce engine on a simulated device.

Test infrastructure.  The simulated device records streams/events/copies/launches as a dependency
graph, runs it in random topological order and checks it for unordered conflicting accesses; it
exists so that the engine's host logic is tested on the CPU.  It is not part of the product.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SIM_SO = os.path.join(HERE, "support", "libibcomm_sim.so")


class EngineStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "calls", "reduce_launches", "reduce_segments", "reduce_elements", "landing_copies", "landing_bytes",
        "gather_copies", "gather_bytes", "messages_sent", "messages_received", "events_recorded", "stream_waits",
        "streams_created", "slots_high_water", "slot_count", "pool_blocks", "pool_bytes", "progress_passes", "reduce_kernel_segments",
        "largest_reduce_elements", "largest_reduce_kernel_segments", "largest_reduce_launches")]


class Report(C.Structure):
    _fields_ = [("rc", C.c_int), ("nodes", C.c_long), ("races", C.c_long), ("unrecorded_waits", C.c_long),
                ("rank0", EngineStats), ("error", C.c_char * 512), ("first_race", C.c_char * 256),
                ("launches_collected", C.c_long), ("launches_issued", C.c_long)]


_lib = None


def lib():
    global _lib
    if _lib is None or not hasattr(_lib, 'sim_record_replay'):
        subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "support")])
        _lib = C.CDLL(SIM_SO)
        _lib.sim_world_allreduce.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                             C.c_size_t, C.c_int, C.c_int, C.c_uint, C.c_int, C.c_int, C.POINTER(Report)]
        _lib.sim_record_replay.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                           C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_uint, C.c_void_p, C.c_int,
                                           C.POINTER(Report)]
    return _lib


DT = {np.dtype(np.float32): 0, np.dtype(np.int32): 1, np.dtype(np.float64): 2, np.dtype(np.int64): 3}


def allreduce(algo, sendbufs, chunksize=None, max_fuse=48, landing=0, seed=0, threaded=False, repeats=1,
              pool_bytes=1 << 16, in_place=False, streams=None, copy=True):
    """-> (rc, [recvbuf per rank], Report).  Environment knobs are set for the duration of the call.
    threaded: False = one thread steps all ranks, True (1) = one thread per rank, each with its own engine,
    2 = one thread per rank, the blocking calls meet and the last to arrive steps all ranks, 3 = one thread, all ranks
    on one stream with their launches merged across ranks (a recording of a world)."""
    world = len(sendbufs)
    if copy:  # copy=False: run on the caller's arrays, whatever their alignment
        sendbufs = [np.ascontiguousarray(s).copy() for s in sendbufs]
    n = sendbufs[0].size
    if in_place:
        recv = sendbufs
    else:
        recv = []
        for _ in range(world):
            r = np.empty(n, dtype=sendbufs[0].dtype)
            r.view(np.uint8)[:] = 0x55
            recv.append(r)
    sp = (C.c_void_p * world)(*[s.ctypes.data for s in sendbufs])
    rp = (C.c_void_p * world)(*[r.ctypes.data for r in recv])
    saved = {k: os.environ.get(k) for k in ("IBCOMM_CHUNKSIZE", "IBCOMM_MEMORY_POOL_PRE_ALLOC", "IBCOMM_NUM_CUDA_STREAM")}
    try:
        if chunksize is None:
            os.environ.pop("IBCOMM_CHUNKSIZE", None)
        else:
            os.environ["IBCOMM_CHUNKSIZE"] = str(chunksize)
        os.environ["IBCOMM_MEMORY_POOL_PRE_ALLOC"] = str(pool_bytes)
        if streams is not None:
            os.environ["IBCOMM_NUM_CUDA_STREAM"] = str(streams)
        rep = Report()
        rc = lib().sim_world_allreduce(algo, DT[sendbufs[0].dtype], world, sp, rp, n, max_fuse, landing, seed,
                                       int(threaded), repeats, C.byref(rep))
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    return rc, recv, rep


def record_replay(algo, sendbufs, rank, chunksize=None, max_fuse=64, landing=1, seed=0, replays=1, pool_bytes=1 << 16):
    """World run recording `rank`, then `rank` alone against the recording.
    -> (rc, [world recvbuf per rank], replayed recvbuf of `rank`, Report with that rank's replay stats)"""
    world = len(sendbufs)
    sendbufs = [np.ascontiguousarray(s).copy() for s in sendbufs]
    n = sendbufs[0].size
    recv = []
    for _ in range(world + 1):
        r = np.empty(n, dtype=sendbufs[0].dtype)
        r.view(np.uint8)[:] = 0x55
        recv.append(r)
    out = recv.pop()
    sp = (C.c_void_p * world)(*[s.ctypes.data for s in sendbufs])
    rp = (C.c_void_p * world)(*[r.ctypes.data for r in recv])
    saved = {k: os.environ.get(k) for k in ("IBCOMM_CHUNKSIZE", "IBCOMM_MEMORY_POOL_PRE_ALLOC")}
    try:
        if chunksize is None:
            os.environ.pop("IBCOMM_CHUNKSIZE", None)
        else:
            os.environ["IBCOMM_CHUNKSIZE"] = str(chunksize)
        os.environ["IBCOMM_MEMORY_POOL_PRE_ALLOC"] = str(pool_bytes)
        rep = Report()
        rc = lib().sim_record_replay(algo, DT[sendbufs[0].dtype], world, sp, rp, n, rank, max_fuse, landing, seed,
                                     out.ctypes.data, replays, C.byref(rep))
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    return rc, recv, out, rep
