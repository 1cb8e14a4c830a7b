"""Python binding of libibcomm_hip.so over its C ABI (include/ibcomm_hip.h), via ctypes.

A loopback world of emulated ranks on the current HIP device: World(n) creates the fabric and one
communicator per rank; allreduce_ptrs() drives all ranks from the calling thread, allreduce_threads()
uses one blocking call per rank like the reference's one process per rank.  Buffers are raw device
pointers (e.g. torch.Tensor.data_ptr()).  The library is loaded as built next to this file; if it is
missing this module raises -- there is no fallback of any kind.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_PATH = os.path.join(HERE, "libibcomm_hip.so")

OK, INVALID_ARGUMENT, TRANSPORT_ERROR, DEVICE_ERROR, NOT_SUPPORTED = 0, 1, 2, 3, 4
F32, I32, F64, I64 = 0, 1, 2, 3
RING, RABENSEIFNER = 0, 1
LAND_MEMCPY, LAND_KERNEL, LAND_DIRECT, LAND_STAGED = 0, 1, 2, 3

EXPORTS = [
    "ibcomm_hip_last_error", "ibcomm_hip_fabric_create", "ibcomm_hip_fabric_destroy", "ibcomm_hip_comm_create",
    "ibcomm_hip_comm_destroy", "ibcomm_hip_comm_register_myself", "ibcomm_hip_allreduce_ring",
    "ibcomm_hip_allreduce_rabenseifner", "ibcomm_hip_allreduce_ring_host", "ibcomm_hip_allreduce_rabenseifner_host",
    "ibcomm_hip_allreduce_ring_f32", "ibcomm_hip_allreduce_ring_i32",
    "ibcomm_hip_allreduce_rabenseifner_f32", "ibcomm_hip_allreduce_rabenseifner_i32", "ibcomm_hip_world_allreduce", "ibcomm_hip_world_record", "ibcomm_hip_replay_allreduce",
    "ibcomm_hip_reduce", "ibcomm_hip_reduce_segments", "ibcomm_hip_max_segments", "ibcomm_hip_split_buffer",
    "ibcomm_hip_rank_to_chunk", "ibcomm_hip_get_exp_of_two", "ibcomm_hip_plan_create", "ibcomm_hip_plan_destroy",
    "ibcomm_hip_plan_counts", "ibcomm_hip_plan_range", "ibcomm_hip_plan_recv", "ibcomm_hip_plan_send",
    "ibcomm_hip_fabric_set_graph_mode", "ibcomm_hip_fabric_graph_counters", "ibcomm_hip_comm_set_max_fuse", "ibcomm_hip_comm_set_landing", "ibcomm_hip_comm_stats", "ibcomm_hip_comm_reset_stats",
    "ibcomm_hip_send", "ibcomm_hip_recv", "ibcomm_hip_send_poll", "ibcomm_hip_recv_poll", "ibcomm_hip_send_wait",
    "ibcomm_hip_recv_wait", "ibcomm_hip_bcast", "ibcomm_hip_comm_set_trace", "ibcomm_hip_comm_set_timer_base", "ibcomm_hip_comm_dump_trace",
    "ibcomm_hip_world_allreduce_noalloc", "ibcomm_hip_describe_launch", "ibcomm_hip_copy_segments",
    "ibcomm_hip_fabric_set_merge_mode", "ibcomm_hip_fabric_merge_counters",
]


class Stats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "calls", "reduce_launches", "reduce_segments", "reduce_elements", "landing_copies", "landing_bytes",
        "gather_copies", "gather_bytes", "messages_sent", "messages_received", "events_recorded", "stream_waits",
        "streams_created", "slots_high_water", "slot_count", "pool_blocks", "pool_bytes", "progress_passes", "reduce_kernel_segments",
        "largest_reduce_elements", "largest_reduce_kernel_segments", "largest_reduce_launches")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is not built; run __graft_entry__.build() (or make -C allreduce-proto_amd/csrc)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    vp, sz, i = C.c_void_p, C.c_size_t, C.c_int
    L.ibcomm_hip_last_error.restype = C.c_char_p
    L.ibcomm_hip_fabric_create.argtypes = [i, C.POINTER(vp)]
    L.ibcomm_hip_fabric_destroy.argtypes = [vp]
    L.ibcomm_hip_comm_create.argtypes = [vp, i, C.POINTER(vp)]
    L.ibcomm_hip_comm_destroy.argtypes = [vp]
    L.ibcomm_hip_comm_register_myself.argtypes = [vp, i]
    for name in ("ibcomm_hip_allreduce_ring", "ibcomm_hip_allreduce_rabenseifner"):
        getattr(L, name).argtypes = [vp, i, vp, vp, sz]
        getattr(L, name + "_host").argtypes = [vp, i, vp, vp, sz]
        for suffix in ("_f32", "_i32"):
            getattr(L, name + suffix).argtypes = [vp, vp, vp, sz]
    L.ibcomm_hip_world_allreduce.argtypes = [C.POINTER(vp), i, i, i, C.POINTER(vp), C.POINTER(vp), sz]
    L.ibcomm_hip_world_allreduce_noalloc.argtypes = [i, i, i, C.POINTER(vp), C.POINTER(vp), sz, vp]
    L.ibcomm_hip_world_record.argtypes = [C.POINTER(vp), i, i, i, i, C.POINTER(vp), C.POINTER(vp), sz]
    L.ibcomm_hip_replay_allreduce.argtypes = [vp, i, i, vp, vp, sz]
    L.ibcomm_hip_reduce.argtypes = [i, vp, vp, vp, sz, vp]
    L.ibcomm_hip_reduce_segments.argtypes = [i, i, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp), C.POINTER(sz), vp]
    L.ibcomm_hip_copy_segments.argtypes = [i, i, C.POINTER(vp), C.POINTER(vp), C.POINTER(sz), vp]
    L.ibcomm_hip_describe_launch.argtypes = [i, i, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp), C.POINTER(sz), C.POINTER(i), C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    L.ibcomm_hip_split_buffer.argtypes = [sz, sz, i, C.c_char_p, C.POINTER(sz), C.POINTER(sz), i, C.POINTER(i)]
    L.ibcomm_hip_rank_to_chunk.argtypes = [i, i, C.POINTER(i), C.POINTER(i)]
    L.ibcomm_hip_get_exp_of_two.argtypes = [i]
    L.ibcomm_hip_plan_create.argtypes = [i, i, i, sz, sz, C.c_char_p, C.POINTER(vp)]
    L.ibcomm_hip_plan_destroy.argtypes = [vp]
    L.ibcomm_hip_plan_destroy.restype = None
    L.ibcomm_hip_plan_counts.argtypes = [vp, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    L.ibcomm_hip_plan_range.argtypes = [vp, i, C.POINTER(sz), C.POINTER(sz)]
    L.ibcomm_hip_plan_recv.argtypes = [vp, i, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    L.ibcomm_hip_plan_send.argtypes = [vp, i, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    L.ibcomm_hip_fabric_set_graph_mode.argtypes = [vp, i]
    L.ibcomm_hip_fabric_graph_counters.argtypes = [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
    L.ibcomm_hip_fabric_set_merge_mode.argtypes = [vp, i]
    L.ibcomm_hip_fabric_merge_counters.argtypes = [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
    L.ibcomm_hip_comm_set_max_fuse.argtypes = [vp, i]
    L.ibcomm_hip_comm_set_landing.argtypes = [vp, i]
    L.ibcomm_hip_comm_stats.argtypes = [vp, C.POINTER(Stats)]
    L.ibcomm_hip_comm_reset_stats.argtypes = [vp]
    L.ibcomm_hip_send.argtypes = [vp, i, vp, sz, i]
    L.ibcomm_hip_recv.argtypes = [vp, i, vp, sz, i]
    L.ibcomm_hip_send_poll.argtypes = [vp, i, C.POINTER(i)]
    L.ibcomm_hip_recv_poll.argtypes = [vp, i, C.POINTER(i)]
    L.ibcomm_hip_send_wait.argtypes = [vp, i]
    L.ibcomm_hip_recv_wait.argtypes = [vp, i]
    L.ibcomm_hip_bcast.argtypes = [vp, vp, sz, i]
    L.ibcomm_hip_comm_set_trace.argtypes = [vp, i]
    L.ibcomm_hip_comm_set_timer_base.argtypes = [vp]
    L.ibcomm_hip_comm_dump_trace.argtypes = [vp]
    _lib = L
    return L


def last_error():
    return lib().ibcomm_hip_last_error().decode(errors="replace")


def _env(chunksize):
    return None if chunksize is None else str(chunksize).encode()


def split_buffer(length, sizeof_element, world, chunksize=None, cap=1 << 16):
    starts = (C.c_size_t * cap)()
    ends = (C.c_size_t * cap)()
    n = C.c_int(0)
    rc = lib().ibcomm_hip_split_buffer(length, sizeof_element, world, _env(chunksize), starts, ends, cap, C.byref(n))
    if rc == 0 and n.value > cap:
        return split_buffer(length, sizeof_element, world, chunksize, cap=n.value)
    return rc, [(starts[k], ends[k]) for k in range(min(n.value, cap))]


def rank_to_chunk(n_ranges, world):
    first = (C.c_int * world)()
    count = (C.c_int * world)()
    assert lib().ibcomm_hip_rank_to_chunk(n_ranges, world, first, count) == 0
    return [list(range(first[r], first[r] + count[r])) for r in range(world)]


def world_allreduce_noalloc(world, algo, dtype, send_ptrs, recv_ptrs, length, stream=None):
    """The whole-world allreduce that allocates nothing, enqueued on `stream` (a hipStream_t value or
    None for the default stream); the caller synchronises.  Returns the library's status code."""
    sp = (C.c_void_p * world)(*send_ptrs)
    rp = (C.c_void_p * world)(*recv_ptrs)
    return lib().ibcomm_hip_world_allreduce_noalloc(world, algo, dtype, sp, rp, length, stream)


class Plan:
    """One rank's message plan: .ranges, .recvs [(chunk, peer, kind)], .sends [(chunk, peer, dep)]."""

    def __init__(self, algo, world, rank, length, sizeof_element=4, chunksize=None):
        h = C.c_void_p()
        self.rc = lib().ibcomm_hip_plan_create(algo, world, rank, length, sizeof_element, _env(chunksize), C.byref(h))
        self.ranges, self.recvs, self.sends = [], [], []
        if self.rc != 0:
            return
        L = lib()
        nc, nr, ns = C.c_int(), C.c_int(), C.c_int()
        L.ibcomm_hip_plan_counts(h, C.byref(nc), C.byref(nr), C.byref(ns))
        a, b, c = C.c_int(), C.c_int(), C.c_int()
        s, e = C.c_size_t(), C.c_size_t()
        for k in range(nc.value):
            L.ibcomm_hip_plan_range(h, k, C.byref(s), C.byref(e))
            self.ranges.append((s.value, e.value))
        for k in range(nr.value):
            L.ibcomm_hip_plan_recv(h, k, C.byref(a), C.byref(b), C.byref(c))
            self.recvs.append((a.value, b.value, c.value))
        for k in range(ns.value):
            L.ibcomm_hip_plan_send(h, k, C.byref(a), C.byref(b), C.byref(c))
            self.sends.append((a.value, b.value, c.value))
        L.ibcomm_hip_plan_destroy(h)


class World:
    """A loopback world of `n` emulated ranks on the current HIP device."""

    def __init__(self, n):
        L = lib()
        self.n = n
        self.fabric = C.c_void_p()
        self.comms = []
        rc = L.ibcomm_hip_fabric_create(n, C.byref(self.fabric))
        if rc:
            raise RuntimeError("fabric_create: %d %s" % (rc, last_error()))
        for r in range(n):
            h = C.c_void_p()
            rc = L.ibcomm_hip_comm_create(self.fabric, n, C.byref(h))
            if rc:
                self.close()
                raise RuntimeError("comm_create: %d %s" % (rc, last_error()))
            L.ibcomm_hip_comm_register_myself(h, r)
            self.comms.append(h)

    def set_graph_mode(self, mode):
        assert lib().ibcomm_hip_fabric_set_graph_mode(self.fabric, mode) == 0, last_error()

    def graph_counters(self):
        """-> (eager calls, graphs captured, graph replays) of the single-thread driver."""
        a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert lib().ibcomm_hip_fabric_graph_counters(self.fabric, C.byref(a), C.byref(b), C.byref(c)) == 0
        return a.value, b.value, c.value

    def set_merge_mode(self, mode):
        assert lib().ibcomm_hip_fabric_set_merge_mode(self.fabric, mode) == 0, last_error()

    def merge_counters(self):
        """-> (launches the ranks handed in while worlds were recorded, launches recorded after merging)."""
        a, b = C.c_uint64(), C.c_uint64()
        assert lib().ibcomm_hip_fabric_merge_counters(self.fabric, C.byref(a), C.byref(b)) == 0
        return a.value, b.value

    def set_max_fuse(self, f):
        for h in self.comms:
            assert lib().ibcomm_hip_comm_set_max_fuse(h, f) == 0, last_error()

    def set_landing(self, mode):
        for h in self.comms:
            assert lib().ibcomm_hip_comm_set_landing(h, mode) == 0, last_error()

    def allreduce_ptrs(self, algo, dtype, send_ptrs, recv_ptrs, length):
        """Single-thread driver over raw device pointers.  Returns the library's status code."""
        n = self.n
        comms = (C.c_void_p * n)(*[h.value for h in self.comms])
        sp = (C.c_void_p * n)(*send_ptrs)
        rp = (C.c_void_p * n)(*recv_ptrs)
        return lib().ibcomm_hip_world_allreduce(comms, n, algo, dtype, sp, rp, length)

    def record(self, rank, algo, dtype, send_ptrs, recv_ptrs, length):
        """World allreduce that also records what `rank` receives, for replay()."""
        n = self.n
        comms = (C.c_void_p * n)(*[h.value for h in self.comms])
        sp = (C.c_void_p * n)(*send_ptrs)
        rp = (C.c_void_p * n)(*recv_ptrs)
        return lib().ibcomm_hip_world_record(comms, n, rank, algo, dtype, sp, rp, length)

    def replay(self, rank, algo, dtype, send_ptr, recv_ptr, length):
        """`rank` alone against the recorded peers."""
        return lib().ibcomm_hip_replay_allreduce(self.comms[rank], algo, dtype, send_ptr, recv_ptr, length)

    def allreduce_threads(self, algo, dtype, send_ptrs, recv_ptrs, length, host=False):
        """One host thread per rank, each in the blocking per-rank call (how the reference is used).
        With host=True the pointers are host memory (the AllreduceRing / AllreduceRabenseifner calls)."""
        import threading
        L = lib()
        if host:
            fn = L.ibcomm_hip_allreduce_ring_host if algo == RING else L.ibcomm_hip_allreduce_rabenseifner_host
        else:
            fn = L.ibcomm_hip_allreduce_ring if algo == RING else L.ibcomm_hip_allreduce_rabenseifner
        rcs = [None] * self.n
        msgs = [""] * self.n

        def run(r):
            rcs[r] = fn(self.comms[r], dtype, send_ptrs[r], recv_ptrs[r], length)
            if rcs[r]:
                msgs[r] = last_error()

        th = [threading.Thread(target=run, args=(r,)) for r in range(self.n)]
        for t in th:
            t.start()
        for t in th:
            t.join()
        return rcs, msgs

    def set_trace(self, enabled=True):
        for h in self.comms:
            lib().ibcomm_hip_comm_set_trace(h, 1 if enabled else 0)
            lib().ibcomm_hip_comm_set_timer_base(h)

    def dump_trace(self):
        """Writes ${IBCOMM_TRACE_FILE:-ibcomm_trace}_<rank>.dat for every rank."""
        for h in self.comms:
            assert lib().ibcomm_hip_comm_dump_trace(h) == 0, last_error()

    def stats(self, rank=0):
        s = Stats()
        assert lib().ibcomm_hip_comm_stats(self.comms[rank], C.byref(s)) == 0
        return s.as_dict()

    def reset_stats(self):
        for h in self.comms:
            lib().ibcomm_hip_comm_reset_stats(h)

    def close(self):
        L = lib()
        for h in self.comms:
            L.ibcomm_hip_comm_destroy(h)
        self.comms = []
        if self.fabric:
            L.ibcomm_hip_fabric_destroy(self.fabric)
            self.fabric = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()
