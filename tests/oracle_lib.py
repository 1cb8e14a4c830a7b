"""ctypes view of the CPU oracle (oracle/libibcomm_oracle.so) for the tests.

The oracle is test infrastructure: it restates the reference's algorithms on
the CPU so that the HIP path can be compared with it bit for bit.  This module
is only ever imported from tests/, __graft_entry__.smoke() and bench.py's CPU
baseline leg.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libibcomm_oracle.so")
REF_UTIL_SO = os.path.join(ORACLE_DIR, "_ref", "libibcomm_ref_util.so")

OK, INVALID_ARGUMENT, IBVERBS_ERROR, CUDA_ERROR, NOT_SUPPORTED = 0, 1, 2, 3, 4
F32, I32, F64, I64 = 0, 1, 2, 3
RING_CPU, RABEN_CPU, RING_GPU, RABEN_GPU = 0, 1, 2, 3
NP_DTYPE = {F32: np.float32, I32: np.int32, F64: np.float64, I64: np.int64}
DTYPE_OF = {np.dtype(v): k for k, v in NP_DTYPE.items()}


class Stats(C.Structure):
    _fields_ = [("pool_slots_high_water", C.c_int), ("pool_blocks", C.c_int),
                ("slots_leaked", C.c_int), ("messages", C.c_long)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "libibcomm_oracle.so"])
    L = C.CDLL(ORACLE_SO)
    L.orc_ceil_div.restype = C.c_int64
    L.orc_ceil_div.argtypes = [C.c_int64, C.c_int64]
    L.orc_get_exp_of_two.argtypes = [C.c_int]
    L.orc_read_chunk_size.argtypes = [C.c_char_p, C.POINTER(C.c_int)]
    L.orc_split_buffer.argtypes = [C.c_size_t, C.c_size_t, C.c_int, C.c_char_p, C.POINTER(C.c_size_t),
                                   C.POINTER(C.c_size_t), C.c_int, C.POINTER(C.c_int)]
    L.orc_rank_to_chunk.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    L.orc_rank_to_chunk.restype = None
    L.orc_reduce_inplace.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]
    L.orc_reduce_inplace.restype = None
    L.orc_allreduce.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                C.c_size_t, C.c_char_p, C.c_size_t, C.POINTER(Stats)]
    L.orc_wire_count.restype = C.c_long
    L.orc_wire_count.argtypes = [C.c_int, C.c_int]
    L.orc_wire_get.argtypes = [C.c_int, C.c_int, C.c_long, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    L.orc_closed_form_ring.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_void_p), C.c_void_p, C.c_size_t, C.c_char_p]
    L.orc_closed_form_tree.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_void_p), C.c_void_p, C.c_size_t]
    L.orc_time_reduce_f32.restype = C.c_double
    L.orc_time_reduce_f32.argtypes = [C.c_size_t, C.c_int]
    _lib = L
    return L


def _env(chunksize):
    if chunksize is None:
        return None
    return str(chunksize).encode()


def split_buffer(length, sizeof_element, world, chunksize=None):
    """-> (rc, [(start, end), ...])"""
    cap = 4 * world
    if chunksize is not None:
        try:
            v = int(str(chunksize))
            if v >= sizeof_element:
                cap = max(cap, -(-length // (v // sizeof_element)))
        except ValueError:
            pass
    cap = int(cap) + 1
    starts = (C.c_size_t * cap)()
    ends = (C.c_size_t * cap)()
    n = C.c_int(0)
    rc = lib().orc_split_buffer(length, sizeof_element, world, _env(chunksize), starts, ends, cap, C.byref(n))
    return rc, [(starts[i], ends[i]) for i in range(min(n.value, cap))]


def rank_to_chunk(n_ranges, world):
    first = (C.c_int * world)()
    count = (C.c_int * world)()
    lib().orc_rank_to_chunk(n_ranges, world, first, count)
    return [list(range(first[r], first[r] + count[r])) for r in range(world)]


def _ptr_array(arrays):
    arr = (C.c_void_p * len(arrays))()
    for i, a in enumerate(arrays):
        arr[i] = a.ctypes.data
    return arr


def allreduce(algo, sendbufs, chunksize=None, pool_block_bytes=0):
    """sendbufs: list of equal-length 1-D numpy arrays (one per rank).
    -> (rc, [recvbuf per rank], Stats)"""
    world = len(sendbufs)
    sendbufs = [np.ascontiguousarray(s) for s in sendbufs]
    dt = DTYPE_OF[sendbufs[0].dtype]
    n = sendbufs[0].size
    recv = []
    for _ in range(world):
        r = np.empty(n, dtype=sendbufs[0].dtype)
        r.view(np.uint8)[:] = 0x55  # poison: every element must be overwritten
        recv.append(r)
    st = Stats()
    rc = lib().orc_allreduce(algo, dt, world, _ptr_array(sendbufs), _ptr_array(recv), n, _env(chunksize),
                             pool_block_bytes, C.byref(st))
    return rc, recv, st


def allreduce_into(algo, sendbufs, recvbufs, chunksize=None, pool_block_bytes=0):
    """Like allreduce() into caller-owned contiguous recvbufs, with nothing but the oracle call inside
    (what a timing loop wants). -> rc"""
    st = Stats()
    return lib().orc_allreduce(algo, DTYPE_OF[sendbufs[0].dtype], len(sendbufs), _ptr_array(sendbufs), _ptr_array(recvbufs),
                               sendbufs[0].size, _env(chunksize), pool_block_bytes, C.byref(st))


def wire_log(world):
    """{(src, dst): [(offset, n), ...]} of the last allreduce() call."""
    out = {}
    L = lib()
    for s in range(world):
        for d in range(world):
            k = L.orc_wire_count(s, d)
            if k <= 0:
                continue
            off = C.c_size_t()
            n = C.c_size_t()
            msgs = []
            for i in range(k):
                assert L.orc_wire_get(s, d, i, C.byref(off), C.byref(n)) == 0
                msgs.append((off.value, n.value))
            out[(s, d)] = msgs
    return out


def closed_form_ring(sendbufs, chunksize=None):
    sendbufs = [np.ascontiguousarray(s) for s in sendbufs]
    out = np.empty_like(sendbufs[0])
    rc = lib().orc_closed_form_ring(DTYPE_OF[sendbufs[0].dtype], len(sendbufs), _ptr_array(sendbufs),
                                    out.ctypes.data, out.size, _env(chunksize))
    return rc, out


def closed_form_tree(sendbufs):
    sendbufs = [np.ascontiguousarray(s) for s in sendbufs]
    out = np.empty_like(sendbufs[0])
    rc = lib().orc_closed_form_tree(DTYPE_OF[sendbufs[0].dtype], len(sendbufs), _ptr_array(sendbufs),
                                    out.ctypes.data, out.size)
    return rc, out


def ref_util():
    """The reference's own util.h compiled into oracle/_ref, or None if it was not built."""
    if not os.path.exists(REF_UTIL_SO):
        return None
    L = C.CDLL(REF_UTIL_SO)
    L.ref_ceil_div.restype = C.c_longlong
    L.ref_ceil_div.argtypes = [C.c_longlong, C.c_longlong]
    L.ref_get_exp_of_two.argtypes = [C.c_int]
    L.ref_error_code.argtypes = [C.c_int]
    return L


# --------------------------------------------------------------------------
# Independent numpy statements of what the schedules must compute.  They share
# no code with the oracle: partitioning is re-derived here from the rule
# (ibverbs_communicator.cpp:637-707), and sums are explicit numpy adds in the
# order that reading the schedules gives (ring: the owner of the chunk group starts; tree: pairwise).
# --------------------------------------------------------------------------

def np_partition(length, itemsize, world, chunksize=None):
    if chunksize is None:
        chunks = 4 * world
        epc = -(-length // chunks)
    else:
        epc = int(chunksize) // itemsize
        chunks = -(-length // epc)
    ranges = []
    for i in range(chunks):
        s, e = epc * i, min(length, epc * (i + 1))
        if s < e:
            ranges.append((s, e))
    per, rem = divmod(len(ranges), world)
    groups, cid = [], 0
    for r in range(world):
        k = per + (1 if r < rem else 0)
        groups.append(list(range(cid, cid + k)))
        cid += k
    return ranges, groups


def np_ring(sendbufs, chunksize=None):
    """Left fold starting at the rank that owns the element's chunk group."""
    world = len(sendbufs)
    if world == 1:
        return sendbufs[0].copy()
    n = sendbufs[0].size
    ranges, groups = np_partition(n, sendbufs[0].itemsize, world, chunksize)
    out = np.empty_like(sendbufs[0])
    with np.errstate(over="ignore"):
        for g, cids in enumerate(groups):
            for c in cids:
                s, e = ranges[c]
                acc = sendbufs[g][s:e].copy()
                for j in range(1, world):
                    acc = acc + sendbufs[(g + j) % world][s:e]
                out[s:e] = acc
    return out


def np_tree(sendbufs):
    """Balanced pairwise tree over rank index."""
    level = [s.copy() for s in sendbufs]
    with np.errstate(over="ignore"):
        while len(level) > 1:
            level = [level[i] + level[i + 1] for i in range(0, len(level), 2)]
    return level[0]


def bits(a):
    """View as unsigned integers so that comparisons are bit-exact (NaN-safe, -0 != +0)."""
    a = np.ascontiguousarray(a)
    return a.view({4: np.uint32, 8: np.uint64}[a.itemsize])
