"""CPU tests of the product library's host side through its C ABI (no device calls):
exports, partitioning parity with the oracle, and message plans against the wire order of the
oracle's restatement of the reference state machines."""
import ctypes as C
import re

import numpy as np
import pytest

import hip_lib as H
import oracle_lib as O


def test_library_exports_every_declared_symbol():
    header = open(H.ROOT + "/include/ibcomm_hip.h").read()
    declared = sorted(set(re.findall(r"\b(ibcomm_hip_[a-z0-9_]+)\s*\(", header)))
    assert declared, "no declarations found"
    L = H.lib()
    for name in declared:
        assert hasattr(L, name), "%s is declared in include/ibcomm_hip.h but not exported" % name
    assert sorted(H.EXPORTS) == declared


def test_error_codes_are_the_reference_exit_codes():
    assert (H.INVALID_ARGUMENT, H.TRANSPORT_ERROR, H.DEVICE_ERROR, H.NOT_SUPPORTED) == (1, 2, 3, 4)


def test_get_exp_of_two_matches_oracle():
    for n in range(0, 3000):
        assert H.lib().ibcomm_hip_get_exp_of_two(n) == O.lib().orc_get_exp_of_two(n)


def test_split_buffer_matches_oracle():
    for world in range(1, 9):
        for length in list(range(0, 70)) + [2521, 100003]:
            for chunk in (None, "4", "8", "12", "64", "0", "3", "-8", "1k", "100000000"):
                a = H.split_buffer(length, 4, world, chunk)
                b = O.split_buffer(length, 4, world, chunk)
                assert a[0] == b[0], (world, length, chunk, H.last_error())
                if a[0] == 0:
                    assert a[1] == b[1]
                    assert H.rank_to_chunk(len(a[1]), world) == O.rank_to_chunk(len(b[1]), world)
    assert H.split_buffer(536870911, 4, 32, 16777216) == O.split_buffer(536870911, 4, 32, 16777216)
    # beyond the reference's int range the ranges simply continue (documented deviation)
    rc, r = H.split_buffer(3 * 2**31 + 5, 4, 4)
    assert rc == 0 and r[-1][1] == 3 * 2**31 + 5 and len(r) == 16


def wire_of_plan(algo, world, n, chunk):
    """{(src, dst): [(offset, count), ...]} from every rank's plan."""
    wire = {}
    plans = [H.Plan(algo, world, r, n, 4, chunk) for r in range(world)]
    for r, p in enumerate(plans):
        assert p.rc == 0, H.last_error()
        for c, peer, dep in p.sends:
            s, e = p.ranges[c]
            wire.setdefault((r, peer), []).append((s, e - s))
    return plans, wire


@pytest.mark.parametrize("world,n,chunk", [(2, 64, None), (3, 100, None), (4, 256, 16), (5, 1003, None), (8, 4096, 64)])
def test_ring_plan_wire_order_is_the_reference_order(world, n, chunk):
    bufs = [np.arange(n, dtype=np.int32) + r for r in range(world)]
    assert O.allreduce(O.RING_GPU, bufs, chunk)[0] == 0
    want = O.wire_log(world)
    plans, wire = wire_of_plan(H.RING, world, n, chunk)
    assert wire == want
    for r, p in enumerate(plans):
        # receives mirror the predecessor's sends one for one
        prev = plans[(r - 1) % world]
        assert [c for c, _, _ in p.recvs] == [c for c, _, _ in prev.sends]
        assert all(peer == (r - 1) % world for _, peer, _ in p.recvs)
        kinds = [k for _, _, k in p.recvs]
        assert kinds == [0] * (len(kinds) // 2) + [2] * (len(kinds) // 2)


@pytest.mark.parametrize("world,n,chunk", [(2, 64, None), (4, 256, 16), (8, 8 * 24, None), (16, 4099, None), (4, 1021, None)])
def test_rabenseifner_plan_wire_order_is_the_reference_order(world, n, chunk):
    bufs = [np.arange(n, dtype=np.int32) + r for r in range(world)]
    assert O.allreduce(O.RABEN_GPU, bufs, chunk)[0] == 0
    want = O.wire_log(world)
    plans, wire = wire_of_plan(H.RABENSEIFNER, world, n, chunk)
    assert wire == want
    for r, p in enumerate(plans):
        # what r consumes from a peer is, in order, what that peer emits towards r
        for peer in {q for _, q, _ in p.recvs}:
            got = [c for c, q, _ in p.recvs if q == peer]
            sent = [c for c, q, _ in plans[peer].sends if q == r]
            assert got == sent
        # first halving step adds to sendbuf, later ones accumulate, doubling steps store
        kinds = [k for _, _, k in p.recvs]
        assert kinds == sorted(kinds)
        # every send out of recvbuf names the receive that produced the data
        for c, _, dep in p.sends:
            if dep >= 0:
                assert p.recvs[dep][0] == c


def test_plan_validation_order_and_codes():
    assert H.Plan(H.RABENSEIFNER, 3, 0, 12).rc == 4     # not a power of two
    assert H.Plan(H.RABENSEIFNER, 3, 0, 1).rc == 4
    assert H.Plan(H.RING, 2, 0, 1).rc == 4              # too short
    assert H.Plan(H.RING, 4, 0, 256, 4, "3").rc == 1    # not a multiple of sizeof(T)
    assert H.Plan(H.RING, 4, 0, 256, 4, "1024").rc == 1  # fewer than 2N chunks
    assert H.Plan(H.RING, 4, 4, 256).rc == 1            # rank outside the world
    p = H.Plan(H.RING, 1, 0, 10)
    assert p.rc == 0 and p.recvs == [] and p.sends == []


def test_baseline_config_plan_shapes():
    # cfg 2: ring, 8 ranks, 32 chunks: 28 reductions, 28 gathers, 4 + 28 + 24 sends per rank
    p = H.Plan(H.RING, 8, 0, 67108864, 4, 8388608)
    assert len(p.ranges) == 32 and len(p.recvs) == 56 and len(p.sends) == 56
    assert sum(1 for _, _, k in p.recvs if k == 0) == 28
    # cfg 3: Rabenseifner, 16 ranks, 98 chunks (7,7,6,...): reductions per rank as derived from the schedule
    want = {0: 90, 1: 92, 3: 94, 7: 97, 15: 97, 5: 92, 11: 94, 14: 90}
    for r, k in want.items():
        p = H.Plan(H.RABENSEIFNER, 16, r, 102760448, 4, 4194304)
        assert len(p.ranges) == 98
        assert sum(1 for _, _, kind in p.recvs if kind != 2) == k, r
        assert sum(1 for _, _, kind in p.recvs if kind == 2) == (91 if r in (7, 15) else 92)
    # cfg 5: ragged tail
    p = H.Plan(H.RING, 32, 31, 536870911, 4, 16777216)
    assert len(p.ranges) == 128 and p.ranges[-1] == (127 * 4194304, 536870911)
    assert len(p.recvs) == 2 * 31 * 4


def test_launch_geometry_follows_the_segment_size():
    # ibcomm_hip_describe_launch touches no device: how a launch would be issued is decided on the host.
    # The reference fixes 512 threads and min(ceil(n / 512), 65535) blocks for every size
    # (allreduce_cuda_impl.h:24, 116-117); here the aligned kernel runs one 16-byte vector per lane,
    # 256-thread workgroups up to 2 Mi fp32 per segment and 128 beyond, die-local tile order from 64 tiles
    # up to 32 Mi fp32, and anything off the 16-byte grid goes to the general kernel, which keeps that geometry
    # around its peeled ends.
    import ctypes as C
    L = H.lib()

    def describe(lens, dtype=H.F32, base=(0x10000000, 0x20000000, 0x30000000)):
        k = len(lens)
        vp = C.c_void_p
        d = (vp * k)(*[base[0] + i * 0x1000000 for i in range(k)])
        a = (vp * k)(*[base[1] + i * 0x1000000 for i in range(k)])
        b = (vp * k)(*[base[2] + i * 0x1000000 for i in range(k)])
        ln = (C.c_size_t * k)(*lens)
        al, th, dl, wt = C.c_int(-1), C.c_int(-1), C.c_int(-1), C.c_int(-1)
        assert L.ibcomm_hip_describe_launch(dtype, k, d, a, b, ln, C.byref(al), C.byref(th), C.byref(dl), C.byref(wt)) == 0, H.last_error()
        through.append(wt.value)
        return al.value, th.value, dl.value

    through = []

    assert describe([16384]) == (1, 256, 0)            # config 4's chunk on its own: 16 tiles, too few to permute
    assert describe([65536]) == (1, 256, 1)            # 64 tiles
    assert describe([2097152]) == (1, 256, 1)          # config 4's merged ring step
    assert describe([2097152 + 1024]) == (1, 128, 1)   # 2049 tiles: 128-thread workgroups from here
    assert describe([8388608]) == (1, 128, 1)          # config 2's ring step
    assert describe([25165824, 25165824]) == (1, 128, 1)  # config 3's first halving step, two segments
    assert describe([33554432]) == (1, 128, 1)
    assert describe([33554432 + 1024]) == (1, 128, 0)  # beyond 32 Mi fp32 the plain order is the faster one
    assert describe([67108864]) == (1, 128, 0)
    assert describe([8388608], H.F64) == (1, 128, 1) and describe([1048576], H.F64) == (1, 256, 1)  # limits are in bytes
    assert describe([4194303]) == (0, 128, 1)          # config 5's ragged last chunk: not a whole number of vectors
    assert describe([4194304, 4194304, 4194304, 4194303]) == (0, 128, 1)  # its whole last ring step
    assert describe([8388608], base=(0x10000004, 0x20000004, 0x30000004)) == (0, 128, 1)  # off the 16-byte grid
    assert describe([2521]) == (0, 256, 0)             # the reference tester's 2521 elements
    assert describe([8388608], base=(0x10000010, 0x20000000, 0x30000000)) == (0, 128, 1)  # dst off the 128-byte grid
    assert describe([8388608], base=(0x10000080, 0x20000010, 0x30000020)) == (1, 128, 1)  # operands need 16 bytes only
    assert describe([0, 8388608, 0]) == (1, 128, 1)    # empty segments do not count
    assert describe([]) == (0, 256, 0)
    assert L.ibcomm_hip_describe_launch(7, 0, None, None, None, None, None, None, None, None) == H.INVALID_ARGUMENT
    # stores go through the memory-side cache while a launch writes at most 128 MiB
    through.clear()
    for lens in ([8388608], [16777216], [33554432], [33554432 + 4], [25165824, 25165824], [4194304] * 8, [4194304] * 9):
        describe(lens)
    assert through == [1, 1, 1, 0, 0, 1, 0]
