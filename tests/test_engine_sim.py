"""Host-logic tests of the allreduce engine (allreduce-proto_amd/csrc/engine.hpp, plan.hpp, loopback.hpp,
memory_pool.hpp) on a simulated device.

The same engine templates the product instantiates with the HIP runtime are instantiated here with
tests/support/sim_backend.hpp, which defers every copy and launch, runs them in a random order that
respects the recorded stream/event dependencies, and checks that every pair of conflicting memory
accesses is ordered.  Results must be bit-identical to the oracle's restatement of
AllreduceRingCuda / AllreduceRabenseifnerCuda.
"""
import numpy as np
import pytest

import oracle_lib as O
import sim_lib as S

RING, RABEN = 0, 1
ORACLE_ALGO = {RING: O.RING_GPU, RABEN: O.RABEN_GPU}


def rand_bufs(world, n, seed=0, dtype=np.float32):
    return [(np.random.default_rng(seed + r).standard_normal(n) * 3).astype(dtype) for r in range(world)]


def check(algo, bufs, chunk=None, unchecked_ok=False, **kw):
    """unchecked_ok: the run may be too large for the simulator's race check (races == -1)."""
    rc, recv, rep = S.allreduce(algo, bufs, chunk, **kw)
    assert rc == 0, rep.error.decode()
    orc, want, _ = O.allreduce(ORACLE_ALGO[algo], bufs, chunk)
    assert orc == 0
    for r in range(len(bufs)):
        assert np.array_equal(O.bits(recv[r]), O.bits(want[r])), "rank %d differs from the oracle" % r
    assert rep.unrecorded_waits == 0
    if kw.get("threaded", 0) != 1:  # with one engine per thread the graph of device work is not checked for races
        assert rep.races == 0 or (unchecked_ok and rep.races == -1), rep.first_race.decode()
    return rep


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
@pytest.mark.parametrize("fuse", [1, 3, 48, 64])
@pytest.mark.parametrize("world", [2, 3, 4, 5, 8])
def test_ring_matches_oracle(world, fuse, landing):
    for n, chunk in [(world, None), (4 * world + 1, None), (1000 + world, None), (512, 16)]:
        if chunk and -(-n // (chunk // 4)) < 2 * world:
            continue
        check(RING, rand_bufs(world, n, seed=n), chunk, max_fuse=fuse, landing=landing, seed=world * 7 + fuse)


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
@pytest.mark.parametrize("fuse", [1, 3, 48, 64])
@pytest.mark.parametrize("world", [2, 4, 8, 16])
def test_rabenseifner_matches_oracle(world, fuse, landing):
    for n, chunk in [(world, None), (4 * world + 3, None), (2000 + world, None), (1024, 16)]:
        if chunk and -(-n // (chunk // 4)) < 2 * world:
            continue
        check(RABEN, rand_bufs(world, n, seed=n + 1), chunk, max_fuse=fuse, landing=landing, seed=world * 11 + fuse)


@pytest.mark.parametrize("algo,world", [(RING, 4), (RING, 3), (RABEN, 4), (RABEN, 8)])
def test_many_random_schedules(algo, world):
    bufs = rand_bufs(world, 777, seed=42)
    for seed in range(12):
        check(algo, bufs, 32, max_fuse=1 + seed % 5, landing=seed % 4, seed=seed, streams=1 + seed % 4)


@pytest.mark.parametrize("algo,world", [(RING, 4), (RABEN, 4)])
def test_tiny_pool_forces_slot_reuse(algo, world):
    # two slots only: every landing has to order itself after the previous reader of its slot
    bufs = rand_bufs(world, 4096, seed=3)
    stride = 256 + 256  # 64-byte chunks + 16 B margin round up to 256; pool of 512 B gives two slots
    for fuse in (1, 2, 7):
        rep = check(algo, bufs, 64, max_fuse=fuse, landing=0, pool_bytes=stride, seed=fuse)
        assert rep.rank0.slot_count >= 2
    # a pool smaller than one chunk grows instead of failing
    rep = check(algo, bufs, 1024, max_fuse=4, landing=1, pool_bytes=64, seed=9)
    assert rep.rank0.pool_blocks >= 2


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
@pytest.mark.parametrize("pool_bytes", [1 << 16, 64 << 20])
def test_thousands_of_chunks_per_step_do_not_grow_the_pool(landing, pool_bytes):
    # 4 ranks x 1 Mi fp32 in 256-byte chunks: 4,096 chunks per ring step.  A rank collects every message
    # that is there before it launches, and each of them wants a landing or a staging slot: with slots
    # for 256 chunks (64 KiB block) or 262,144 (64 MiB) the collective must get by on the one block the
    # pool was created with -- launching early, or leaving partial sums in recvbuf -- and stay bit-exact.
    bufs = rand_bufs(4, 1 << 20, seed=21)
    big = landing == 0  # one device copy per message: some 200,000 operations
    rep = check(RING, bufs, 256, unchecked_ok=big, max_fuse=64, landing=landing, pool_bytes=pool_bytes, seed=landing)
    assert rep.rank0.pool_blocks == 1 and rep.rank0.pool_bytes == pool_bytes
    assert rep.rank0.slot_count == pool_bytes // 256
    assert rep.rank0.slots_high_water <= rep.rank0.slot_count
    if landing == 3:
        assert rep.rank0.slots_high_water == min(pool_bytes // 256, 2 * 4096)
    rep = check(RABEN, bufs, 256, unchecked_ok=big, max_fuse=64, landing=landing, pool_bytes=pool_bytes, seed=landing)
    assert rep.rank0.pool_blocks == 1


@pytest.mark.parametrize("algo,world", [(RING, 2), (RING, 4), (RABEN, 2), (RABEN, 8)])
def test_threads_one_per_rank(algo, world):
    bufs = rand_bufs(world, 3000, seed=8)
    for rep_i in range(3):
        check(algo, bufs, 64, max_fuse=4, landing=1 + rep_i % 3, threaded=True, seed=rep_i)


@pytest.mark.parametrize("algo,world", [(RING, 2), (RING, 5), (RABEN, 4), (RABEN, 8)])
def test_blocking_calls_of_all_ranks_meet_and_one_thread_drives(algo, world):
    # what the library's per-rank entry points do: every rank thread leaves its arguments, the last to
    # arrive runs the whole world; six calls in a row on the same communicators
    bufs = rand_bufs(world, 3000, seed=18)
    for landing in (0, 1, 2, 3):
        rep = check(algo, bufs, 64, max_fuse=64, landing=landing, threaded=2, repeats=6, seed=landing)
        assert rep.rank0.calls == 6


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
@pytest.mark.parametrize("algo,world", [(RING, 2), (RING, 5), (RING, 8), (RABEN, 4), (RABEN, 16)])
def test_launches_of_the_ranks_merge_while_a_world_is_recorded(algo, world, landing):
    # every rank issues on one stream, as while a world is recorded, and hands its launches to the collector:
    # launches that touch no common memory become one.  Bit-exact, free of conflicting accesses inside a
    # launch (the simulator checks the segments of one launch against one another), twice in a row.
    bufs = rand_bufs(world, 64 * 4 * world, seed=31)
    rep = check(algo, bufs, 256, max_fuse=64, landing=landing, threaded=3, repeats=2, pool_bytes=1 << 20, seed=landing)
    steps = 2 * (world - 1) if algo == RING else 2 * int(np.log2(world))
    per_call = rep.launches_issued // 2
    if landing in (2, 3):
        # nothing but the algorithm's own steps is left: one launch per step, whatever the number of ranks
        assert per_call == steps, (per_call, steps, rep.launches_collected)
    if landing == 0:
        assert rep.launches_issued <= rep.launches_collected  # reductions merge, the device copies stay
    if landing == 1:
        # a rank's landing copy and the reduction that reads it stay in order: the adds of a step merge, the copies do not
        assert steps < per_call < rep.launches_collected // 2


def test_merged_launches_on_random_shapes():
    rng = np.random.default_rng(77)
    for case in range(40):
        algo = int(rng.integers(0, 2))
        world = int(rng.choice([2, 4, 8, 16])) if algo == RABEN else int(rng.integers(2, 10))
        n = int(rng.integers(world, 5000))
        chunk = None
        if rng.random() < 0.6:
            epc = int(rng.integers(1, max(2, n // (2 * world) + 1)))
            if -(-n // epc) >= 2 * world:
                chunk = 4 * epc
        bufs = [(np.random.default_rng(case * 50 + r).standard_normal(n) * 9).astype(np.float32) for r in range(world)]
        in_place = bool(rng.random() < 0.2)  # (a second call in place would add up the first one's results)
        check(algo, bufs, chunk, max_fuse=int(rng.integers(1, 65)), landing=int(rng.integers(0, 4)), seed=case, threaded=3,
              repeats=1 if in_place else int(rng.integers(1, 3)), pool_bytes=int(rng.choice([512, 4096, 65536])), in_place=in_place)


def test_meeting_of_blocking_calls_handles_failures():
    held = S.lib().sim_rendezvous()
    names = ["five rounds, one driver each", "disagreeing ranks are all told", "a failed collective reaches every rank",
             "the same rank twice is refused", "a rank that gives up marks the world", "an abandoned world refuses meetings",
             "a waiting peer stops when another rank gives up", "usable again after a reset"]
    missing = [n for k, n in enumerate(names) if not held >> k & 1]
    assert not missing, missing


@pytest.mark.parametrize("algo", [RING, RABEN])
def test_repeated_calls_reuse_events_and_slots(algo):
    bufs = rand_bufs(4, 2048, seed=5)
    rep = check(algo, bufs, 64, max_fuse=3, repeats=4, seed=1)
    assert rep.rank0.calls == 4
    check(algo, bufs, 64, max_fuse=3, repeats=3, threaded=True, seed=2)
    check(algo, bufs, 64, max_fuse=3, repeats=4, landing=3, seed=3)  # staging slots are recycled across calls


@pytest.mark.parametrize("algo,world", [(RING, 3), (RING, 4), (RABEN, 4)])
def test_in_place(algo, world):
    bufs = rand_bufs(world, 1500, seed=6)
    orc, want, _ = O.allreduce(ORACLE_ALGO[algo], bufs)
    for landing in (0, 1, 2, 3):
        rc, recv, rep = S.allreduce(algo, bufs, max_fuse=5, landing=landing, in_place=True, seed=landing)
        assert rc == 0, rep.error.decode()
        for r in range(world):
            assert np.array_equal(O.bits(recv[r]), O.bits(want[r]))
        assert rep.races == 0, rep.first_race.decode()


def test_single_rank_is_a_copy():
    bufs = rand_bufs(1, 100)
    for algo in (RING, RABEN):
        rc, recv, rep = S.allreduce(algo, bufs)
        assert rc == 0 and np.array_equal(O.bits(recv[0]), O.bits(bufs[0]))


def test_dtypes():
    for dtype in (np.int32, np.float64, np.int64):
        bufs = [(np.random.default_rng(r).standard_normal(500) * 1000).astype(dtype) for r in range(4)]
        check(RING, bufs, max_fuse=4)
        check(RABEN, bufs, max_fuse=4)


def test_error_codes_match_reference():
    # tests/allreduce_test.py:198-225 and :132-153
    bufs = [np.arange(256, dtype=np.int32) for _ in range(4)]
    for chunk in ["0", "1", "2", "3", "-128", "1k", "1024"]:
        rc, _, rep = S.allreduce(RING, bufs, chunk)
        assert rc == 1, (chunk, rep.error)
    one = [np.ones(1, dtype=np.int32) for _ in range(2)]
    assert S.allreduce(RING, one)[0] == 4
    assert S.allreduce(RABEN, one)[0] == 4
    for world in (3, 5, 6):
        assert S.allreduce(RABEN, [np.arange(2 * world, dtype=np.int32) for _ in range(world)])[0] == 4
    # a failed call leaves the communicators usable
    rc, recv, rep = S.allreduce(RING, bufs, "16")
    assert rc == 0


def test_work_per_rank_matches_the_schedule():
    # ring, N ranks, q chunks per group: (N-1)q reductions and (N-1)q gathers per rank, 2(N-1)q messages
    world, n, chunk = 4, 4096, 64
    bufs = rand_bufs(world, n)
    rep = check(RING, bufs, chunk, max_fuse=1)
    q = n * 4 // chunk // world
    st = rep.rank0
    assert st.reduce_segments == (world - 1) * q and st.reduce_launches == (world - 1) * q
    assert st.reduce_elements == (world - 1) * n // world
    assert st.gather_bytes == (world - 1) * n // world * 4
    assert st.messages_received == 2 * (world - 1) * q and st.messages_sent == 2 * (world - 1) * q
    # fused: the driver steps all ranks in lockstep, so each pass sees exactly one ring step's
    # group (64 chunks here) and reduces it with as few launches as the segment limit allows
    rep = check(RING, bufs, chunk, max_fuse=64)
    assert rep.rank0.reduce_launches == world - 1 and rep.rank0.reduce_segments == (world - 1) * q
    rep = check(RING, bufs, chunk, max_fuse=48)
    assert rep.rank0.reduce_launches == 2 * (world - 1)
    # Rabenseifner rank 0 of 4: halving windows of 2 and 1 groups
    rep = check(RABEN, bufs, chunk, max_fuse=1)
    assert rep.rank0.reduce_segments == 3 * q and rep.rank0.gather_bytes == 3 * q * chunk


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
def test_contiguous_chunks_merge_into_one_kernel_segment(landing):
    # 256-byte chunks in 16-byte aligned buffers: pool slots lie back to back, so the 16 chunks of a
    # ring step follow one another in every operand and each launch carries a single segment
    world, n, chunk = 4, 4096, 256
    bufs = rand_bufs(world, n, seed=5)
    q = n * 4 // chunk // world
    st = check(RING, bufs, chunk, max_fuse=64, landing=landing, pool_bytes=1 << 20).rank0
    assert st.reduce_segments == (world - 1) * q
    assert st.reduce_launches == world - 1 and st.reduce_kernel_segments == world - 1
    # the chunks of a gather step merge as well: one copy-kernel launch, or (landing 0) one device copy, per step
    assert st.gather_copies == world - 1
    if landing == 0:
        assert st.landing_copies == world - 1  # a step's messages land in adjacent slots through one device copy
    # Rabenseifner rank 0 of 4: two halving steps over 2 and 1 groups
    st = check(RABEN, bufs, chunk, max_fuse=64, landing=landing, pool_bytes=1 << 20).rank0
    # (staged: the half of the first window that is passed on in the second step goes to send staging,
    # the half that is kept goes to recvbuf, which makes two segments of the first launch)
    assert st.reduce_launches == 2 and st.reduce_segments == 3 * q
    assert st.reduce_kernel_segments == (3 if landing == 3 else 2)
    # 64-byte chunks occupy 256-byte slots: nothing that passes through the pool can merge, while
    # reductions that read and write the callers' buffers only (direct) still do
    q = n * 4 // 64 // world
    st = check(RING, bufs, 64, max_fuse=64, landing=landing, pool_bytes=1 << 20).rank0
    assert st.reduce_launches == world - 1
    if landing == 2:
        assert st.reduce_kernel_segments == world - 1
    elif landing == 3:  # the last step writes recvbuf and reads the sender's slots
        assert st.reduce_kernel_segments == (world - 1) * q
    else:
        assert st.reduce_kernel_segments == (world - 1) * q
    # below the knob's ceiling the knob counts chunks, merged or not
    st = check(RING, bufs, chunk, max_fuse=5, landing=landing, pool_bytes=1 << 20).rank0
    assert st.reduce_launches == (world - 1) * 4  # 16 chunks per step, 5 at a time


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
def test_more_chunks_per_step_than_kernel_segments(landing):
    # 130 chunks per ring step.  Merged they fit one launch; unmerged they need ceil(130 / 64) = 3.
    world, q = 2, 130
    bufs = rand_bufs(world, world * q * 64, seed=6)
    st = check(RING, bufs, 256, max_fuse=64, landing=landing, pool_bytes=1 << 20).rank0
    assert st.reduce_segments == q and st.reduce_launches == 1 and st.reduce_kernel_segments == 1
    # 64-byte chunks in 256-byte slots, three ranks (so that partial sums pass through send staging)
    world = 3
    bufs = rand_bufs(world, world * q * 16, seed=7)
    st = check(RING, bufs, 64, max_fuse=64, landing=landing, pool_bytes=1 << 20).rank0
    assert st.reduce_segments == 2 * q
    if landing == 2:
        assert st.reduce_launches == 2 and st.reduce_kernel_segments == 2
    else:
        assert st.reduce_launches == 6 and st.reduce_kernel_segments == 2 * q
    world = 2
    # a pool of 40 slots is recycled several times within the step: slots come back out of address
    # order, runs break where they do, and the result is the same
    st = check(RING, rand_bufs(world, world * q * 64, seed=8), 256, max_fuse=64, landing=landing, pool_bytes=40 * 256).rank0
    assert st.reduce_segments == q


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
@pytest.mark.parametrize("algo", [RING, RABEN])
def test_replay_launches_the_merged_shapes_of_the_world(algo, landing):
    # the recording log is laid out in the direction the chunks are visited in, so a rank replayed
    # alone merges its chunks exactly as it does among real peers
    world, n, chunk = 4, 4096, 256
    bufs = rand_bufs(world, n, seed=11)
    in_world = check(algo, bufs, chunk, max_fuse=64, landing=landing, pool_bytes=1 << 20).rank0
    rc, recv, out, rep = S.record_replay(algo, bufs, 0, chunk, max_fuse=64, landing=landing, pool_bytes=1 << 20)
    assert rc == 0 and rep.races == 0, (rep.error, rep.first_race)
    assert np.array_equal(O.bits(out), O.bits(recv[0]))
    alone = rep.rank0
    assert (alone.reduce_launches, alone.reduce_kernel_segments, alone.reduce_segments) == \
        (in_world.reduce_launches, in_world.reduce_kernel_segments, in_world.reduce_segments)
    assert alone.gather_copies == in_world.gather_copies


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
def test_recvbuf_off_the_16_byte_grid_keeps_the_phase_margin(landing):
    # recvbuf starting 4 bytes past a 16-byte boundary: every slot keeps its spare bytes, landings
    # share the phase of their target, nothing through the pool merges, results are unchanged
    world, n = 4, 2048
    bufs = rand_bufs(world, n, seed=9)
    backing = [np.empty(n + 1, dtype=np.float32) for _ in range(world)]
    sends = []
    for b, src in zip(backing, bufs):
        b[1:] = src
        sends.append(b[1:])
    assert all(s.ctypes.data % 16 == 4 for s in sends)
    rc, recv, rep = S.allreduce(RING, sends, 256, max_fuse=64, landing=landing, in_place=True, pool_bytes=1 << 20, copy=False)
    assert rc == 0 and rep.races == 0, (rep.error, rep.first_race)
    _, want, _ = O.allreduce(O.RING_GPU, bufs, 256)
    for r in range(world):
        assert np.array_equal(O.bits(recv[r]), O.bits(want[r]))


@pytest.mark.parametrize("landing", [0, 1, 2, 3])
@pytest.mark.parametrize("algo,world", [(RING, 2), (RING, 4), (RING, 5), (RABEN, 4), (RABEN, 8)])
def test_one_rank_replayed_against_recorded_peers(algo, world, landing):
    # a rank run alone against the recording of its incoming traffic must end with the very result
    # it had in the full world, and must launch the same shapes (one step of the algorithm per pass)
    n, chunk = 4096 + 5, 64
    bufs = rand_bufs(world, n, seed=17)
    orc, want, _ = O.allreduce(ORACLE_ALGO[algo], bufs, chunk)
    for rank in sorted({0, world // 2, world - 1}):
        rc, recv, out, rep = S.record_replay(algo, bufs, rank, chunk, landing=landing, replays=2, seed=rank)
        assert rc == 0, rep.error.decode()
        for r in range(world):
            assert np.array_equal(O.bits(recv[r]), O.bits(want[r]))
        assert np.array_equal(O.bits(out), O.bits(want[rank])), "replayed rank %d differs" % rank
        assert rep.races == 0, rep.first_race.decode()
        assert rep.rank0.calls == 2
        if algo == RING:
            q = -(-n // (chunk // 4)) // world  # chunks per group (the last groups may hold one fewer)
            launches_per_call = rep.rank0.reduce_launches // 2
            assert world - 1 <= launches_per_call <= (world - 1) * (-(-(q + 1) // 64))


def test_replay_refuses_a_different_call():
    bufs = rand_bufs(4, 1000, seed=1)
    rc, _, _, rep = S.record_replay(RING, bufs, 1, 40, replays=1)
    assert rc == 0


def pool_rules(chunk_bytes=4096, **env):
    import ctypes as C
    import os
    L = S.lib()
    L.sim_pool_rules.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_ulonglong), C.POINTER(C.c_int), C.POINTER(C.c_int),
                                 C.c_ulonglong]
    keys = ("IBCOMM_NUM_CUDA_STREAM", "IBCOMM_MEMORY_POOL_PRE_ALLOC", "IBCOMM_HIP_MAX_FUSE", "IBCOMM_HIP_LANDING")
    saved = {k: os.environ.get(k) for k in keys}
    try:
        for k in keys:
            os.environ.pop(k, None)
        os.environ["IBCOMM_MEMORY_POOL_PRE_ALLOC"] = "65536"
        for k, v in env.items():
            os.environ[k] = str(v)
        second, block, streams, slots = C.c_int(-1), C.c_ulonglong(0), C.c_int(0), C.c_int(0)
        rc = L.sim_pool_rules(C.byref(second), C.byref(block), C.byref(streams), C.byref(slots), chunk_bytes)
        return rc, second.value, block.value, streams.value, slots.value
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def test_pool_knobs_and_single_controller_rule():
    # defaults and the one-controller-at-a-time rule (memory_pool.h:111-121 -> NOT_SUPPORTED)
    rc, second, block, streams, slots = pool_rules()
    assert rc == 0 and second == 4 and block == 65536 and streams == 8
    # every slot that fits is used: stride = round_up(4096 + 16, 256) = 4352 -> 15 slots in 64 KiB
    assert slots == 65536 // 4352 == 15
    # IBCOMM_NUM_CUDA_STREAM must be in (0, 1024] (memory_pool.h:139-154 -> INVALID_ARGUMENT)
    for bad in ("0", "-1", "1025", "abc"):
        assert pool_rules(IBCOMM_NUM_CUDA_STREAM=bad)[0] == 1
    assert pool_rules(IBCOMM_NUM_CUDA_STREAM="1024")[3] == 1024
    assert pool_rules(IBCOMM_NUM_CUDA_STREAM="64")[3] == 64
    # IBCOMM_MEMORY_POOL_PRE_ALLOC below 4 is refused (memory_pool.h:158-173); the 1 GiB ceiling is lifted
    for bad in ("3", "0", "-5", "x"):
        assert pool_rules(IBCOMM_MEMORY_POOL_PRE_ALLOC=bad)[0] == 1
    assert pool_rules(IBCOMM_MEMORY_POOL_PRE_ALLOC="131072")[2] == 131072
    # this build's own knobs are validated too
    assert pool_rules(IBCOMM_HIP_MAX_FUSE="0")[0] == 1
    assert pool_rules(IBCOMM_HIP_MAX_FUSE="65")[0] == 1
    assert pool_rules(IBCOMM_HIP_LANDING="bogus")[0] == 1
    assert pool_rules(IBCOMM_HIP_LANDING="direct")[0] == 0


def test_working_gpu_memory_knob(capfd):
    # IBCOMM_WORK_GPU_MEMORY_SIZE (ibverbs_communicator_cuda.cpp:12-37): atoi, -1 / unset = 32 MiB, anything
    # else as given; smaller than a chunk -> the reference's warning at a Rabenseifner call and the call
    # goes on (allreduce_cuda_impl.h:372-385); a size nothing could allocate -> CUDA_ERROR (3).
    import os
    world, n = 4, 4096
    bufs = rand_bufs(world, n, seed=11)
    rc, base, _ = S.allreduce(RABEN, bufs, 1024)
    assert rc == 0
    capfd.readouterr()
    warning = "IBCOMM_GPU_WORK_MEMORY_SIZE is smaller than chunk size."
    cases = [("1", True), ("1023", True), ("1024", False), ("garbage", True), ("0", True), ("-1", False), ("33554432", False)]
    try:
        for value, warns in cases:
            os.environ["IBCOMM_WORK_GPU_MEMORY_SIZE"] = value
            for algo in (RABEN, RING):
                want = base if algo == RABEN else S.allreduce(RING, bufs, 1024, max_fuse=1)[1]
                capfd.readouterr()
                rc, got, rep = S.allreduce(algo, bufs, 1024)
                err = capfd.readouterr().err
                assert rc == 0 and rep.races == 0, (value, rep.error)
                assert all(np.array_equal(O.bits(g), O.bits(w)) for g, w in zip(got, want)), value
                assert (warning in err) == (warns and algo == RABEN), (value, algo, err)
                if warning in err:
                    assert err.count(warning) == world and "runtime-reallocation is occured." in err  # once per rank
        os.environ["IBCOMM_WORK_GPU_MEMORY_SIZE"] = "-5"
        rc, _, rep = S.allreduce(RABEN, bufs, 1024)
        assert rc == 3 and b"IBCOMM_WORK_GPU_MEMORY_SIZE" in rep.error
    finally:
        os.environ.pop("IBCOMM_WORK_GPU_MEMORY_SIZE", None)


def test_trace_file_has_the_reference_format(tmp_path):
    # ibcomm/ibverbs_communicator.cpp:157-212: seven lines "name,start_ms,dur_ms,...", scientific notation
    import ctypes as C
    import os
    world, n = 4, 4096
    bufs = rand_bufs(world, n, seed=2)
    recv = [np.empty_like(b) for b in bufs]
    L = S.lib()
    L.sim_trace.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p), C.c_size_t, C.c_int, C.c_char_p,
                            C.POINTER(C.c_ulonglong)]
    pairs = (C.c_ulonglong * 7)()
    path = str(tmp_path / "trace_0.dat")
    os.environ["IBCOMM_CHUNKSIZE"] = "1024"
    os.environ["IBCOMM_MEMORY_POOL_PRE_ALLOC"] = "65536"
    try:
        rc = L.sim_trace(RING, world, (C.c_void_p * world)(*[b.ctypes.data for b in bufs]),
                         (C.c_void_p * world)(*[r.ctypes.data for r in recv]), n, 1, path.encode(), pairs)
    finally:
        os.environ.pop("IBCOMM_CHUNKSIZE")
        os.environ.pop("IBCOMM_MEMORY_POOL_PRE_ALLOC")
    assert rc == 0
    lines = open(path).read().splitlines()
    names = ["received", "reduced", "issue-send", "issue-copy-kernel", "issue-redu-kernel", "issue-recv", "other"]
    # exactly the reference's seven lines: the device-duration lines are written only when device work was
    # timed, and the simulated device keeps no time
    assert [ln.split(",")[0] for ln in lines] == names
    q = n * 4 // 1024 // world  # chunks per group
    want_pairs = {"received": 2 * (world - 1) * q, "reduced": (world - 1) * q, "issue-send": 2 * (world - 1) * q,
                  "issue-redu-kernel": (world - 1) * q, "issue-recv": (world - 1) * q, "other": 2}
    for k, ln in enumerate(lines):
        fields = ln.split(",")
        assert fields[-1] == ""  # every value is followed by a comma
        vals = [float(x) for x in fields[1:-1]]
        assert len(vals) == 2 * pairs[k]
        assert all("e" in x for x in fields[1:-1])  # std::scientific
        starts, durs = vals[0::2], vals[1::2]
        assert all(d >= 0 for d in durs) and starts == sorted(starts) and all(s >= 0 for s in starts)
        if names[k] in want_pairs:
            assert pairs[k] == want_pairs[names[k]], names[k]


def test_point_to_point_over_the_loopback():
    # Send / Recv / SendPoll / RecvPoll / SendWait / RecvWait / Bcast semantics
    # (ibcomm/ibverbs_communicator.cpp:371-606, usage as in tests/sendrecv_test.cpp)
    held = S.lib().sim_p2p()
    names = ["ping", "pong", "second send refused", "second recv refused", "send not complete before pull",
             "one recv completion", "one send completion", "fifo", "oversized message", "bad rank", "bcast"]
    missing = [n for k, n in enumerate(names) if not held >> k & 1]
    assert not missing, missing


def test_failure_handling_is_reported_not_hung():
    # a missing peer, disagreeing ranks, re-entrancy, bad arguments and a mismatched replay all come
    # back as the reference's error codes, and the communicators stay usable
    held = S.lib().sim_failures()
    names = ["missing peer times out", "usable after a timeout", "length mismatch", "second collective refused",
             "p2p refused during a collective", "bad arguments", "replay without recording", "replay of another rank",
             "replay of another call", "replay still works", "an abandoned world refuses collectives until reset",
             "a waiting peer stops when another rank gives up"]
    missing = [n for k, n in enumerate(names) if not held >> k & 1]
    assert not missing, missing


def test_randomised_shapes_and_knobs():
    # random worlds, lengths, chunk sizes, fusion limits, landing modes, stream counts and schedules;
    # every case must be bit-identical to the oracle and free of unordered conflicting accesses
    rng = np.random.default_rng(2024)
    for case in range(60):
        algo = int(rng.integers(0, 2))
        world = int(rng.choice([2, 4, 8, 16])) if algo == RABEN else int(rng.integers(2, 10))
        n = int(rng.integers(world, 6000))
        chunk = None
        if rng.random() < 0.6:
            epc = int(rng.integers(1, max(2, n // (2 * world) + 1)))
            if -(-n // epc) >= 2 * world:
                chunk = 4 * epc
        dtype = [np.float32, np.int32, np.float64][int(rng.integers(0, 3))]
        if chunk is not None and dtype == np.float64:
            chunk *= 2
        bufs = [(np.random.default_rng(case * 100 + r).standard_normal(n) * 50).astype(dtype) for r in range(world)]
        kw = dict(max_fuse=int(rng.integers(1, 65)), landing=int(rng.integers(0, 4)), seed=case,
                  streams=int(rng.integers(1, 9)), pool_bytes=int(rng.choice([512, 4096, 65536])),
                  in_place=bool(rng.random() < 0.2), threaded=bool(rng.random() < 0.15))
        orc, want, _ = O.allreduce(ORACLE_ALGO[algo], bufs, chunk)
        assert orc == 0, (case, algo, world, n, chunk)
        rc, recv, rep = S.allreduce(algo, bufs, chunk, **kw)
        assert rc == 0, (case, rep.error.decode(), algo, world, n, chunk, kw)
        for r in range(world):
            assert np.array_equal(O.bits(recv[r]), O.bits(want[r])), (case, r, algo, world, n, chunk, kw)
        assert rep.unrecorded_waits == 0
        if not kw["threaded"]:
            assert rep.races == 0, (case, rep.first_race.decode(), kw)
