"""Pins the oracle's four allreduce schedules.

What fixes the answers, independently of oracle/ibcomm_oracle.c:
  * numpy closed forms written in oracle_lib (ring: left fold from the owner of the element's
    chunk group; Rabenseifner: balanced pairwise tree over rank index),
  * a textbook ring reduce-scatter/allgather simulated step by step in Python on tiny inputs,
  * the reference tester's integer known answers: element i of rank p is i*np+p, every rank must
    end with i*np*np + np*(np-1)/2 (tests/allreduce_test.py:66-67),
  * the reference's expected exit codes (tests/allreduce_test.py:102-225).
"""
import numpy as np
import pytest

import oracle_lib as O

RING = (O.RING_CPU, O.RING_GPU)
RABEN = (O.RABEN_CPU, O.RABEN_GPU)


def rand_bufs(world, n, seed=0, dtype=np.float32, scale=1.0):
    return [(np.random.default_rng(seed + r).standard_normal(n) * scale).astype(dtype) for r in range(world)]


def kat_bufs(world, n, dtype=np.int32):
    i = np.arange(n, dtype=np.int64)
    return [(i * world + p).astype(dtype) for p in range(world)]


def kat_answer(world, n, dtype=np.int32):
    i = np.arange(n, dtype=np.int64)
    return (i * world * world + world * (world - 1) // 2).astype(dtype)


def assert_all_ranks(recv, want):
    for r, got in enumerate(recv):
        assert np.array_equal(O.bits(got), O.bits(want)), "rank %d differs" % r


def textbook_ring(sendbufs, chunksize=None):
    """Ring allreduce as in any textbook, one whole group per step, simulated rank by rank."""
    world = len(sendbufs)
    n = sendbufs[0].size
    ranges, groups = O.np_partition(n, sendbufs[0].itemsize, world, chunksize)
    span = [(ranges[g[0]][0], ranges[g[-1]][1]) for g in groups]
    buf = [np.zeros_like(s) for s in sendbufs]  # what each rank currently holds per group
    have = [dict() for _ in range(world)]
    for r in range(world):
        s, e = span[r]
        have[r][r] = sendbufs[r][s:e].copy()
    for step in range(world - 1):          # reduce-scatter: rank r forwards group r-step
        msgs = [(r, (r - step) % world, have[r][(r - step) % world]) for r in range(world)]
        for r, g, data in msgs:
            dst = (r + 1) % world
            s, e = span[g]
            have[dst][g] = data + sendbufs[dst][s:e]      # incoming + own contribution
    for r in range(world):                 # rank r now holds the finished group r+1
        g = (r + 1) % world
        s, e = span[g]
        buf[r][s:e] = have[r][g]
    final = {(r + 1) % world: have[r][(r + 1) % world] for r in range(world)}
    for r in range(world):
        for g in range(world):
            s, e = span[g]
            buf[r][s:e] = final[g]
    return buf


# ------------------------------------------------------------------ closed forms, random fp32

@pytest.mark.parametrize("algo", RING)
@pytest.mark.parametrize("world", [1, 2, 3, 4, 5, 8])
def test_ring_equals_left_fold(algo, world):
    for n, chunk in [(world, None), (2 * world, None), (257, None), (4096 + 3, None), (4096, 64), (1000, 4)]:
        if n < world:
            continue
        if chunk is not None and -(-n // (chunk // 4)) < 2 * world:
            continue
        bufs = rand_bufs(world, n, seed=world * 1000 + n)
        rc, recv, st = O.allreduce(algo, bufs, chunk)
        assert rc == O.OK
        assert_all_ranks(recv, O.np_ring(bufs, chunk))
        assert st.slots_leaked == 0


@pytest.mark.parametrize("algo", RABEN)
@pytest.mark.parametrize("world", [1, 2, 4, 8, 16])
def test_rabenseifner_equals_balanced_tree(algo, world):
    for n, chunk in [(16 * world, None), (257 * world, None), (8192, 64), (4099 * 16, None)]:
        if chunk is not None and -(-n // (chunk // 4)) < 2 * world:
            continue
        bufs = rand_bufs(world, n, seed=world * 77 + n, scale=1e-2)
        rc, recv, st = O.allreduce(algo, bufs, chunk)
        assert rc == O.OK
        assert_all_ranks(recv, O.np_tree(bufs))
        assert st.slots_leaked == 0


def test_rabenseifner_gpu_ragged_lengths():
    # chunked variant partitions with SplitBuffer, so any len >= world works
    for world in (2, 4, 8):
        for n in (world, world + 1, 3 * world + 1, 1021):
            bufs = rand_bufs(world, n, seed=n)
            rc, recv, _ = O.allreduce(O.RABEN_GPU, bufs)
            assert rc == O.OK
            assert_all_ranks(recv, O.np_tree(bufs))


def test_rabenseifner_cpu_ragged_lengths():
    # un-chunked variant: N ranges of ceilDiv(len, N) (allreduce_cpu_impl.h:264-271)
    for world, n in [(2, 7), (4, 10), (4, 1021), (8, 64 + 5)]:
        bufs = rand_bufs(world, n, seed=n)
        rc, recv, _ = O.allreduce(O.RABEN_CPU, bufs)
        assert rc == O.OK
        assert_all_ranks(recv, O.np_tree(bufs))
    # a length for which the reference would build an inverted range is refused by the oracle
    rc, _, _ = O.allreduce(O.RABEN_CPU, rand_bufs(8, 9))
    assert rc == O.NOT_SUPPORTED


def test_order_matters_for_these_inputs():
    # the vectors must be able to tell the two association orders (and numpy's) apart,
    # otherwise bit-exact parity would pin nothing about order
    bufs = rand_bufs(8, 4096, seed=5)
    ring, tree = O.np_ring(bufs), O.np_tree(bufs)
    naive = bufs[0].copy()
    for b in bufs[1:]:
        naive = naive + b
    assert (O.bits(ring) != O.bits(tree)).any()
    assert (O.bits(ring) != O.bits(naive)).any()


@pytest.mark.parametrize("world", [2, 3, 4, 5])
def test_textbook_ring_simulation_agrees(world):
    n = 8 * world + 3
    bufs = rand_bufs(world, n, seed=world)
    want = textbook_ring(bufs)
    for algo in RING:
        rc, recv, _ = O.allreduce(algo, bufs)
        assert rc == O.OK
        for r in range(world):
            assert np.array_equal(O.bits(recv[r]), O.bits(want[r]))


def test_bruteforce_tiny_integer_inputs():
    # exhaustive over small worlds/lengths: with integers every order gives the exact sum
    for world in (2, 3, 4):
        for n in range(world, 4 * world + 6):
            bufs = kat_bufs(world, n)
            for algo in RING + ((O.RABEN_GPU,) if world in (2, 4) else ()):
                rc, recv, _ = O.allreduce(algo, bufs)
                assert rc == O.OK, (algo, world, n)
                assert_all_ranks(recv, kat_answer(world, n))


# ------------------------------------------------------------------ reference tester cases

@pytest.mark.parametrize("algo", RING + RABEN)
def test_1proc(algo):
    # tests/allreduce_test.py:102-108
    bufs = kat_bufs(1, 256)
    rc, recv, _ = O.allreduce(algo, bufs)
    assert rc == O.OK and np.array_equal(recv[0], bufs[0])


@pytest.mark.parametrize("algo", RING)
@pytest.mark.parametrize("world,n", [(1, 2), (2, 4), (3, 6), (5, 10), (2, 2521)])
def test_small_buffer_ring(algo, world, n):
    # tests/allreduce_test.py:110-130
    rc, recv, _ = O.allreduce(algo, kat_bufs(world, n))
    assert rc == O.OK
    assert_all_ranks(recv, kat_answer(world, n))


@pytest.mark.parametrize("world,n,want_rc", [(1, 2, 0), (2, 4, 0), (3, 6, 4), (5, 10, 4), (2, 2521, 0)])
def test_small_buffer_rabenseifner(world, n, want_rc):
    # tests/allreduce_test.py:132-153 (the tester drives the chunked GPU variant)
    rc, recv, _ = O.allreduce(O.RABEN_GPU, kat_bufs(world, n))
    assert rc == want_rc
    if rc == 0:
        assert_all_ranks(recv, kat_answer(world, n))


@pytest.mark.parametrize("chunk", [4, 8, 16, 32, 64, 128])
def test_chunk_size(chunk):
    # tests/allreduce_test.py:177-196
    for algo in RING + (O.RABEN_GPU,):
        rc, recv, _ = O.allreduce(algo, kat_bufs(4, 256), str(chunk))
        assert rc == O.OK
        assert_all_ranks(recv, kat_answer(4, 256))


def test_invalid_error():
    # tests/allreduce_test.py:198-225
    for chunk in ["0", "1", "2", "3", "-128", "1k"]:
        assert O.allreduce(O.RING_GPU, kat_bufs(4, 256), chunk)[0] == O.INVALID_ARGUMENT
    one = [np.ones(1, dtype=np.int32) for _ in range(2)]
    assert O.allreduce(O.RING_GPU, one)[0] == O.NOT_SUPPORTED
    assert O.allreduce(O.RABEN_GPU, one)[0] == O.NOT_SUPPORTED


def test_rabenseifner_copies_before_validating():
    # allreduce_cuda_impl.h:332-351: recvbuf <- sendbuf happens before the power-of-two check
    bufs = kat_bufs(3, 12)
    rc, recv, _ = O.allreduce(O.RABEN_GPU, bufs)
    assert rc == O.NOT_SUPPORTED
    for r in range(3):
        assert np.array_equal(recv[r], bufs[r])


@pytest.mark.parametrize("algo,world", [(O.RING_GPU, 3), (O.RABEN_GPU, 4), (O.RING_CPU, 2)])
def test_basic_large_default_chunks(algo, world):
    # tests/allreduce_test.py:155-175 uses 128 MiB; 16 MiB keeps the CPU suite short
    n = 4 * 1024 * 1024
    rc, recv, _ = O.allreduce(algo, kat_bufs(world, n))
    assert rc == O.OK
    assert_all_ranks(recv, kat_answer(world, n))


def test_baseline_config_1_cpu_ring_exact_integer_sum():
    # 4 ranks, 4,194,304 fp32, integers uniform in [-1000, 1000] stored as float (examples/allreduce.cpp:87-94)
    world, n = 4, 4194304
    bufs = [np.random.default_rng(100 + r).integers(-1000, 1001, n).astype(np.float32) for r in range(world)]
    exact = sum(b.astype(np.int64) for b in bufs).astype(np.float32)
    rc, recv, st = O.allreduce(O.RING_CPU, bufs)
    assert rc == O.OK
    assert_all_ranks(recv, exact)
    assert st.messages == world * 2 * (world - 1) * 4  # 16 chunks, 4 per group, 2(N-1) hops each


# ------------------------------------------------------------------ wire order, pool, closed forms

def expected_ring_wire(world, r, groups, ranges):
    """Order in which rank r puts chunks on the wire to r+1 (both ring variants)."""
    order = []
    for g in [r] + [(r - 1 - i) % world for i in range(world - 1)]:       # own group, then reduced groups
        order += list(reversed(groups[g]))
    for g in [(r - i) % world for i in range(world - 1)]:                # allgather forwards
        if g != (r + 2) % world:
            order += list(reversed(groups[g]))
    return [(ranges[c][0], ranges[c][1] - ranges[c][0]) for c in order]


@pytest.mark.parametrize("algo", RING)
@pytest.mark.parametrize("world,n,chunk", [(2, 64, None), (3, 100, None), (4, 256, 16), (5, 1003, None)])
def test_ring_wire_order(algo, world, n, chunk):
    bufs = kat_bufs(world, n)
    rc, _, _ = O.allreduce(algo, bufs, chunk)
    assert rc == O.OK
    log = O.wire_log(world)
    ranges, groups = O.np_partition(n, 4, world, chunk)
    assert set(log) == {(r, (r + 1) % world) for r in range(world)}
    for r in range(world):
        assert log[(r, (r + 1) % world)] == expected_ring_wire(world, r, groups, ranges)


def test_rabenseifner_gpu_wire_partners_and_volume():
    world, n = 8, 8 * 24
    bufs = kat_bufs(world, n)
    rc, _, _ = O.allreduce(O.RABEN_GPU, bufs)
    assert rc == O.OK
    log = O.wire_log(world)
    # partners differ in exactly one bit
    assert set(log) == {(r, r ^ (1 << b)) for r in range(world) for b in range(3)}
    for r in range(world):
        # bit b is halving step b (window len/2^(b+1)) and doubling step 2-b (same window)
        for b in range(3):
            sent = sum(k for _, k in log[(r, r ^ (1 << b))])
            assert sent == 2 * n // (2 << b)
    # after reduce-scatter rank r owns group world-1-bitrev(r): its first doubling send is that group
    ranges, groups = O.np_partition(n, 4, world)
    for r in range(world):
        bitrev = int(format(r, "03b")[::-1], 2)
        own = world - 1 - bitrev
        first_ag = [m for m in log[(r, r ^ 4)]][-len(groups[own]):]
        assert first_ag == [(ranges[c][0], ranges[c][1] - ranges[c][0]) for c in groups[own]]


def test_pool_growth_and_no_leaks():
    # 64-byte chunks in 1 KiB blocks: strict '<' carving gives 15 slots per block (memory_pool.h:269)
    world, n = 4, 4096
    bufs = kat_bufs(world, n)
    for algo in (O.RING_GPU, O.RABEN_GPU):
        rc, recv, st = O.allreduce(algo, bufs, "64", pool_block_bytes=1024)
        assert rc == O.OK
        assert_all_ranks(recv, kat_answer(world, n))
        assert st.slots_leaked == 0
        assert st.pool_blocks == -(-st.pool_slots_high_water // 15)
    # Rabenseifner keeps allgather slots to the end: the pool grows to most of the buffer (256 chunks here;
    # how many slots are held at once depends on how the rank threads interleave, 159..192 observed)
    assert st.pool_slots_high_water >= (n // 16) // 2


def test_pool_block_not_larger_than_chunk_is_reported():
    # memory_pool.h:229-233: the reference pops an empty queue here; the oracle reports it instead
    rc, _, _ = O.allreduce(O.RING_GPU, kat_bufs(2, 64), "32", pool_block_bytes=32)
    assert rc == 100


def test_closed_form_helpers_agree_with_schedules_and_numpy():
    for world in (2, 3, 4, 8):
        n = 3000 + world
        bufs = rand_bufs(world, n, seed=9 * world)
        rc, out = O.closed_form_ring(bufs)
        assert rc == O.OK and np.array_equal(O.bits(out), O.bits(O.np_ring(bufs)))
        rc, out = O.closed_form_ring(bufs, "64")
        assert rc == O.OK and np.array_equal(O.bits(out), O.bits(O.np_ring(bufs, 64)))
        rc, out = O.closed_form_tree(bufs)
        if world == 3:
            assert rc == O.NOT_SUPPORTED
        else:
            assert rc == O.OK and np.array_equal(O.bits(out), O.bits(O.np_tree(bufs)))
    bufs = rand_bufs(4, 50000, seed=3, dtype=np.float64)
    assert np.array_equal(O.bits(O.closed_form_tree(bufs)[1]), O.bits(O.np_tree(bufs)))
    assert np.array_equal(O.bits(O.closed_form_ring(bufs)[1]), O.bits(O.np_ring(bufs)))


def test_other_dtypes():
    for dtype in (np.float64, np.int64, np.int32):
        bufs = [(np.random.default_rng(r).standard_normal(999) * 100).astype(dtype) for r in range(4)]
        for algo in RING:
            rc, recv, _ = O.allreduce(algo, bufs)
            assert rc == O.OK
            assert_all_ranks(recv, O.np_ring(bufs))
        rc, recv, _ = O.allreduce(O.RABEN_GPU, bufs)
        assert rc == O.OK
        assert_all_ranks(recv, O.np_tree(bufs))
