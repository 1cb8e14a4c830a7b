"""Pins orc_split_buffer / orc_rank_to_chunk (ibverbs_communicator.cpp:618-707)."""
import pytest

import oracle_lib as O


def check_invariants(length, itemsize, world, chunksize, ranges):
    if chunksize is None:
        epc = -(-length // (4 * world))
    else:
        epc = int(chunksize) // itemsize
    assert ranges[0][0] == 0 and ranges[-1][1] == length
    for (s0, e0), (s1, e1) in zip(ranges, ranges[1:]):
        assert e0 == s1 and e0 - s0 == epc
    assert 0 < ranges[-1][1] - ranges[-1][0] <= epc
    assert len(ranges) == -(-length // epc) >= world
    groups = O.rank_to_chunk(len(ranges), world)
    flat = [c for g in groups for c in g]
    assert flat == list(range(len(ranges)))
    sizes = [len(g) for g in groups]
    assert max(sizes) - min(sizes) <= 1
    assert sizes == sorted(sizes, reverse=True)
    assert sum(1 for s in sizes if s == max(sizes)) in (len(ranges) % world, world)


def test_bruteforce_default_chunking():
    for world in range(1, 10):
        for length in range(world, 201):
            rc, ranges = O.split_buffer(length, 4, world)
            assert rc == O.OK
            check_invariants(length, 4, world, None, ranges)
            assert ranges == O.np_partition(length, 4, world)[0]
            assert O.rank_to_chunk(len(ranges), world) == O.np_partition(length, 4, world)[1]


def test_bruteforce_env_chunking():
    for itemsize in (4, 8):
        for world in range(1, 7):
            for length in range(world, 120):
                for epc in (1, 2, 3, 5, 8, 16):
                    chunk = epc * itemsize
                    rc, ranges = O.split_buffer(length, itemsize, world, chunk)
                    if -(-length // epc) < 2 * world:
                        assert rc == O.INVALID_ARGUMENT, (length, world, epc)
                    else:
                        assert rc == O.OK
                        check_invariants(length, itemsize, world, chunk, ranges)


def test_too_short_vector():
    # tests/allreduce_test.py:219-225: one element, two processes -> NOT_SUPPORTED
    assert O.split_buffer(1, 4, 2)[0] == O.NOT_SUPPORTED
    for world in range(2, 9):
        assert O.split_buffer(world - 1, 4, world)[0] == O.NOT_SUPPORTED
        assert O.split_buffer(world, 4, world)[0] == O.OK
    # the length is checked before the variable is read (cpp:642 before :650)
    assert O.split_buffer(1, 4, 2, "0")[0] == O.NOT_SUPPORTED


def test_reference_prime_length_case():
    # tests/allreduce_test.py:127-130: 2521 ints on 2 processes, default chunking
    rc, ranges = O.split_buffer(2521, 4, 2)
    assert rc == O.OK
    assert len(ranges) == 8
    assert all(e - s == 316 for s, e in ranges[:-1])
    assert ranges[-1] == (2212, 2521) and 2521 - 2212 == 309
    assert O.rank_to_chunk(8, 2) == [[0, 1, 2, 3], [4, 5, 6, 7]]


@pytest.mark.parametrize("chunk,nchunks", [(4, 256), (8, 128), (16, 64), (32, 32), (64, 16), (128, 8)])
def test_reference_chunk_size_cases(chunk, nchunks):
    # tests/allreduce_test.py:177-196: 1 KiB of ints on 4 processes
    rc, ranges = O.split_buffer(256, 4, 4, str(chunk))
    assert rc == O.OK and len(ranges) == nchunks
    assert all(e - s == chunk // 4 for s, e in ranges)


@pytest.mark.parametrize("chunk", ["0", "1", "2", "3", "-128", "1k", "1024", "256", "abc", ""])
def test_reference_invalid_chunk_sizes(chunk):
    # tests/allreduce_test.py:200-217.  "1k" is read by atoi as 1 (not a multiple of sizeof(int));
    # 256 B gives 4 chunks < 2 * 4; 1024 B gives 1 chunk.
    assert O.split_buffer(256, 4, 4, chunk)[0] == O.INVALID_ARGUMENT


def test_read_chunk_size_atoi_semantics():
    import ctypes as C
    L = O.lib()
    out = C.c_int(0)
    assert L.orc_read_chunk_size(None, C.byref(out)) == 0 and out.value == -1
    assert L.orc_read_chunk_size(b"8388608", C.byref(out)) == 0 and out.value == 8388608
    assert L.orc_read_chunk_size(b"  64 trailing", C.byref(out)) == 0 and out.value == 64
    assert L.orc_read_chunk_size(b"4M", C.byref(out)) == 0 and out.value == 4  # no SI suffixes
    for bad in (b"0", b"-1", b"x", b""):
        assert L.orc_read_chunk_size(bad, C.byref(out)) == O.INVALID_ARGUMENT


def test_baseline_config_shapes():
    # cfg 1: CPU ring, 4 ranks, 4,194,304 fp32, default chunking
    rc, r = O.split_buffer(4194304, 4, 4)
    assert rc == 0 and len(r) == 16 and all(e - s == 262144 for s, e in r)
    assert [len(g) for g in O.rank_to_chunk(16, 4)] == [4] * 4
    # cfg 2: ring, 8 ranks, 256 MiB, 8 MiB chunks
    rc, r = O.split_buffer(67108864, 4, 8, 8388608)
    assert rc == 0 and len(r) == 32 and all(e - s == 2097152 for s, e in r)
    assert [len(g) for g in O.rank_to_chunk(32, 8)] == [4] * 8
    # cfg 3: Rabenseifner, 16 ranks, 102,760,448 fp32, 4 MiB chunks
    rc, r = O.split_buffer(102760448, 4, 16, 4194304)
    assert rc == 0 and len(r) == 98 and all(e - s == 1048576 for s, e in r)
    assert [len(g) for g in O.rank_to_chunk(98, 16)] == [7, 7] + [6] * 14
    # cfg 4: ring, 8 ranks, 64 MiB, 64 KiB chunks
    rc, r = O.split_buffer(16777216, 4, 8, 65536)
    assert rc == 0 and len(r) == 1024 and all(e - s == 16384 for s, e in r)
    assert [len(g) for g in O.rank_to_chunk(1024, 8)] == [128] * 8
    # cfg 5: ring, 32 ranks, 2 GiB - 4 B, 16 MiB chunks, ragged tail
    rc, r = O.split_buffer(536870911, 4, 32, 16777216)
    assert rc == 0 and len(r) == 128
    assert all(e - s == 4194304 for s, e in r[:-1]) and r[-1][1] - r[-1][0] == 4194303
    assert [len(g) for g in O.rank_to_chunk(128, 32)] == [4] * 32
