"""The entry point that allocates nothing, ibcomm_hip_world_allreduce_noalloc, against the entry point it is
a variant of, ibcomm_hip_world_allreduce: same inputs through the C ABI, outputs compared bit for bit, on
two calls in a row of which the second is smaller (it finds the first call's staging data in the
library's built-in array).  Also against the CPU oracle, that free device memory does not move across
the calls, that a size beyond the built-in array is refused before anything is enqueued, that the largest
accepted size with thousands of chunks per rank completes, and that the call can be recorded into a HIP
graph and replayed."""
import numpy as np
import pytest

import hip_lib as H
import oracle_lib as O

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
import gpu_util as G  # noqa: E402


def bufs(world, n, seed, scale=1.0):
    return [(np.random.default_rng(seed + r).standard_normal(n) * scale).astype(np.float32) for r in range(world)]


def existing_entry_point(world, algo, send, chunk):
    recv = [G.poisoned_like(t) for t in send]
    with H.World(world) as w:
        assert G.run_world(w, algo, send, recv, chunk) == 0, H.last_error()
    return recv


def no_alloc(world, algo, send, chunk, stream=None):
    recv = [G.poisoned_like(t) for t in send]
    torch.cuda.synchronize()
    with G.env(IBCOMM_CHUNKSIZE=chunk):
        rc = H.world_allreduce_noalloc(world, algo, H.F32, [t.data_ptr() for t in send], [t.data_ptr() for t in recv],
                                       send[0].numel(), stream)
    torch.cuda.synchronize()
    return rc, recv


@pytest.mark.parametrize("algo,world", [(H.RING, 4), (H.RABENSEIFNER, 4), (H.RING, 3), (H.RABENSEIFNER, 8)])
def test_two_calls_in_a_row_match_the_allocating_entry_point(algo, world):
    cases = [(300007, None, 11), (70001, None, 23)]  # the second call is smaller and ragged
    inputs = [G.to_device(bufs(world, n, seed, 0.1)) for n, _, seed in cases]
    want = [existing_entry_point(world, algo, send, chunk) for send, (_, chunk, _) in zip(inputs, cases)]
    got = []
    for send, (_, chunk, _) in zip(inputs, cases):
        rc, recv = no_alloc(world, algo, send, chunk)
        assert rc == 0, H.last_error()
        got.append(recv)
    for g, wnt in zip(got, want):
        for r in range(world):
            assert G.bits_equal(g[r], wnt[r]), "rank %d differs from ibcomm_hip_world_allreduce" % r
    # and the oracle agrees with both
    for (n, chunk, seed), g in zip(cases, got):
        rc, ref, _ = O.allreduce(G.ORACLE_ALGO[algo], bufs(world, n, seed, 0.1), chunk)
        assert rc == 0
        for r in range(world):
            assert np.array_equal(O.bits(g[r].cpu().numpy()), O.bits(ref[r]))


def test_no_device_memory_is_allocated():
    world, n = 4, 262144
    send = G.to_device(bufs(world, n, 5))
    recv = [G.poisoned_like(t) for t in send]
    sp, rp = [t.data_ptr() for t in send], [t.data_ptr() for t in recv]
    # first call on the device: looks up the built-in array (and loads the library's code object)
    assert H.world_allreduce_noalloc(world, H.RING, H.F32, sp, rp, n, None) == 0, H.last_error()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for algo in (H.RING, H.RABENSEIFNER, H.RING):
        assert H.world_allreduce_noalloc(world, algo, H.F32, sp, rp, n, None) == 0, H.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0


def test_on_a_caller_stream_with_chunk_size_and_one_rank():
    world, n = 4, 65536
    send = G.to_device(bufs(world, n, 9))
    want = existing_entry_point(world, H.RING, send, 4096)
    s = torch.cuda.Stream()
    rc, got = no_alloc(world, H.RING, send, 4096, s.cuda_stream)
    assert rc == 0, H.last_error()
    assert all(G.bits_equal(got[r], want[r]) for r in range(world))
    one = G.to_device(bufs(1, 1000, 3))
    rc, got = no_alloc(1, H.RING, one, None)
    assert rc == 0, H.last_error()
    assert G.bits_equal(got[0], one[0])


def test_sizes_beyond_the_built_in_array_are_refused():
    world, n = 8, 4 * 1024 * 1024  # 8 ranks x 16 MiB: twice the buffer per rank is 256 MiB of staging
    send = [torch.zeros(n, device="cuda") for _ in range(world)]
    recv = [torch.full((n,), 7.0, device="cuda") for _ in range(world)]
    rc = H.world_allreduce_noalloc(world, H.RING, H.F32, [t.data_ptr() for t in send], [t.data_ptr() for t in recv], n, None)
    torch.cuda.synchronize()
    assert rc == H.INVALID_ARGUMENT
    assert "built-in" in H.last_error() and "ibcomm_hip_world_allreduce" in H.last_error()
    assert all(bool((t == 7.0).all()) for t in recv)  # nothing was enqueued
    # the reference's argument errors come through unchanged
    small = [torch.zeros(1, device="cuda") for _ in range(2)]
    rc = H.world_allreduce_noalloc(2, H.RING, H.F32, [t.data_ptr() for t in small], [t.data_ptr() for t in small], 1, None)
    assert rc == H.NOT_SUPPORTED
    three = [torch.zeros(64, device="cuda") for _ in range(3)]
    out = [torch.full((64,), 7.0, device="cuda") for _ in range(3)]
    rc = H.world_allreduce_noalloc(3, H.RABENSEIFNER, H.F32, [t.data_ptr() for t in three], [t.data_ptr() for t in out], 64, None)
    torch.cuda.synchronize()
    assert rc == H.NOT_SUPPORTED  # Rabenseifner on a world that is not a power of two


def test_the_largest_accepted_call_with_thousands_of_chunks_completes():
    # 4 ranks x 1 Mi fp32 in 256-byte chunks: 16,384 chunks, 4,096 per ring step; the refusal rule
    # (ranks x 2 x chunks x 512 bytes) comes to exactly the 64 MiB the array holds, so the call is accepted
    # -- and then has to finish: every rank's one block must hold the slots the rule promised.
    world, n, chunk = 4, 1 << 20, 256
    host = bufs(world, n, 31)
    send = G.to_device(host)
    for algo in (H.RING, H.RABENSEIFNER):
        rc, got = no_alloc(world, algo, send, chunk)
        assert rc == 0, H.last_error()
        orc, want, _ = O.allreduce(G.ORACLE_ALGO[algo], host, chunk)
        assert orc == 0
        for r in range(world):
            assert np.array_equal(O.bits(got[r].cpu().numpy()), O.bits(want[r])), (algo, r)
    # one element more per rank and the rule refuses, with recvbufs untouched
    send = G.to_device(bufs(world, n + 64, 32))
    recv = [torch.full((n + 64,), 7.0, device="cuda") for _ in range(world)]
    with G.env(IBCOMM_CHUNKSIZE=chunk):
        rc = H.world_allreduce_noalloc(world, H.RING, H.F32, [t.data_ptr() for t in send], [t.data_ptr() for t in recv], n + 64, None)
    torch.cuda.synchronize()
    assert rc == H.INVALID_ARGUMENT and "built-in" in H.last_error()
    assert all(bool((t == 7.0).all()) for t in recv)


@pytest.mark.parametrize("algo", [H.RING, H.RABENSEIFNER])
def test_recorded_into_a_hip_graph_and_replayed(algo):
    # a caller under stream capture cannot allocate: the call must record as kernel launches only.  The
    # first call on the device (which looks up the built-in array) is made outside the capture; the
    # graph is replayed three times with fresh inputs and other device work in between, and every
    # replay is checked against the eager result of the allocating entry point.
    world, n, chunk = 4, 100003, None
    send = G.to_device(bufs(world, n, 41))
    recv = [G.poisoned_like(t) for t in send]
    sp, rp = [t.data_ptr() for t in send], [t.data_ptr() for t in recv]
    assert H.world_allreduce_noalloc(world, algo, H.F32, sp, rp, n, None) == 0, H.last_error()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s, capture_error_mode="thread_local"):
        rc = H.world_allreduce_noalloc(world, algo, H.F32, sp, rp, n, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, H.last_error()
    for k in range(3):
        host = bufs(world, n, 50 + k)
        for t, h in zip(send, host):
            t.copy_(torch.from_numpy(h))
        for t in recv:
            t.view(torch.uint8).fill_(0x55)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = existing_entry_point(world, algo, send, chunk)
        for r in range(world):
            assert G.bits_equal(recv[r], want[r]), (k, r)
