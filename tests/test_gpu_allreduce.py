"""GPU parity of the allreduce engines through the C ABI, bit-exact against the CPU oracle's
restatement of AllreduceRingCuda / AllreduceRabenseifnerCuda, plus the reference tester's cases
(tests/allreduce_test.py:102-225) and the five benchmark configurations at full size."""
import numpy as np
import pytest

import hip_lib as H
import oracle_lib as O

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
import gpu_util as G  # noqa: E402


def rand_bufs(world, n, seed=0, dtype=np.float32, scale=1.0):
    return [(np.random.default_rng(seed + r).standard_normal(n) * scale).astype(dtype) for r in range(world)]


def kat_bufs(world, n):
    i = np.arange(n, dtype=np.int64)
    return [(i * world + p).astype(np.int32) for p in range(world)]


def kat_answer(world, n):
    i = np.arange(n, dtype=np.int64)
    return (i * world * world + world * (world - 1) // 2).astype(np.int32)


# ------------------------------------------------------------------ engines vs oracle

@pytest.mark.parametrize("landing", [H.LAND_MEMCPY, H.LAND_KERNEL, H.LAND_DIRECT, H.LAND_STAGED])
@pytest.mark.parametrize("fuse", [1, 4, 48, 64])
@pytest.mark.parametrize("world_size", [2, 3, 4, 8])
def test_ring_matches_oracle(world_size, fuse, landing):
    with H.World(world_size) as w:
        w.set_max_fuse(fuse)
        w.set_landing(landing)
        for n, chunk in [(world_size, None), (4 * world_size + 1, None), (100003, None), (65536, 1024), (1 << 20, None)]:
            G.check_against_oracle(w, H.RING, rand_bufs(world_size, n, seed=n), chunk)


@pytest.mark.parametrize("landing", [H.LAND_MEMCPY, H.LAND_KERNEL, H.LAND_DIRECT, H.LAND_STAGED])
@pytest.mark.parametrize("fuse", [1, 4, 48, 64])
@pytest.mark.parametrize("world_size", [2, 4, 8, 16])
def test_rabenseifner_matches_oracle(world_size, fuse, landing):
    with H.World(world_size) as w:
        w.set_max_fuse(fuse)
        w.set_landing(landing)
        for n, chunk in [(world_size, None), (4 * world_size + 3, None), (100003, None), (65536, 1024), (1 << 20, None)]:
            G.check_against_oracle(w, H.RABENSEIFNER, rand_bufs(world_size, n, seed=n + 1, scale=1e-2), chunk)


@pytest.mark.parametrize("algo,world_size", [(H.RING, 33), (H.RING, 64), (H.RABENSEIFNER, 64), (H.RABENSEIFNER, 128)])
def test_many_ranks(algo, world_size):
    with H.World(world_size) as w:
        G.check_against_oracle(w, algo, rand_bufs(world_size, 300007, seed=world_size, scale=0.1), None)
        G.check_against_oracle(w, algo, rand_bufs(world_size, 65536 * 4, seed=world_size + 1, scale=0.1), 1024)


@pytest.mark.parametrize("algo", [H.RING, H.RABENSEIFNER])
def test_one_thread_per_rank_blocking_calls(algo):
    # the reference's usage: every rank inside its own blocking call at the same time.  The calls meet
    # and the last rank to arrive drives the world: eager on the first call of a shape, recorded on the
    # second, replayed afterwards.  Six calls per shape on the same buffers with fresh contents, every
    # one checked against the oracle.
    with H.World(4) as w:
        for n, chunk in ((300001, None), (65536, 4096)):
            send = G.to_device(rand_bufs(4, n, seed=0))
            recv = [G.poisoned_like(t) for t in send]
            for k in range(6):
                host = rand_bufs(4, n, seed=10 * k + 1)
                for t, h in zip(send, host):
                    t.copy_(torch.from_numpy(h))
                for t in recv:
                    t.view(torch.uint8).fill_(0x55)
                assert G.run_world(w, algo, send, recv, chunk, threads=True) == 0, H.last_error()
                orc, want, _ = O.allreduce(G.ORACLE_ALGO[algo], host, chunk)
                assert orc == 0
                for r in range(4):
                    assert np.array_equal(O.bits(recv[r].cpu().numpy()), O.bits(want[r])), (n, k, r)
        eager, captured, replayed = w.graph_counters()
        assert (eager, captured, replayed) == (2, 2, 10), (eager, captured, replayed)
        # fresh buffers every call (no shape is ever seen twice in a row at the same addresses)
        for k in range(3):
            G.check_against_oracle(w, algo, rand_bufs(4, 300001, seed=k), None, threads=True)


@pytest.mark.parametrize("algo", [H.RING, H.RABENSEIFNER])
def test_one_thread_per_rank_each_with_its_own_engine(algo, monkeypatch):
    # IBCOMM_HIP_RENDEZVOUS=0: the rank threads do not meet; each runs its own engine and the ranks
    # exchange messages through the loopback as separate processes would
    monkeypatch.setenv("IBCOMM_HIP_RENDEZVOUS", "0")
    with H.World(4) as w:
        for k in range(3):
            G.check_against_oracle(w, algo, rand_bufs(4, 300001, seed=k), None, threads=True)
        G.check_against_oracle(w, algo, rand_bufs(4, 65536, seed=9), 4096, threads=True)
        assert w.graph_counters() == (0, 0, 0)


@pytest.mark.parametrize("algo", [H.RING, H.RABENSEIFNER])
def test_repeated_calls_and_changing_shapes(algo):
    with H.World(4) as w:
        for k, (n, chunk) in enumerate([(50000, None), (50000, None), (777, None), (1 << 18, 16384), (50000, 1000)]):
            G.check_against_oracle(w, algo, rand_bufs(4, n, seed=k), chunk)


@pytest.mark.parametrize("algo", [H.RING, H.RABENSEIFNER])
def test_in_place(algo):
    with H.World(4) as w:
        G.check_against_oracle(w, algo, rand_bufs(4, 200003, seed=2), None, in_place=True)


@pytest.mark.parametrize("dtype", [np.int32, np.float64, np.int64])
def test_element_types(dtype):
    with H.World(4) as w:
        bufs = [(np.random.default_rng(r).standard_normal(70001) * 1e4).astype(dtype) for r in range(4)]
        G.check_against_oracle(w, H.RING, bufs)
        G.check_against_oracle(w, H.RABENSEIFNER, bufs)


def test_odd_chunk_offsets_keep_vector_path_correct():
    # 2521 elements on 2 ranks -> chunks of 316 and a tail of 309; 1003 on 5 ranks -> chunks of 51
    with H.World(2) as w:
        G.check_against_oracle(w, H.RING, rand_bufs(2, 2521))
        G.check_against_oracle(w, H.RABENSEIFNER, rand_bufs(2, 2521))
    with H.World(5) as w:
        G.check_against_oracle(w, H.RING, rand_bufs(5, 1003))


@pytest.mark.parametrize("seed", range(48))
def test_random_worlds_lengths_chunks_and_buffer_phases(seed):
    # Seeded draws over everything a caller can vary at once: algorithm, world size, odd lengths, chunk size,
    # landing mode, chunks per launch, element type, and the 4-byte phase of every rank's sendbuf and recvbuf
    # (each its own, so the three operands of a reduction can sit at three different phases).
    rng = np.random.default_rng(1000 + seed)
    algo = H.RING if rng.integers(2) else H.RABENSEIFNER
    world = int(rng.choice([2, 3, 4, 5, 7, 8]) if algo == H.RING else rng.choice([2, 4, 8, 16]))
    n = int(rng.integers(world, 300000))
    dtype = [np.float32, np.int32, np.float64][int(rng.integers(3))]
    es = np.dtype(dtype).itemsize
    chunk = None
    if rng.integers(2):
        per = int(rng.integers(1, max(2, n // (2 * world) + 1)))  # elements per chunk, at least 2 * world chunks
        if (n + per - 1) // per >= 2 * world:
            chunk = per * es
    if dtype == np.int32:
        host = [rng.integers(-2**31, 2**31 - 1, n, dtype=np.int64).astype(np.int32) for _ in range(world)]
    else:
        host = [(rng.standard_normal(n) * 10.0 ** float(rng.integers(-3, 3))).astype(dtype) for _ in range(world)]
    tdt = G.TORCH_DT[G.NP_TO_H[np.dtype(dtype)]]
    send_off = [int(rng.integers(4)) for _ in range(world)]
    recv_off = [int(rng.integers(4)) for _ in range(world)]
    send_t = [torch.zeros(n + 8, dtype=tdt, device="cuda") for _ in range(world)]
    recv_t = [torch.full((n + 8,), 85, dtype=tdt, device="cuda") for _ in range(world)]
    for r in range(world):
        send_t[r][send_off[r]:send_off[r] + n] = torch.from_numpy(host[r]).cuda()
    with H.World(world) as w:
        w.set_landing(int(rng.choice([H.LAND_MEMCPY, H.LAND_KERNEL, H.LAND_DIRECT, H.LAND_STAGED])))
        w.set_max_fuse(int(rng.choice([1, 3, 16, 64])))
        torch.cuda.synchronize()
        for call in range(3):  # eager, recorded, replayed
            with G.env(IBCOMM_CHUNKSIZE=chunk):
                rc = w.allreduce_ptrs(algo, G.NP_TO_H[np.dtype(dtype)], [t.data_ptr() + o * es for t, o in zip(send_t, send_off)],
                                      [t.data_ptr() + o * es for t, o in zip(recv_t, recv_off)], n)
            assert rc == 0, "seed %d call %d: %s" % (seed, call, H.last_error())
            torch.cuda.synchronize()
            orc, want, _ = O.allreduce(G.ORACLE_ALGO[algo], host, chunk)
            assert orc == 0
            for r in range(world):
                got = recv_t[r].cpu().numpy()
                o = recv_off[r]
                assert np.array_equal(O.bits(got[o:o + n]), O.bits(want[r])), "seed %d call %d rank %d" % (seed, call, r)
                assert (got[:o] == 85).all() and (got[o + n:] == 85).all(), "seed %d rank %d wrote outside recvbuf" % (seed, r)
                recv_t[r][o:o + n] = 85


@pytest.mark.parametrize("landing", [H.LAND_MEMCPY, H.LAND_KERNEL, H.LAND_DIRECT, H.LAND_STAGED])
@pytest.mark.parametrize("algo,world_size,chunk", [(H.RING, 4, None), (H.RING, 8, 4096), (H.RABENSEIFNER, 8, None)])
def test_graph_replays_match_eager_results(algo, world_size, chunk, landing):
    # the single-thread driver records a call shape on its second use and replays it afterwards;
    # every replay must give what an eager run gives, with other device work in between
    n = 262144 + 3
    with H.World(world_size) as w:
        w.set_graph_mode(1)  # whatever IBCOMM_HIP_GRAPH says
        w.set_landing(landing)
        w.set_max_fuse(5)
        send = [torch.empty(n, device="cuda") for _ in range(world_size)]
        recv = [torch.empty(n, device="cuda") for _ in range(world_size)]
        scratch = torch.zeros(1 << 20, device="cuda")
        for it in range(7):
            host = rand_bufs(world_size, n, seed=100 * it)
            for t, h in zip(send, host):
                t.copy_(torch.from_numpy(h))
            for t in recv:
                t.view(torch.uint8).fill_(0x55)
            scratch.add_(1.0).mul_(0.5)  # unrelated eager work between replays
            assert G.run_world(w, algo, send, recv, chunk) == 0, H.last_error()
            orc, want, _ = O.allreduce(G.ORACLE_ALGO[algo], host, chunk)
            assert orc == 0
            for r in range(world_size):
                assert np.array_equal(O.bits(recv[r].cpu().numpy()), O.bits(want[r])), "call %d rank %d" % (it, r)
        eager, captured, replayed = w.graph_counters()
        if landing == H.LAND_MEMCPY:  # per-message hipMemcpyAsync is never recorded
            assert (eager, captured, replayed) == (7, 0, 0)
        else:
            assert (eager, captured, replayed) == (1, 1, 6)
        # a different shape is a different graph; graph mode 0 goes back to eager issue
        G.check_against_oracle(w, algo, rand_bufs(world_size, 5000, seed=1))
        w.set_graph_mode(0)
        for _ in range(2):
            assert G.run_world(w, algo, send, recv, chunk) == 0
        assert w.graph_counters()[0] == eager + 3


@pytest.mark.parametrize("landing", [H.LAND_KERNEL, H.LAND_DIRECT, H.LAND_STAGED])
@pytest.mark.parametrize("algo,world_size,n,chunk", [(H.RING, 8, 1 << 20, 1 << 17), (H.RING, 5, 300007, None), (H.RABENSEIFNER, 16, 1 << 20, 1 << 14),
                                                     (H.RABENSEIFNER, 4, 70001, None)])
def test_recorded_world_merges_the_ranks_launches(algo, world_size, n, chunk, landing):
    # While a world is recorded the launches the ranks issue for one step are merged into one as far as their
    # memory accesses allow.  Replays of the merged graph, of the unmerged one and the eager call must agree
    # bit for bit with the oracle, on fresh inputs each time; the counters show that merging happened.
    host = [rand_bufs(world_size, n, seed=100 + k, scale=0.1) for k in range(4)]
    results = {}
    for merge in (1, 0):
        with H.World(world_size) as w:
            w.set_landing(landing)
            w.set_merge_mode(merge)
            send = G.to_device(host[0])
            recv = [G.poisoned_like(t) for t in send]
            got = []
            for k in range(4):
                for t, h in zip(send, host[k]):
                    t.copy_(torch.from_numpy(h))
                for t in recv:
                    t.view(torch.uint8).fill_(0x55)
                assert G.run_world(w, algo, send, recv, chunk) == 0, H.last_error()
                got.append([t.clone() for t in recv])
            assert w.graph_counters() == (1, 1, 3)
            collected, recorded = w.merge_counters()
            results[merge] = got
            steps = 2 * (world_size - 1) if algo == H.RING else 2 * (world_size.bit_length() - 1)
            if merge:
                assert collected >= world_size * steps
                if landing != H.LAND_KERNEL:
                    assert recorded == steps, (collected, recorded)  # one launch per step of the algorithm
                else:
                    assert recorded < collected
            else:
                assert (collected, recorded) == (0, 0)
    for k in range(4):
        orc, want, _ = O.allreduce(G.ORACLE_ALGO[algo], host[k], chunk)
        assert orc == 0
        for r in range(world_size):
            assert np.array_equal(O.bits(results[1][k][r].cpu().numpy()), O.bits(want[r])), (k, r)
            assert G.bits_equal(results[1][k][r], results[0][k][r]), (k, r)


@pytest.mark.parametrize("landing", [H.LAND_MEMCPY, H.LAND_KERNEL, H.LAND_DIRECT, H.LAND_STAGED])
@pytest.mark.parametrize("algo,world_size,chunk", [(H.RING, 8, 65536), (H.RING, 3, None), (H.RABENSEIFNER, 8, 65536)])
def test_one_rank_replayed_against_recorded_peers(algo, world_size, chunk, landing):
    # the measured unit of the benchmark: one rank's complete schedule, peers replaced by a recording
    n = (1 << 20) + 7
    host = rand_bufs(world_size, n, seed=31)
    with G.env(IBCOMM_CHUNKSIZE=chunk):
        orc, want, _ = O.allreduce(G.ORACLE_ALGO[algo], host, chunk)
        assert orc == 0
        with H.World(world_size) as w:
            w.set_graph_mode(1)  # whatever IBCOMM_HIP_GRAPH says
            w.set_landing(landing)
            send = G.to_device(host)
            recv = [G.poisoned_like(t) for t in send]
            sp, rp = [t.data_ptr() for t in send], [t.data_ptr() for t in recv]
            for rank in sorted({0, world_size - 1}):
                torch.cuda.synchronize()
                assert w.record(rank, algo, H.F32, sp, rp, n) == 0, H.last_error()
                torch.cuda.synchronize()
                for r in range(world_size):
                    assert np.array_equal(O.bits(recv[r].cpu().numpy()), O.bits(want[r]))
                before = w.graph_counters()
                out = torch.empty_like(send[rank])
                for it in range(5):  # eager, recorded into a graph, replayed
                    out.view(torch.uint8).fill_(0x55)
                    torch.cuda.synchronize()
                    assert w.replay(rank, algo, H.F32, send[rank].data_ptr(), out.data_ptr(), n) == 0, H.last_error()
                    torch.cuda.synchronize()
                    assert np.array_equal(O.bits(out.cpu().numpy()), O.bits(want[rank])), "rank %d replay %d" % (rank, it)
                after = w.graph_counters()
                if landing != H.LAND_MEMCPY:
                    assert after[1] - before[1] >= 1 and after[2] - before[2] >= 3
            # the world still works after replays, and a replay without a matching recording is refused
            assert w.allreduce_ptrs(algo, H.F32, sp, rp, n) == 0
            assert w.replay(1, algo, H.F32, sp[1], rp[1], n) == H.INVALID_ARGUMENT


# ------------------------------------------------------------------ reference tester cases

def run_kat(world_size, algo, n, chunk=None):
    with H.World(world_size) as w:
        send = G.to_device(kat_bufs(world_size, n))
        recv = [G.poisoned_like(t) for t in send]
        rc = G.run_world(w, algo, send, recv, chunk)
        return rc, [t.cpu().numpy() for t in recv]


@pytest.mark.parametrize("algo", [H.RING, H.RABENSEIFNER])
def test_1proc(algo):
    rc, recv = run_kat(1, algo, 256)
    assert rc == 0 and np.array_equal(recv[0], kat_bufs(1, 256)[0])


@pytest.mark.parametrize("world_size,n", [(1, 2), (2, 4), (3, 6), (5, 10), (2, 2521)])
def test_small_buffer_ring(world_size, n):
    rc, recv = run_kat(world_size, H.RING, n)
    assert rc == 0
    for r in recv:
        assert np.array_equal(r, kat_answer(world_size, n))


@pytest.mark.parametrize("world_size,n,want", [(1, 2, 0), (2, 4, 0), (3, 6, 4), (5, 10, 4), (2, 2521, 0)])
def test_small_buffer_rabenseifner(world_size, n, want):
    rc, recv = run_kat(world_size, H.RABENSEIFNER, n)
    assert rc == want
    if rc == 0:
        for r in recv:
            assert np.array_equal(r, kat_answer(world_size, n))


@pytest.mark.parametrize("world_size,algo", [(2, H.RING), (3, H.RING), (4, H.RING), (2, H.RABENSEIFNER), (4, H.RABENSEIFNER)])
def test_basic_128m(world_size, algo):
    n = 128 * 1024 * 1024 // 4
    rc, recv = run_kat(world_size, algo, n)
    assert rc == 0
    want = kat_answer(world_size, n)
    for r in recv:
        assert np.array_equal(r, want)


def test_basic_128m_rabenseifner_three_ranks_not_supported():
    rc, _ = run_kat(3, H.RABENSEIFNER, 1024)
    assert rc == H.NOT_SUPPORTED


@pytest.mark.parametrize("chunk", [4, 8, 16, 32, 64, 128])
def test_chunk_size(chunk):
    rc, recv = run_kat(4, H.RING, 256, chunk)
    assert rc == 0
    for r in recv:
        assert np.array_equal(r, kat_answer(4, 256))


def test_invalid_error():
    for chunk in ["0", "1", "2", "3", "-128", "1k"]:
        rc, _ = run_kat(4, H.RING, 256, chunk)
        assert rc == H.INVALID_ARGUMENT, chunk
    with H.World(2) as w:
        one = G.to_device([np.ones(1, dtype=np.int32)] * 2)
        out = [G.poisoned_like(t) for t in one]
        assert G.run_world(w, H.RING, one, out) == H.NOT_SUPPORTED
        assert G.run_world(w, H.RABENSEIFNER, one, out) == H.NOT_SUPPORTED
        # the world is still usable after a refused call
        G.check_against_oracle(w, H.RING, rand_bufs(2, 1000))


def test_aging_short():
    # tests/allreduce_test.py:227-235 repeats 100 x 128 MiB; a short version of the same idea
    with H.World(4) as w:
        send = G.to_device(kat_bufs(4, 1 << 20))
        want = torch.from_numpy(kat_answer(4, 1 << 20)).cuda()
        for algo in (H.RING, H.RABENSEIFNER):
            for _ in range(25):
                recv = [G.poisoned_like(t) for t in send]
                assert G.run_world(w, algo, send, recv) == 0
                assert all(torch.equal(r, want) for r in recv)


# ------------------------------------------------------------------ benchmark configurations, full size

def device_inputs(world_size, n, seed, kind):
    out = []
    for r in range(world_size):
        g = torch.Generator(device="cuda").manual_seed(seed + r)
        if kind == "normal":
            t = torch.randn(n, device="cuda", generator=g)
        elif kind == "normal1e-2":
            t = torch.randn(n, device="cuda", generator=g) * 1e-2
        elif kind == "uniform":
            t = torch.rand(n, device="cuda", generator=g) * 2 - 1
        elif kind == "ints":
            t = torch.randint(-1000, 1001, (n,), device="cuda", generator=g).float()
        out.append(t)
    return out


def check_ring_on_device(send, recv, chunk):
    world_size, n = len(send), send[0].numel()
    rc, ranges = O.split_buffer(n, 4, world_size, chunk)
    assert rc == 0
    groups = O.rank_to_chunk(len(ranges), world_size)
    for g, cids in enumerate(groups):
        span = (ranges[cids[0]][0], ranges[cids[-1]][1])
        want = G.device_ring_fold(send, span, g)
        for r in range(world_size):
            assert G.bits_equal(recv[r][span[0]:span[1]], want), "rank %d group %d" % (r, g)


def check_stripes_against_oracle(send, recv0, algo, chunk, stripes):
    """Sampled element ranges, recomputed on the host by the oracle's closed form."""
    world_size, n = len(send), send[0].numel()
    rc, ranges = O.split_buffer(n, 4, world_size, chunk)
    groups = O.rank_to_chunk(len(ranges), world_size)
    owner_of_chunk = {c: g for g, cids in enumerate(groups) for c in cids}
    for c in stripes:
        s, e = ranges[c]
        host = [t[s:e].cpu().numpy() for t in send]
        if algo == H.RING:
            g = owner_of_chunk[c]
            rot = host[g:] + host[:g]
            acc = rot[0].copy()
            for x in rot[1:]:
                O.lib().orc_reduce_inplace(O.F32, acc.ctypes.data, x.ctypes.data, acc.size)
            want = acc
        else:
            rc, want = O.closed_form_tree(host)
            assert rc == 0
        assert np.array_equal(O.bits(recv0[s:e].cpu().numpy()), O.bits(want)), "chunk %d" % c


def test_config_2_ring_8_ranks_256mib_full_oracle():
    world_size, n, chunk = 8, 67108864, 8388608
    with H.World(world_size) as w:
        send = device_inputs(world_size, n, 200, "normal")
        recv = [G.poisoned_like(t) for t in send]
        assert G.run_world(w, H.RING, send, recv, chunk) == 0, H.last_error()
        # every element of every rank against the oracle's closed form on the host
        host = [t.cpu().numpy() for t in send]
        rc, want = O.closed_form_ring(host, chunk)
        assert rc == 0
        wbits = O.bits(want)
        for r in range(world_size):
            assert np.array_equal(O.bits(recv[r].cpu().numpy()), wbits), "rank %d" % r
        st = w.stats(0)
        assert st["reduce_elements"] == 58720256 and st["gather_bytes"] == 58720256 * 4


def test_config_3_rabenseifner_16_ranks_resnet50():
    world_size, n, chunk = 16, 102760448, 4194304
    with H.World(world_size) as w:
        send = device_inputs(world_size, n, 300, "normal1e-2")
        recv = [G.poisoned_like(t) for t in send]
        assert G.run_world(w, H.RABENSEIFNER, send, recv, chunk) == 0, H.last_error()
        want = G.device_tree(send, (0, n))
        for r in range(world_size):
            assert G.bits_equal(recv[r], want), "rank %d" % r
        check_stripes_against_oracle(send, recv[0], H.RABENSEIFNER, chunk, [0, 6, 7, 13, 14, 50, 97])
        st = w.stats(0)
        assert st["reduce_elements"] == 90 * 1048576  # rank 0 reduces 90 chunks


@pytest.mark.parametrize("cfg", [2, 3, 4])
def test_full_size_configs_through_the_blocking_per_rank_calls(cfg):
    # The reference's usage at the benchmark's sizes: one thread per rank, each in its blocking call; the calls meet,
    # the world is issued eagerly, recorded with the ranks' launches merged, and replayed.  Four calls on fresh
    # inputs; every element of every rank after every call, with torch's fp32 adds in the reference's order.
    algo, world_size, n, chunk, kind = {2: (H.RING, 8, 67108864, 8388608, "normal"), 3: (H.RABENSEIFNER, 16, 102760448, 4194304, "normal1e-2"),
                                        4: (H.RING, 8, 16777216, 65536, "uniform")}[cfg]
    with G.env(IBCOMM_NUM_CUDA_STREAM=64 if cfg == 4 else None):
        with H.World(world_size) as w:
            send = device_inputs(world_size, n, 500 + cfg, kind)
            recv = [G.poisoned_like(t) for t in send]
            for call in range(4):
                if call:
                    for r, t in enumerate(send):  # fresh contents in the same buffers
                        t.mul_(-0.5).add_(send[(r + 1) % world_size], alpha=0.25)
                    for t in recv:
                        t.view(torch.uint8).fill_(0x55)
                assert G.run_world(w, algo, send, recv, chunk, threads=True) == 0, H.last_error()
                if algo == H.RING:
                    check_ring_on_device(send, recv, chunk)
                else:
                    want = G.device_tree(send, (0, n))
                    for r in range(world_size):
                        assert G.bits_equal(recv[r], want), "call %d rank %d" % (call, r)
            assert w.graph_counters() == (1, 1, 3)
            collected, recorded = w.merge_counters()
            assert 0 < recorded < collected
    if cfg == 4:
        assert recorded == 14  # one launch per step of the ring for all 8 ranks


def test_config_4_ring_small_chunks_64_streams():
    world_size, n, chunk = 8, 16777216, 65536
    with G.env(IBCOMM_NUM_CUDA_STREAM=64):
        with H.World(world_size) as w:
            send = device_inputs(world_size, n, 400, "uniform")
            for fuse in (48, 1):
                w.set_max_fuse(fuse)
                recv = [G.poisoned_like(t) for t in send]
                assert G.run_world(w, H.RING, send, recv, chunk) == 0, H.last_error()
                check_ring_on_device(send, recv, chunk)
            host = [t.cpu().numpy() for t in send]
            rc, want = O.closed_form_ring(host, chunk)
            assert np.array_equal(O.bits(recv[3].cpu().numpy()), O.bits(want))
            assert w.stats(0)["streams_created"] == 64


def test_config_5_ring_32_ranks_2gib_ragged_tail():
    world_size, n, chunk = 32, 536870911, 16777216
    free, _ = torch.cuda.mem_get_info()
    if free < 150 * 2**30:
        pytest.skip("needs ~140 GiB of free HBM")
    with H.World(world_size) as w:
        send = device_inputs(world_size, n, 500, "normal")
        recv = [torch.empty_like(t) for t in send]
        assert G.run_world(w, H.RING, send, recv, chunk) == 0, H.last_error()
        check_ring_on_device(send, recv, chunk)
        check_stripes_against_oracle(send, recv[0], H.RING, chunk, [0, 3, 4, 63, 124, 127])
        check_stripes_against_oracle(send, recv[31], H.RING, chunk, [127])
        del send, recv
    torch.cuda.empty_cache()


def test_config_5_pool_on_the_receive_path_with_4_gib_blocks():
    # The staging pool at the size 288 GB of HBM allows: one 4 GiB block per rank (four times the ceiling
    # the reference puts on IBCOMM_MEMORY_POOL_PRE_ALLOC, memory_pool.h:163), and every partial sum a rank
    # receives landing in a slot of its pool through the copy kernel before it is reduced ("kernel"
    # landing), at the full size of config 5.  In place, so that 64 GiB of buffers and 128 GiB of pools
    # fit side by side; the inputs are generated again afterwards to check the result against.
    world_size, n, chunk = 32, 536870911, 16777216
    free, _ = torch.cuda.mem_get_info()
    if free < 215 * 2**30:
        pytest.skip("needs ~200 GiB of free HBM")
    with G.env(IBCOMM_MEMORY_POOL_PRE_ALLOC=4 << 30):
        with H.World(world_size) as w:
            w.set_landing(H.LAND_KERNEL)
            bufs = device_inputs(world_size, n, 500, "normal")
            assert G.run_world(w, H.RING, bufs, bufs, chunk) == 0, H.last_error()
            stats = [w.stats(r) for r in range(world_size)]
    torch.cuda.empty_cache()
    reduced_chunks = (world_size - 1) * 4  # 31 ring steps of one group of 4 chunks
    for r, s in enumerate(stats):
        assert s["pool_blocks"] == 1 and s["pool_bytes"] == 4 << 30, r
        assert s["slot_count"] == 256  # 4 GiB carved into 16 MiB slots, none wasted (the reference's strict '<' would leave 255)
        assert 4 <= s["slots_high_water"] <= 8, s["slots_high_water"]  # one ring step's chunks, reused first-in first-out
        assert s["reduce_segments"] == reduced_chunks
        # every received partial sum went through the pool; the group that holds the ragged tail is the last one
        assert s["landing_bytes"] in (reduced_chunks * chunk, reduced_chunks * chunk - 4), r
        assert s["landing_copies"] == world_size - 1
    send = device_inputs(world_size, n, 500, "normal")
    check_ring_on_device(send, bufs, chunk)
    check_stripes_against_oracle(send, bufs[0], H.RING, chunk, [0, 63, 127])
    check_stripes_against_oracle(send, bufs[31], H.RING, chunk, [127])
    del send, bufs
    torch.cuda.empty_cache()


@pytest.mark.parametrize("algo,world_size", [(H.RING, 3), (H.RABENSEIFNER, 2)])
def test_more_than_2_to_the_31_elements(algo, world_size):
    # The reference indexes chunk ranges with int (ibverbs_communicator.cpp:676-677) and stops short of
    # 2^31 elements; here offsets are size_t.  int32 data, so that the sum is exact in any order (wrapping).
    n = 2**31 + 4099
    free, _ = torch.cuda.mem_get_info()
    if free < (2 * world_size * 4 * n) + 24 * 2**30:
        pytest.skip("needs about %d GiB of free HBM" % ((2 * world_size * 4 * n >> 30) + 24))
    with H.World(world_size) as w:
        i = torch.arange(n, device="cuda", dtype=torch.int64)
        send = [((i * 2654435761 + r * 40503) & 0xFFFFFFFF).to(torch.int32) for r in range(world_size)]
        del i
        recv = [torch.empty_like(t) for t in send]
        ptrs = lambda ts: [t.data_ptr() for t in ts]  # noqa: E731
        torch.cuda.synchronize()
        assert w.allreduce_ptrs(algo, H.I32, ptrs(send), ptrs(recv), n) == 0, H.last_error()
        torch.cuda.synchronize()
        want = send[0].clone()
        for t in send[1:]:
            want += t
        for r in range(world_size):
            assert torch.equal(recv[r], want), "rank %d" % r
        # the elements on either side of the 2^31 boundary and the ragged tail, on the host
        for lo, hi in ((2**31 - 3, 2**31 + 3), (n - 5, n)):
            host = sum(t[lo:hi].cpu().numpy().astype(np.int64) for t in send).astype(np.int32)
            assert np.array_equal(recv[world_size - 1][lo:hi].cpu().numpy(), host)
        assert w.stats(0)["reduce_elements"] > 2**30
        del send, recv, want
    torch.cuda.empty_cache()


def test_config_1_values_cpu_shape_on_gpu():
    # the CPU configuration's data (integers in [-1000, 1000] as float): any order gives the exact sum
    world_size, n = 4, 4194304
    with H.World(world_size) as w:
        send = device_inputs(world_size, n, 100, "ints")
        recv = [G.poisoned_like(t) for t in send]
        assert G.run_world(w, H.RING, send, recv) == 0
        exact = sum(t.double() for t in send).float()
        for r in range(world_size):
            assert torch.equal(recv[r], exact)


def test_working_gpu_memory_knob_on_the_device(capfd):
    # IBCOMM_WORK_GPU_MEMORY_SIZE (ibverbs_communicator_cuda.cpp:12-37, allreduce_cuda_impl.h:372-385): read when
    # a communicator is created; whatever it says the results are the oracle's, a value below the chunk size
    # draws the reference's warning at a Rabenseifner call and nothing else, a size no allocation could
    # satisfy ends the communicator's creation with CUDA_ERROR (3) as the reference's cudaMalloc would.
    world, n, chunk = 4, 65536, 4096
    bufs = rand_bufs(world, n, seed=77, scale=1e-2)
    warning = "IBCOMM_GPU_WORK_MEMORY_SIZE is smaller than chunk size."
    for value, warns in [("1", True), ("4095", True), ("4096", False), ("not a number", True), (None, False)]:
        with G.env(IBCOMM_WORK_GPU_MEMORY_SIZE=value):
            with H.World(world) as w:
                for algo in (H.RABENSEIFNER, H.RING):
                    capfd.readouterr()
                    G.check_against_oracle(w, algo, bufs, chunk)
                    err = capfd.readouterr().err
                    assert (warning in err) == (warns and algo == H.RABENSEIFNER), (value, algo, err)
                capfd.readouterr()
                G.check_against_oracle(w, H.RABENSEIFNER, bufs, chunk)  # the buffer has "grown": no second warning
                assert warning not in capfd.readouterr().err
    with G.env(IBCOMM_WORK_GPU_MEMORY_SIZE="-4096"):
        with pytest.raises(RuntimeError, match="comm_create: 3 .*IBCOMM_WORK_GPU_MEMORY_SIZE"):
            H.World(world)
