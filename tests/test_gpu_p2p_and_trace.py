"""GPU checks of the transport facade (Send/Recv/Poll/Wait/Bcast over the loopback, host and device
buffers) and of the pipeline trace, through the C ABI."""
import ctypes as C
import os
import threading

import numpy as np
import pytest

import hip_lib as H

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")
import gpu_util as G  # noqa: E402


def test_ping_pong_device_and_host_buffers():
    # tests/sendrecv_test.cpp: non-blocking Send, blocking Recv, then SendWait
    L = H.lib()
    with H.World(2) as w:
        a, b = w.comms
        src = torch.arange(1000, dtype=torch.int32, device="cuda")
        dst = torch.zeros(1000, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        assert L.ibcomm_hip_send(a, 1, src.data_ptr(), 4000, 0) == 0
        assert L.ibcomm_hip_recv(b, 0, dst.data_ptr(), 4000, 1) == 0
        assert L.ibcomm_hip_send_wait(a, 1) == 0
        assert torch.equal(src, dst)
        # device -> host and host -> device
        host = np.zeros(1000, dtype=np.int32)
        assert L.ibcomm_hip_send(b, 0, dst.data_ptr(), 4000, 0) == 0
        assert L.ibcomm_hip_recv(a, 1, host.ctypes.data, 4000, 1) == 0
        assert L.ibcomm_hip_send_wait(b, 0) == 0
        assert np.array_equal(host, np.arange(1000, dtype=np.int32))
        host2 = (host * 3).astype(np.int32)
        assert L.ibcomm_hip_send(a, 1, host2.ctypes.data, 4000, 0) == 0
        assert L.ibcomm_hip_send(a, 1, host2.ctypes.data, 4000, 0) == H.NOT_SUPPORTED  # SendWait must come first
        done = C.c_int(-1)
        assert L.ibcomm_hip_send_poll(a, 1, C.byref(done)) == 0 and done.value == 0
        assert L.ibcomm_hip_recv(b, 0, dst.data_ptr(), 4000, 0) == 0
        assert L.ibcomm_hip_recv_poll(b, 0, C.byref(done)) == 0 and done.value == 1
        assert L.ibcomm_hip_send_poll(a, 1, C.byref(done)) == 0 and done.value == 1
        assert np.array_equal(dst.cpu().numpy(), host2)


def test_bcast_one_thread_per_rank():
    L = H.lib()
    n = 4
    with H.World(n) as w:
        bufs = [torch.full((4096,), float(r), device="cuda") for r in range(n)]
        torch.cuda.synchronize()
        rcs = [None] * n

        def run(r):
            rcs[r] = L.ibcomm_hip_bcast(w.comms[r], bufs[r].data_ptr(), 4096 * 4, 2)

        th = [threading.Thread(target=run, args=(r,)) for r in range(n)]
        [t.start() for t in th]
        [t.join() for t in th]
        assert rcs == [0] * n
        for r in range(n):
            assert torch.equal(bufs[r], torch.full((4096,), 2.0, device="cuda"))


TRACE_NAMES = ["received", "reduced", "issue-send", "issue-copy-kernel", "issue-redu-kernel", "issue-recv", "other"]
DEVICE_NAMES = ["device-redu-kernel", "device-copy-kernel", "device-graph"]


def read_trace(path):
    lines = open(path).read().splitlines()
    # the reference's seven lines; the three device lines follow when device work was timed, else nothing does
    assert [ln.split(",")[0] for ln in lines] in (TRACE_NAMES, TRACE_NAMES + DEVICE_NAMES)
    t = {name: [] for name in DEVICE_NAMES}
    t.update({ln.split(",")[0]: [float(x) for x in ln.split(",")[1:-1]] for ln in lines})
    t["lines"] = len(lines)
    return t


def test_trace_files(tmp_path):
    base = str(tmp_path / "trace")
    with G.env(IBCOMM_TRACE_FILE=base, IBCOMM_CHUNKSIZE=None):
        with H.World(4) as w:
            w.set_graph_mode(0)
            w.set_trace(True)
            send = [torch.randn(1 << 18, device="cuda") for _ in range(4)]
            recv = [torch.empty_like(t) for t in send]
            assert G.run_world(w, H.RING, send, recv) == 0
            w.dump_trace()
    for r in range(4):
        t = read_trace("%s_%d.dat" % (base, r))
        received = t["received"]
        assert len(received) == 2 * 2 * 3 * 4  # (start, duration) x 2(N-1) groups x 4 chunks
        assert all(d >= 0 for d in received[1::2])
        # device durations, one HIP-event pair per launch: N-1 reductions and N-1 gathers per rank, eagerly issued
        assert len(t["device-redu-kernel"]) == 2 * 3 and len(t["device-copy-kernel"]) == 2 * 3 and t["device-graph"] == []
        for name in ("device-redu-kernel", "device-copy-kernel"):
            assert all(0 < d < 50 for d in t[name][1::2]), t[name]        # milliseconds, positive, sane
            assert t[name][0::2] == sorted(t[name][0::2])                   # launches of one rank follow one another
        assert len(t["issue-redu-kernel"]) == len(t["device-redu-kernel"])  # one host issue span per device span
        assert t["lines"] == 10


def test_trace_without_device_work_has_the_reference_seven_lines(tmp_path):
    # point-to-point traffic only: nothing is timed on the device, and the file is what DumpTrace writes
    # in the reference (ibcomm/ibverbs_communicator.cpp:183-212), seven lines
    base = str(tmp_path / "p2p")
    with G.env(IBCOMM_TRACE_FILE=base):
        with H.World(2) as w:
            w.set_trace(True)
            w.dump_trace()
    for r in range(2):
        assert read_trace("%s_%d.dat" % (base, r))["lines"] == 7


def test_trace_of_graph_replays(tmp_path):
    # Every call leaves records: the first is issued eagerly, the second records the graph and replays
    # it, the others replay.  A replay does no host-side pipeline work; what it leaves is two "other"
    # spans (the launch call, the wait for the completion flag) and one device-graph duration.
    base = str(tmp_path / "replay")
    calls = 6
    with G.env(IBCOMM_TRACE_FILE=base, IBCOMM_CHUNKSIZE=None):
        with H.World(4) as w:
            w.set_graph_mode(1)
            w.set_trace(True)
            send = [torch.randn(1 << 18, device="cuda") for _ in range(4)]
            recv = [torch.empty_like(t) for t in send]
            want = None
            for _ in range(calls):
                assert G.run_world(w, H.RING, send, recv) == 0
                if want is None:
                    want = [t.clone() for t in recv]
                assert all(G.bits_equal(a, b) for a, b in zip(recv, want))
            assert w.graph_counters() == (1, 1, calls - 1)
            w.dump_trace()
    t0 = read_trace(base + "_0.dat")
    assert len(t0["device-graph"]) == 2 * (calls - 1)
    assert all(0 < d < 50 for d in t0["device-graph"][1::2])
    assert len(t0["device-redu-kernel"]) == 2 * 3  # the eager first call only; recording a graph times nothing
    # Begin and Finish of the eager call and of the recorded one, then two spans per replay
    assert len(t0["other"]) == 2 * (2 + 1 + 2 * (calls - 1)), len(t0["other"])
    t1 = read_trace(base + "_1.dat")
    assert t1["device-graph"] == []  # the replay belongs to the world; it is booked on rank 0's trace


@pytest.mark.parametrize("algo,oracle_algo,world_size", [(H.RING, 0, 4), (H.RING, 0, 3), (H.RABENSEIFNER, 1, 4), (H.RABENSEIFNER, 1, 8)])
def test_host_buffer_calls_match_the_reference_cpu_path(algo, oracle_algo, world_size):
    # AllreduceRing<T> / AllreduceRabenseifner<T> on host memory (ibcomm/allreduce_cpu_impl.h), bit-exact
    # against the oracle's restatement of those CPU routines (O.RING_CPU = 0, O.RABEN_CPU = 1)
    import oracle_lib as O
    n = 100003 if algo == H.RING else 8 * 12500 + 3 * world_size  # the CPU Rabenseifner needs ceil(n/N)*(N-1) <= n
    host = [np.random.default_rng(50 + r).standard_normal(n).astype(np.float32) for r in range(world_size)]
    orc, want, _ = O.allreduce(oracle_algo, host)
    assert orc == 0
    out = [np.full(n, 7.0, dtype=np.float32) for _ in range(world_size)]
    with G.env(IBCOMM_CHUNKSIZE=None):
        with H.World(world_size) as w:
            for _ in range(2):
                rcs, msgs = w.allreduce_threads(algo, H.F32, [h.ctypes.data for h in host], [o.ctypes.data for o in out], n, host=True)
                assert rcs == [0] * world_size, msgs
                for r in range(world_size):
                    assert np.array_equal(O.bits(out[r]), O.bits(want[r])), "rank %d" % r


@pytest.mark.parametrize("world_size,n", [(4, 5), (8, 13), (8, 1001), (4, 4)])
def test_host_rabenseifner_lengths_the_reference_cannot_split(world_size, n):
    # The reference's CPU Rabenseifner cuts the buffer into N ranges of ceilDiv(len, N) elements
    # (allreduce_cpu_impl.h:264-271).  When (N-1) * ceilDiv(len, N) > len (5 elements on 4 ranks: ranges
    # (0,2) (2,4) (4,5) (6,5)) a range is inverted and its size_t lengths wrap; the oracle refuses such
    # input.  Here the host call goes through SplitBuffer like the device path, so every len >= N works,
    # and the result is the balanced tree, which does not depend on how the buffer is cut.
    import oracle_lib as O
    host = [np.random.default_rng(70 + r).standard_normal(n).astype(np.float32) for r in range(world_size)]
    if (-(-n // world_size)) * (world_size - 1) > n:
        assert O.allreduce(O.RABEN_CPU, host)[0] == O.NOT_SUPPORTED
    rc, want = O.closed_form_tree(host)
    assert rc == 0
    out = [np.full(n, 7.0, dtype=np.float32) for _ in range(world_size)]
    with G.env(IBCOMM_CHUNKSIZE=None):
        with H.World(world_size) as w:
            rcs, msgs = w.allreduce_threads(H.RABENSEIFNER, H.F32, [h.ctypes.data for h in host], [o.ctypes.data for o in out], n, host=True)
            assert rcs == [0] * world_size, msgs
    for r in range(world_size):
        assert np.array_equal(O.bits(out[r]), O.bits(want)), "rank %d" % r

