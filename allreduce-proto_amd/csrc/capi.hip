// extern "C" surface of libibcomm_hip.so; declarations and reference citations are in
// include/ibcomm_hip.h.
#include "ibcomm_hip.h"

#include <chrono>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "backend_hip.hpp"
#include "engine.hpp"
#include "rendezvous.hpp"
#include "world.hpp"

using namespace ibcomm_hip;

static_assert(sizeof(ibcomm_hip_stats) == sizeof(EngineStats), "ibcomm_hip_stats must mirror EngineStats");
static_assert(IBCOMM_HIP_F32 == kF32 && IBCOMM_HIP_I32 == kI32 && IBCOMM_HIP_F64 == kF64 && IBCOMM_HIP_I64 == kI64,
              "dtype codes");
static_assert(IBCOMM_HIP_RING == kRing && IBCOMM_HIP_RABENSEIFNER == kRabenseifner, "algorithm codes");

// A whole-world allreduce recorded as a HIP graph.  The single-threaded driver issues the same
// sequence of copies, launches and event edges every time it is called with the same buffers,
// length, chunk size and knobs, so the sequence is captured once and replayed: the host then costs
// one hipGraphLaunch instead of hundreds of launches and event calls per collective.
struct GraphKey {
  int algo = 0, dtype = 0, landing = 0, fuse = 0, world = 0, replay_rank = -1;
  size_t len = 0;
  std::string chunk_env;
  std::vector<const void*> send;
  std::vector<void*> recv;
  bool operator==(const GraphKey& o) const {
    return algo == o.algo && dtype == o.dtype && landing == o.landing && fuse == o.fuse && world == o.world &&
           replay_rank == o.replay_rank && len == o.len &&
           chunk_env == o.chunk_env && send == o.send && recv == o.recv;
  }
};

struct CachedGraph {
  GraphKey key;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

// Last node of every recorded graph: stores the device's wall clock into pinned host memory, where
// the blocking call that launched the replay is spinning until the word changes.  Seeing the new
// value costs that call a few microseconds less than asking the runtime to synchronise the stream,
// and a clock reading needs no state on the device: replays of one world never overlap (each call
// waits for its own), and two readings that far apart always differ.
//
// What the host may conclude from the new value: every kernel of the replay has finished (this node
// comes after them in the chain, and a kernel boundary completes the stores of the kernel before
// it).  The store is a system-scope release behind a system-scope fence, so that nothing of this
// node is reordered after it either; the results themselves are read by later device work or device
// copies, which the runtime orders after this stream's work in the usual way once the caller
// synchronises or enqueues behind it.  The runtime may retire the launch a moment after the host
// has seen the word; an executable graph is therefore only destroyed after a stream synchronisation.
__global__ void PublishCompletion(uint64_t* host_flag) {
  __threadfence_system();
  __hip_atomic_store(host_flag, static_cast<uint64_t>(wall_clock64()), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

struct ibcomm_hip_fabric {
  explicit ibcomm_hip_fabric(int n) : fabric(n), meet(n) {
    const char* v = getenv("IBCOMM_HIP_GRAPH");
    graph_mode = v ? atoi(v) : 1;
    v = getenv("IBCOMM_HIP_GRAPH_MAX_OPS");
    graph_max_ops = v ? strtoull(v, nullptr, 10) : 4096;
    v = getenv("IBCOMM_HIP_RENDEZVOUS");
    meet_mode = v ? atoi(v) : 1;
    v = getenv("IBCOMM_HIP_MERGE_RANKS");
    merge_mode = v ? atoi(v) : 1;
    // a merged launch stays within what the kernels store with sc1: its parts were on that side
    v = getenv("IBCOMM_HIP_MERGE_MAX_BYTES");
    collector.set_write_limit(v ? strtoull(v, nullptr, 10) : kWriteThroughMaxBytes);
  }
  ~ibcomm_hip_fabric() {
    DropGraphs();
    if (origin) (void)hipStreamDestroy(origin);
    if (replay_flag) (void)hipHostFree(replay_flag);
    if (timer[0]) (void)hipEventDestroy(timer[0]);
    if (timer[1]) (void)hipEventDestroy(timer[1]);
  }
  // A replay returns when its last node has published the completion word, which can be a moment
  // before the runtime has retired the launch: let it, before an executable graph goes away.
  void DropGraphs() {
    if (origin && !graphs.empty()) (void)hipStreamSynchronize(origin);
    for (CachedGraph& g : graphs) {
      if (g.exec) (void)hipGraphExecDestroy(g.exec);
      if (g.graph) (void)hipGraphDestroy(g.graph);
    }
    graphs.clear();
  }
  Fabric<HipBackend> fabric;
  Rendezvous meet;               // where the blocking per-rank calls of this world find each other
  int meet_mode = 1;             // 0 = every rank thread runs its own engine (IBCOMM_HIP_RENDEZVOUS=0)
  LaunchCollector<HipBackend> collector;  // merges the ranks' launches while a world is recorded (merge.hpp)
  int merge_mode = 1;            // 0 = a recorded world keeps one launch per rank and step (IBCOMM_HIP_MERGE_RANKS=0)
  std::mutex mu;                 // guards live_comms and the graph cache against concurrent create / destroy
  int live_comms = 0;
  int graph_mode = 1;            // 0 = always issue eagerly, 1 = capture a call shape on its second use
  hipStream_t origin = nullptr;  // stream the graphs are captured from and replayed on
  uint64_t graph_max_ops = 4096; // call shapes with more copies + launches than this stay eager
  std::vector<CachedGraph> graphs;
  GraphKey last_eager;           // shape of the most recent eagerly issued call
  bool has_last_eager = false;
  uint64_t graph_captures = 0, graph_replays = 0, eager_calls = 0;
  uint64_t* replay_flag = nullptr;   // pinned host memory the last node of a replay writes the device clock to
  uint64_t* replay_flag_device = nullptr;
  uint64_t replays_issued = 0;
  hipEvent_t timer[2] = {nullptr, nullptr};  // around a replay, when the first communicator traces
};

struct ibcomm_hip_comm {
  ibcomm_hip_comm(ibcomm_hip_fabric* f, int n) : owner(f), comm(&f->fabric, n) {}
  ~ibcomm_hip_comm() {
    if (stage_send) (void)hipFree(stage_send);
    if (stage_recv) (void)hipFree(stage_recv);
  }
  ibcomm_hip_fabric* owner;
  Communicator<HipBackend> comm;
  void* stage_send = nullptr;  // device staging for the host-buffer calls, grown on demand
  void* stage_recv = nullptr;
  size_t stage_bytes = 0;
};

struct ibcomm_hip_plan {
  Plan plan;
};

extern "C" {

const char* ibcomm_hip_last_error(void) { return LastErrorBuffer(); }

int ibcomm_hip_fabric_create(int world_size, ibcomm_hip_fabric** out) {
  if (!out) return Fail(kInvalidArgument, "out is null");
  if (world_size < 1 || world_size > 4096) return Fail(kInvalidArgument, "world_size %d out of range", world_size);
  *out = new (std::nothrow) ibcomm_hip_fabric(world_size);
  return *out ? kOk : Fail(kInvalidArgument, "out of host memory");
}

int ibcomm_hip_fabric_destroy(ibcomm_hip_fabric* fabric) {
  if (!fabric) return kOk;
  if (fabric->live_comms) return Fail(kInvalidArgument, "%d communicators still use this fabric", fabric->live_comms);
  delete fabric;
  return kOk;
}

int ibcomm_hip_comm_create(ibcomm_hip_fabric* fabric, int world_size, ibcomm_hip_comm** out) {
  if (!fabric || !out) return Fail(kInvalidArgument, "fabric or out is null");
  ibcomm_hip_comm* c = new (std::nothrow) ibcomm_hip_comm(fabric, world_size);
  if (!c) return Fail(kInvalidArgument, "out of host memory");
  const int rc = c->comm.Init();
  if (rc != kOk) {
    delete c;
    return rc;
  }
  {
    std::lock_guard<std::mutex> lock(fabric->mu);
    fabric->live_comms++;
  }
  *out = c;
  return kOk;
}

int ibcomm_hip_comm_destroy(ibcomm_hip_comm* comm) {
  if (!comm) return kOk;
  comm->comm.Abort();
  if (comm->comm.trace().enabled()) comm->comm.DumpTrace();  // the reference dumps in its destructor (cpp:145-147)
  {
    std::lock_guard<std::mutex> lock(comm->owner->mu);
    comm->owner->DropGraphs();  // recorded graphs point into this communicator's pool
    comm->owner->has_last_eager = false;
    comm->owner->live_comms--;
  }
  delete comm;
  return kOk;
}

int ibcomm_hip_comm_register_myself(ibcomm_hip_comm* comm, int my_rank) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (my_rank < 0 || my_rank >= comm->comm.world_size())
    return Fail(kInvalidArgument, "rank %d outside world of %d", my_rank, comm->comm.world_size());
  comm->comm.RegisterMyself(my_rank);
  return kOk;
}

}  // extern "C"

namespace {

constexpr size_t kMaxCachedGraphs = 16;

uint64_t DeviceOps(const EngineStats& s) { return s.reduce_launches + s.landing_copies + s.gather_copies; }

// Launches a recorded call and returns when its last node has run.  The wait is a spin on the
// pinned word that node writes; if it has not changed within 20 ms (a long collective, or a device
// in trouble) the runtime's own wait takes over and reports whatever went wrong.
int ReplayGraph(ibcomm_hip_fabric* f, CachedGraph& g, Trace* trace) {
  const bool traced = trace && trace->enabled();
  if (traced) {
    if (!f->timer[0]) IBCOMM_HIP_CHECK(hipEventCreate(&f->timer[0]));
    if (!f->timer[1]) IBCOMM_HIP_CHECK(hipEventCreate(&f->timer[1]));
    trace->Mark(Trace::kOther);
    IBCOMM_HIP_CHECK(hipEventRecord(f->timer[0], f->origin));
  }
  const double issued_ms = traced ? trace->NowMs() : 0;
  const volatile uint64_t* flag = f->replay_flag;
  const uint64_t before = *flag;  // no replay of this world is in flight: nothing writes the word until this one ends
  f->replays_issued++;
  hipError_t e = hipGraphLaunch(g.exec, f->origin);
  if (e != hipSuccess) {
    (void)hipStreamSynchronize(f->origin);
    return Fail(kDeviceError, "hipGraphLaunch failed: %s", hipGetErrorString(e));
  }
  if (traced) {
    IBCOMM_HIP_CHECK(hipEventRecord(f->timer[1], f->origin));
    trace->Mark(Trace::kOther);  // end of the span "graph launched"
    trace->Mark(Trace::kOther);  // start of the span "waiting for the graph"
  }
  const auto t0 = std::chrono::steady_clock::now();
  bool seen = false;
  for (uint32_t spins = 1; !seen; spins++) {
    seen = (*flag != before);
    if (!seen && (spins & 0xfff) == 0 &&
        std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > 0.020)
      break;
  }
  __atomic_thread_fence(__ATOMIC_ACQUIRE);
  // Every so often (and whenever the flag was slow) let the runtime retire what it has queued.
  if (!seen || (f->replays_issued & 0x3ff) == 0 || traced) {
    e = hipStreamSynchronize(f->origin);
    if (e != hipSuccess) return Fail(kDeviceError, "hipStreamSynchronize failed after a graph replay: %s", hipGetErrorString(e));
    if (*flag == before) return Fail(kDeviceError, "a graph replay finished without publishing its completion");
  }
  if (traced) {
    trace->Mark(Trace::kOther);
    float ms = 0;
    IBCOMM_HIP_CHECK(hipEventElapsedTime(&ms, f->timer[0], f->timer[1]));
    trace->AddDevice(Trace::kDeviceGraph, issued_ms, ms);
  }
  f->graph_replays++;
  return kOk;
}

// Records one RunWorld() into a graph.  While recording, every rank issues all of its work on the
// one capturing stream, so the graph is a single ordered chain of kernels in the (dependency
// respecting) order the driver issues them.  A chain is what the runtime handles well: recording
// the ranks' own multi-stream, event-linked work gave graphs whose instantiation did not finish.
// Launches at the default fusion are large enough to fill the GPU on their own, so the chain costs
// little overlap and removes the host's launch and event work from every later call.
template <class IssueFn>
int CaptureIssue(ibcomm_hip_fabric* f, std::vector<Communicator<HipBackend>*>& cs, const GraphKey& key, IssueFn issue,
                 CachedGraph* out) {
  if (!f->origin) IBCOMM_HIP_CHECK(hipStreamCreateWithFlags(&f->origin, hipStreamNonBlocking));
  if (!f->replay_flag) {
    IBCOMM_HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&f->replay_flag), 64, hipHostMallocMapped));
    *f->replay_flag = 0;
    IBCOMM_HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&f->replay_flag_device), f->replay_flag, 0));
  }
  for (auto* c : cs) c->pool().OverrideStream(f->origin);
  hipError_t e = hipStreamBeginCapture(f->origin, hipStreamCaptureModeRelaxed);
  int rc = kOk;
  if (e != hipSuccess) {
    rc = Fail(kDeviceError, "hipStreamBeginCapture failed: %s", hipGetErrorString(e));
  } else {
    rc = issue(false);
    if (rc == kOk) {
      hipLaunchKernelGGL(PublishCompletion, dim3(1), dim3(1), 0, f->origin, f->replay_flag_device);
      const hipError_t le = hipGetLastError();
      if (le != hipSuccess) rc = Fail(kDeviceError, "recording the completion node failed: %s", hipGetErrorString(le));
    }
  }
  for (auto* c : cs) c->pool().ClearOverride();
  if (e != hipSuccess) return rc;
  hipGraph_t graph = nullptr;
  e = hipStreamEndCapture(f->origin, &graph);
  if (rc != kOk) {
    if (graph) (void)hipGraphDestroy(graph);
    return rc;
  }
  if (e != hipSuccess || !graph) return Fail(kDeviceError, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(graph);
    return Fail(kDeviceError, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  out->key = key;
  out->graph = graph;
  out->exec = exec;
  f->graph_captures++;
  return kOk;
}

// Eager on the first use of a call shape, recorded on the second, replayed from then on.
// `issue(synchronize)` issues the device work of one call on the communicators in `cs`.
template <class IssueFn>
int IssueCached(ibcomm_hip_fabric* f, std::vector<Communicator<HipBackend>*>& cs, const GraphKey& key, bool may_record,
                IssueFn issue) {
  if (!may_record) {
    f->eager_calls++;
    return issue(true);
  }
  for (CachedGraph& g : f->graphs)
    if (g.key == key) return ReplayGraph(f, g, &cs[0]->trace());

  if (f->has_last_eager && f->last_eager == key) {
    CachedGraph g;
    const int rc = CaptureIssue(f, cs, key, issue, &g);
    if (rc != kOk) {
      for (auto* c : cs) c->Abort();
      f->fabric.Reset();
      f->fabric.EndLockstep();
      f->has_last_eager = false;
      return rc;
    }
    if (f->graphs.size() >= kMaxCachedGraphs) {
      (void)hipStreamSynchronize(f->origin);  // a replay returns on its completion word, possibly before the runtime has retired it
      (void)hipGraphExecDestroy(f->graphs.front().exec);
      (void)hipGraphDestroy(f->graphs.front().graph);
      f->graphs.erase(f->graphs.begin());
    }
    f->graphs.push_back(g);
    return ReplayGraph(f, f->graphs.back(), &cs[0]->trace());  // recording executes nothing: run it once
  }

  f->eager_calls++;
  uint64_t ops_before = 0, ops_after = 0;
  for (auto* c : cs) ops_before += DeviceOps(c->stats());
  const int rc = issue(true);
  for (auto* c : cs) ops_after += DeviceOps(c->stats());
  // Only shapes of a bounded number of device operations are recorded on their next use.
  f->has_last_eager = (rc == kOk) && (ops_after - ops_before <= f->graph_max_ops);
  if (rc == kOk) f->last_eager = key;
  return rc;
}

GraphKey MakeKey(std::vector<Communicator<HipBackend>*>& cs, int algo, int dtype, size_t len, const void* const* sendbufs,
                 void* const* recvbufs, int replay_rank) {
  GraphKey key;
  key.algo = algo;
  key.dtype = dtype;
  key.landing = cs[0]->landing();
  key.fuse = cs[0]->max_fuse();
  key.world = cs[0]->world_size();
  key.replay_rank = replay_rank;
  key.len = len;
  const char* env = getenv("IBCOMM_CHUNKSIZE");  // read on every call, like the reference
  key.chunk_env = env ? env : "";
  key.send.assign(sendbufs, sendbufs + cs.size());
  key.recv.assign(recvbufs, recvbufs + cs.size());
  for (size_t r = 1; r < cs.size(); r++)
    if (cs[r]->landing() != key.landing || cs[r]->max_fuse() != key.fuse) key.fuse = -1 - static_cast<int>(r);  // mixed knobs: never equal
  return key;
}

int CollectWorld(ibcomm_hip_comm* const* comms, int world_size, std::vector<Communicator<HipBackend>*>* cs) {
  cs->resize(world_size);
  for (int r = 0; r < world_size; r++) {
    if (!comms[r]) return Fail(kInvalidArgument, "comms[%d] is null", r);
    if (comms[r]->owner != comms[0]->owner) return Fail(kInvalidArgument, "communicators belong to different fabrics");
    (*cs)[r] = &comms[r]->comm;
  }
  return kOk;
}

// One allreduce of the whole world from the calling thread: eager on the first use of a call shape,
// recorded on the second, replayed from then on.
int WorldAllreduce(ibcomm_hip_fabric* f, std::vector<Communicator<HipBackend>*>& cs, int algo, int dtype,
                   const void* const* sendbufs, void* const* recvbufs, size_t len) {
  const int world_size = static_cast<int>(cs.size());
  // Recording hipMemcpyAsync device-to-device copies into a graph crashed the host process inside
  // the runtime on ROCm 7.2 (gfx950), so the per-message-memcpy landing mode is never recorded.
  const bool may_record = f->graph_mode != 0 && world_size > 1 && cs[0]->landing() != kLandMemcpy;
  const GraphKey key = MakeKey(cs, algo, dtype, len, sendbufs, recvbufs, -1);
  // `synchronize` is false exactly while the call is being recorded: all ranks then issue on the one
  // recording stream, which is where their launches can be merged.
  return IssueCached(f, cs, key, may_record, [&](bool synchronize) {
    LaunchCollector<HipBackend>* merge = (!synchronize && f->merge_mode != 0) ? &f->collector : nullptr;
    return RunWorld<HipBackend>(cs.data(), world_size, algo, dtype, sendbufs, recvbufs, len, synchronize, merge);
  });
}

double TimeLimitSeconds() {
  const char* t = getenv("IBCOMM_HIP_TIMEOUT_S");
  return t ? atof(t) : 120.0;
}

// The blocking per-rank call, the shape of AllreduceRingCuda / AllreduceRabenseifnerCuda.  The
// ranks of a world meet (rendezvous.hpp): the last to arrive runs the collective for all of them
// through the single-thread driver above, so the reference's own entry point gets the recorded
// graph.  With IBCOMM_HIP_RENDEZVOUS=0 every rank thread runs its own engine instead and the
// ranks exchange messages as separate processes would.
int BlockingAllreduce(ibcomm_hip_comm* comm, int algo, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  ibcomm_hip_fabric* f = comm->owner;
  const int world_size = comm->comm.world_size();
  if (world_size == 1 || f->meet_mode == 0) return comm->comm.AllreduceBlocking(algo, dtype, sendbuf, recvbuf, len);
  RankCall call;
  call.comm = &comm->comm;
  call.algo = algo;
  call.dtype = dtype;
  call.sendbuf = sendbuf;
  call.recvbuf = recvbuf;
  call.len = len;
  return f->meet.Arrive(comm->comm.rank(), call, TimeLimitSeconds(), &f->fabric, [f, world_size](const RankCall* calls) {
    std::vector<Communicator<HipBackend>*> cs(world_size);
    std::vector<const void*> sends(world_size);
    std::vector<void*> recvs(world_size);
    for (int r = 0; r < world_size; r++) {
      cs[r] = static_cast<Communicator<HipBackend>*>(calls[r].comm);
      sends[r] = calls[r].sendbuf;
      recvs[r] = calls[r].recvbuf;
    }
    return WorldAllreduce(f, cs, calls[0].algo, calls[0].dtype, sends.data(), recvs.data(), calls[0].len);
  });
}

// Host buffers in, host buffers out: copy up, run the device collective, copy down.
int AllreduceHost(ibcomm_hip_comm* comm, int algo, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  const size_t es = DTypeSize(dtype);
  if (es == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (!sendbuf || !recvbuf) return Fail(kInvalidArgument, "sendbuf and recvbuf must not be null");
  const size_t bytes = len * es;
  if (bytes > comm->stage_bytes) {
    if (comm->stage_send) IBCOMM_HIP_CHECK(hipFree(comm->stage_send));
    if (comm->stage_recv) IBCOMM_HIP_CHECK(hipFree(comm->stage_recv));
    comm->stage_send = comm->stage_recv = nullptr;
    comm->stage_bytes = 0;
    IBCOMM_HIP_CHECK(hipMalloc(&comm->stage_send, bytes));
    IBCOMM_HIP_CHECK(hipMalloc(&comm->stage_recv, bytes));
    comm->stage_bytes = bytes;
  }
  if (bytes) IBCOMM_HIP_CHECK(hipMemcpy(comm->stage_send, sendbuf, bytes, hipMemcpyHostToDevice));
  IBCOMM_RETURN_IF_ERROR(BlockingAllreduce(comm, algo, dtype, comm->stage_send ? comm->stage_send : sendbuf,
                                           comm->stage_recv ? comm->stage_recv : recvbuf, len));
  if (bytes) IBCOMM_HIP_CHECK(hipMemcpy(recvbuf, comm->stage_recv, bytes, hipMemcpyDeviceToHost));
  return kOk;
}

}  // namespace

extern "C" {

int ibcomm_hip_allreduce_ring(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  return BlockingAllreduce(comm, kRing, dtype, sendbuf, recvbuf, len);
}
int ibcomm_hip_allreduce_rabenseifner(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  return BlockingAllreduce(comm, kRabenseifner, dtype, sendbuf, recvbuf, len);
}
int ibcomm_hip_allreduce_ring_host(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  return AllreduceHost(comm, kRing, dtype, sendbuf, recvbuf, len);
}
int ibcomm_hip_allreduce_rabenseifner_host(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  return AllreduceHost(comm, kRabenseifner, dtype, sendbuf, recvbuf, len);
}
int ibcomm_hip_allreduce_ring_f32(ibcomm_hip_comm* c, const float* s, float* r, size_t n) {
  return BlockingAllreduce(c, kRing, kF32, s, r, n);
}
int ibcomm_hip_allreduce_ring_i32(ibcomm_hip_comm* c, const int32_t* s, int32_t* r, size_t n) {
  return BlockingAllreduce(c, kRing, kI32, s, r, n);
}
int ibcomm_hip_allreduce_rabenseifner_f32(ibcomm_hip_comm* c, const float* s, float* r, size_t n) {
  return BlockingAllreduce(c, kRabenseifner, kF32, s, r, n);
}
int ibcomm_hip_allreduce_rabenseifner_i32(ibcomm_hip_comm* c, const int32_t* s, int32_t* r, size_t n) {
  return BlockingAllreduce(c, kRabenseifner, kI32, s, r, n);
}

int ibcomm_hip_world_allreduce(ibcomm_hip_comm* const* comms, int world_size, int algo, int dtype,
                               const void* const* sendbufs, void* const* recvbufs, size_t len) {
  if (!comms || !sendbufs || !recvbufs || world_size < 1) return Fail(kInvalidArgument, "null argument");
  std::vector<Communicator<HipBackend>*> cs;
  IBCOMM_RETURN_IF_ERROR(CollectWorld(comms, world_size, &cs));
  return WorldAllreduce(comms[0]->owner, cs, algo, dtype, sendbufs, recvbufs, len);
}

int ibcomm_hip_world_record(ibcomm_hip_comm* const* comms, int world_size, int rank, int algo, int dtype,
                            const void* const* sendbufs, void* const* recvbufs, size_t len) {
  if (!comms || !sendbufs || !recvbufs || world_size < 2) return Fail(kInvalidArgument, "recording needs a world of at least 2");
  if (rank < 0 || rank >= world_size) return Fail(kInvalidArgument, "rank %d outside world of %d", rank, world_size);
  std::vector<Communicator<HipBackend>*> cs;
  IBCOMM_RETURN_IF_ERROR(CollectWorld(comms, world_size, &cs));
  ibcomm_hip_fabric* f = comms[0]->owner;
  size_t log_bytes = 0;
  bool descending = false;
  IBCOMM_RETURN_IF_ERROR(cs[rank]->RecordingBytes(algo, dtype, len, &log_bytes, &descending));
  f->DropGraphs();  // replay graphs point into the log, which is about to be rewritten (and may move)
  f->has_last_eager = false;
  IBCOMM_RETURN_IF_ERROR(f->fabric.StartRecording(rank, log_bytes, descending));
  f->eager_calls++;
  const int rc = RunWorld<HipBackend>(cs.data(), world_size, algo, dtype, sendbufs, recvbufs, len, true);
  f->fabric.StopRecording();
  return rc;
}

int ibcomm_hip_replay_allreduce(ibcomm_hip_comm* comm, int algo, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  ibcomm_hip_fabric* f = comm->owner;
  const int rank = comm->comm.rank();
  if (!f->fabric.StartReplay(rank))
    return Fail(kInvalidArgument, "no recording for rank %d: call ibcomm_hip_world_record first", rank);
  std::vector<Communicator<HipBackend>*> cs(1, &comm->comm);
  const void* sends[1] = {sendbuf};
  void* recvs[1] = {recvbuf};
  const bool may_record = f->graph_mode != 0 && comm->comm.landing() != kLandMemcpy;
  const GraphKey key = MakeKey(cs, algo, dtype, len, sends, recvs, rank);
  const int rc = IssueCached(f, cs, key, may_record, [&](bool synchronize) {
    return RunAlone<HipBackend>(&comm->comm, algo, dtype, sendbuf, recvbuf, len, synchronize);
  });
  f->fabric.StopReplay();
  return rc;
}

int ibcomm_hip_fabric_graph_counters(ibcomm_hip_fabric* fabric, uint64_t* eager_calls, uint64_t* captures, uint64_t* replays) {
  if (!fabric) return Fail(kInvalidArgument, "fabric is null");
  if (eager_calls) *eager_calls = fabric->eager_calls;
  if (captures) *captures = fabric->graph_captures;
  if (replays) *replays = fabric->graph_replays;
  return kOk;
}

int ibcomm_hip_fabric_merge_counters(ibcomm_hip_fabric* fabric, uint64_t* launches_collected, uint64_t* launches_recorded) {
  if (!fabric) return Fail(kInvalidArgument, "fabric is null");
  if (launches_collected) *launches_collected = fabric->collector.collected();
  if (launches_recorded) *launches_recorded = fabric->collector.issued();
  return kOk;
}

int ibcomm_hip_fabric_set_merge_mode(ibcomm_hip_fabric* fabric, int mode) {
  if (!fabric) return Fail(kInvalidArgument, "fabric is null");
  if (mode != 0 && mode != 1) return Fail(kInvalidArgument, "merge mode must be 0 or 1");
  if (mode != fabric->merge_mode) {
    fabric->DropGraphs();  // recorded under the other setting
    fabric->has_last_eager = false;
  }
  fabric->merge_mode = mode;
  return kOk;
}

int ibcomm_hip_fabric_set_graph_mode(ibcomm_hip_fabric* fabric, int mode) {
  if (!fabric) return Fail(kInvalidArgument, "fabric is null");
  if (mode != 0 && mode != 1) return Fail(kInvalidArgument, "graph mode must be 0 or 1");
  fabric->graph_mode = mode;
  if (mode == 0) fabric->DropGraphs();
  return kOk;
}

int ibcomm_hip_reduce(int dtype, void* dst, const void* a, const void* b, size_t n, void* stream) {
  if (DTypeSize(dtype) == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (n && (!dst || !a || !b)) return Fail(kInvalidArgument, "null operand");
  IBCOMM_HIP_CHECK(LaunchReduce2(dst, a, b, n, dtype, static_cast<hipStream_t>(stream)));
  return kOk;
}

int ibcomm_hip_max_segments(void) { return kMaxSegments; }

int ibcomm_hip_reduce_segments(int dtype, int n_segments, void* const* dst, const void* const* a, const void* const* b,
                               const size_t* len, void* stream) {
  if (DTypeSize(dtype) == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (n_segments < 0 || n_segments > kMaxSegments) return Fail(kInvalidArgument, "at most %d segments per launch", kMaxSegments);
  if (n_segments && (!dst || !a || !b || !len)) return Fail(kInvalidArgument, "null segment table");
  SegmentBatch batch;
  batch.count = n_segments;
  for (int i = 0; i < n_segments; i++) {
    if (len[i] && (!dst[i] || !a[i] || !b[i])) return Fail(kInvalidArgument, "null operand in segment %d", i);
    batch.seg[i] = Segment{dst[i], a[i], b[i], len[i]};
  }
  IBCOMM_HIP_CHECK(LaunchSegments(batch, dtype, static_cast<hipStream_t>(stream)));
  return kOk;
}

int ibcomm_hip_copy_segments(int dtype, int n_segments, void* const* dst, const void* const* src, const size_t* len, void* stream) {
  if (DTypeSize(dtype) == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (n_segments < 0 || n_segments > kMaxSegments) return Fail(kInvalidArgument, "at most %d segments per launch", kMaxSegments);
  if (n_segments && (!dst || !src || !len)) return Fail(kInvalidArgument, "null segment table");
  SegmentBatch batch;
  batch.count = n_segments;
  for (int i = 0; i < n_segments; i++) {
    if (len[i] && (!dst[i] || !src[i])) return Fail(kInvalidArgument, "null operand in segment %d", i);
    batch.seg[i] = Segment{dst[i], src[i], nullptr, len[i]};
  }
  IBCOMM_HIP_CHECK(LaunchSegments(batch, dtype, static_cast<hipStream_t>(stream)));
  return kOk;
}

int ibcomm_hip_describe_launch(int dtype, int n_segments, void* const* dst, const void* const* a, const void* const* b,
                               const size_t* len, int* aligned, int* threads, int* die_local, int* write_through) {
  if (DTypeSize(dtype) == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (n_segments < 0 || n_segments > kMaxSegments) return Fail(kInvalidArgument, "at most %d segments per launch", kMaxSegments);
  if (n_segments && (!dst || !a || !b || !len)) return Fail(kInvalidArgument, "null segment table");
  SegmentBatch batch;
  batch.count = n_segments;
  for (int i = 0; i < n_segments; i++) batch.seg[i] = Segment{dst[i], a[i], b[i], len[i]};
  LaunchShape shape;
  IBCOMM_HIP_CHECK(DescribeLaunch(batch, dtype, &shape));
  if (aligned) *aligned = shape.aligned ? 1 : 0;
  if (threads) *threads = shape.threads;
  if (die_local) *die_local = shape.die_local ? 1 : 0;
  if (write_through) *write_through = shape.write_through ? 1 : 0;
  return kOk;
}

int ibcomm_hip_split_buffer(size_t len, size_t sizeof_element, int world_size, const char* env_chunksize, size_t* starts,
                            size_t* ends, int cap, int* n_ranges) {
  if (!n_ranges || sizeof_element == 0 || world_size < 1 || cap < 0 || (cap > 0 && (!starts || !ends)))
    return Fail(kInvalidArgument, "bad argument");
  std::vector<Range> ranges;
  *n_ranges = 0;
  IBCOMM_RETURN_IF_ERROR(SplitBuffer(len, sizeof_element, world_size, env_chunksize, &ranges));
  *n_ranges = static_cast<int>(ranges.size());
  for (int i = 0; i < *n_ranges && i < cap; i++) {
    starts[i] = ranges[i].begin;
    ends[i] = ranges[i].end;
  }
  return kOk;
}

int ibcomm_hip_rank_to_chunk(int n_ranges, int world_size, int* first_chunk, int* n_chunks) {
  if (n_ranges < 0 || world_size < 1 || !first_chunk || !n_chunks) return Fail(kInvalidArgument, "bad argument");
  std::vector<int> first, count;
  GetRankToChunk(static_cast<size_t>(n_ranges), world_size, &first, &count);
  for (int r = 0; r < world_size; r++) {
    first_chunk[r] = first[r];
    n_chunks[r] = count[r];
  }
  return kOk;
}

int ibcomm_hip_get_exp_of_two(int n) { return GetExpOfTwo(n); }

int ibcomm_hip_plan_create(int algo, int world_size, int rank, size_t len, size_t sizeof_element, const char* env_chunksize,
                           ibcomm_hip_plan** out) {
  if (!out || sizeof_element == 0) return Fail(kInvalidArgument, "bad argument");
  ibcomm_hip_plan* p = new (std::nothrow) ibcomm_hip_plan();
  if (!p) return Fail(kInvalidArgument, "out of host memory");
  const int rc = BuildPlan(algo, world_size, rank, len, sizeof_element, env_chunksize, &p->plan);
  if (rc != kOk) {
    delete p;
    return rc;
  }
  *out = p;
  return kOk;
}

void ibcomm_hip_plan_destroy(ibcomm_hip_plan* plan) { delete plan; }

int ibcomm_hip_plan_counts(const ibcomm_hip_plan* plan, int* n_chunks, int* n_recvs, int* n_sends) {
  if (!plan) return Fail(kInvalidArgument, "plan is null");
  if (n_chunks) *n_chunks = static_cast<int>(plan->plan.part.ranges.size());
  if (n_recvs) *n_recvs = static_cast<int>(plan->plan.recvs.size());
  if (n_sends) *n_sends = static_cast<int>(plan->plan.sends.size());
  return kOk;
}

int ibcomm_hip_plan_range(const ibcomm_hip_plan* plan, int chunk, size_t* begin, size_t* end) {
  if (!plan || chunk < 0 || chunk >= static_cast<int>(plan->plan.part.ranges.size())) return Fail(kInvalidArgument, "bad chunk");
  *begin = plan->plan.part.ranges[chunk].begin;
  *end = plan->plan.part.ranges[chunk].end;
  return kOk;
}

int ibcomm_hip_plan_recv(const ibcomm_hip_plan* plan, int k, int* chunk, int* peer, int* kind) {
  if (!plan || k < 0 || k >= static_cast<int>(plan->plan.recvs.size())) return Fail(kInvalidArgument, "bad index");
  *chunk = plan->plan.recvs[k].chunk;
  *peer = plan->plan.recvs[k].peer;
  *kind = plan->plan.recvs[k].kind;
  return kOk;
}

int ibcomm_hip_plan_send(const ibcomm_hip_plan* plan, int k, int* chunk, int* peer, int* dep) {
  if (!plan || k < 0 || k >= static_cast<int>(plan->plan.sends.size())) return Fail(kInvalidArgument, "bad index");
  *chunk = plan->plan.sends[k].chunk;
  *peer = plan->plan.sends[k].peer;
  *dep = plan->plan.sends[k].dep;
  return kOk;
}

int ibcomm_hip_comm_set_max_fuse(ibcomm_hip_comm* comm, int f) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (f < 1 || f > kMaxSegments) return Fail(kInvalidArgument, "max fuse must be in [1, %d]", kMaxSegments);
  comm->comm.set_max_fuse(f);
  return kOk;
}

int ibcomm_hip_comm_set_landing(ibcomm_hip_comm* comm, int mode) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (mode < kLandMemcpy || mode > kLandStaged) return Fail(kInvalidArgument, "landing mode must be 0, 1, 2 or 3");
  comm->comm.set_landing(mode);
  return kOk;
}

int ibcomm_hip_send(ibcomm_hip_comm* comm, int dest_rank, const void* buf, size_t len, int blocking) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.Send(dest_rank, buf, len, blocking != 0);
}
int ibcomm_hip_recv(ibcomm_hip_comm* comm, int src_rank, void* buf, size_t len, int blocking) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.Recv(src_rank, buf, len, blocking != 0);
}
int ibcomm_hip_send_poll(ibcomm_hip_comm* comm, int dest_rank, int* completed) {
  if (!comm || !completed) return Fail(kInvalidArgument, "null argument");
  bool ok = false;
  const int rc = comm->comm.SendPoll(dest_rank, &ok);
  *completed = ok ? 1 : 0;
  return rc;
}
int ibcomm_hip_recv_poll(ibcomm_hip_comm* comm, int src_rank, int* completed) {
  if (!comm || !completed) return Fail(kInvalidArgument, "null argument");
  bool ok = false;
  const int rc = comm->comm.RecvPoll(src_rank, &ok);
  *completed = ok ? 1 : 0;
  return rc;
}
int ibcomm_hip_send_wait(ibcomm_hip_comm* comm, int dest_rank) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.SendWait(dest_rank);
}
int ibcomm_hip_recv_wait(ibcomm_hip_comm* comm, int src_rank) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.RecvWait(src_rank);
}
int ibcomm_hip_bcast(ibcomm_hip_comm* comm, void* buf, size_t len, int root) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.Bcast(buf, len, root);
}

int ibcomm_hip_comm_set_timer_base(ibcomm_hip_comm* comm) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  comm->comm.trace().SetTimerBase();
  return kOk;
}

int ibcomm_hip_comm_set_trace(ibcomm_hip_comm* comm, int enabled) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  // switching the trace on starts a fresh recording
  if (enabled != 0 && !comm->comm.trace().enabled()) comm->comm.trace().Clear();
  comm->comm.trace().Enable(enabled != 0);
  return kOk;
}

int ibcomm_hip_comm_dump_trace(ibcomm_hip_comm* comm) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (!comm->comm.DumpTrace()) return Fail(kInvalidArgument, "cannot write the trace file");
  return kOk;
}

int ibcomm_hip_comm_stats(ibcomm_hip_comm* comm, ibcomm_hip_stats* out) {
  if (!comm || !out) return Fail(kInvalidArgument, "null argument");
  const EngineStats s = comm->comm.stats();
  memcpy(out, &s, sizeof s);
  return kOk;
}

int ibcomm_hip_comm_reset_stats(ibcomm_hip_comm* comm) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  comm->comm.reset_stats();
  return kOk;
}

}  // extern "C"
