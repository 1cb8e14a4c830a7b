// The chunk-pipelined allreduce engine of one emulated rank.
//
// Counterpart of IBVerbsCommunicator::AllreduceRingCuda<T> and
// AllreduceRabenseifnerCuda<T> (ibcomm/allreduce_cuda_impl.h:35-301, 326-717).
// The reference runs each as a host state machine that polls the network and
// cudaStreamQuery, and moves every chunk host<->device twice.  Here the whole
// collective is issued as stream-ordered device work:
//
//   * a Plan (plan.hpp) lists, in the reference's wire order, the messages
//     this rank consumes and emits;
//   * Progress() walks the plan without ever waiting for the device: it posts
//     every send whose data has been *enqueued*, takes every message a peer
//     has posted, and launches one segment kernel over all chunks taken in
//     this pass:
//         result[c] = incoming + sendbuf[c]     ring steps, first halving step
//         result[c] = incoming + recvbuf[c]     later halving steps
//     By default ("staged") the kernel reads the incoming partial sum where
//     the sender staged it, and writes result[c] into a pool slot of its own
//     when the sum is only going to be forwarded, into recvbuf when this rank
//     keeps it: the reference's copy to the staging slot (:134-135, :515-516)
//     is the kernel's store.  The other modes first land each message in a
//     local pool slot, by one copy-kernel launch per pass or one
//     hipMemcpyAsync per message.  Finished chunks of the gather phase land
//     straight in recvbuf and are forwarded from there, so they cost one copy
//     instead of the reference's three (:129-135, :528-529);
//   * ordering between ranks, streams and slot reuse is carried by events, so
//     the same sequence of calls can be recorded into a graph.
//
// Summation order is untouched: each element still sees exactly the adds the
// reference performs, one IEEE add per hop, in the reference's association.
//
// A Communicator is driven either by its own thread calling
// AllreduceBlocking() (one thread per emulated rank, like one process per rank
// in the reference), or cooperatively by RunWorld() (world.hpp), which steps
// all ranks from one thread.
#pragma once

#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <deque>
#include <string>
#include <thread>
#include <utility>
#include <vector>

#include "loopback.hpp"
#include "memory_pool.hpp"
#include "merge.hpp"
#include "plan.hpp"
#include "segments.hpp"
#include "status.hpp"
#include "trace.hpp"

namespace ibcomm_hip {

enum LandingMode : int {
  kLandMemcpy = 0,  // one asynchronous device copy per message into a pool slot
  kLandKernel = 1,  // all messages of a pass land through one copy-kernel launch
  kLandDirect = 2,  // no landing: the reduction reads the sender's buffer in place
  kLandStaged = 3,  // like direct, and a partial sum that is only forwarded is written by the reduction
                    // into a pool slot (send staging) instead of recvbuf; the next rank reads it there
};

struct EngineStats {
  uint64_t calls = 0;
  uint64_t reduce_launches = 0;
  uint64_t reduce_segments = 0;
  uint64_t reduce_elements = 0;
  uint64_t landing_copies = 0;  // device copies or copy-kernel launches into pool slots
  uint64_t landing_bytes = 0;
  uint64_t gather_copies = 0;   // copies (or copy-kernel launches) of finished chunks into recvbuf
  uint64_t gather_bytes = 0;
  uint64_t messages_sent = 0;
  uint64_t messages_received = 0;
  uint64_t events_recorded = 0;
  uint64_t stream_waits = 0;
  uint64_t streams_created = 0;
  uint64_t slots_high_water = 0;
  uint64_t slot_count = 0;
  uint64_t pool_blocks = 0;
  uint64_t pool_bytes = 0;
  uint64_t progress_passes = 0;
  uint64_t reduce_kernel_segments = 0;  // segments the reduction launches carried after merging contiguous chunks
  uint64_t largest_reduce_elements = 0;  // the reduction launch with the most elements: its elements ...
  uint64_t largest_reduce_kernel_segments = 0;  // ... and its kernel segments
  uint64_t largest_reduce_launches = 0;  // how many reduction launches had that many elements
};

template <class B>
class Communicator {
 public:
  using Stream = typename B::Stream;
  using Event = typename B::Event;
  using Message = typename Fabric<B>::Message;

  Communicator(Fabric<B>* fabric, int world_size) : fabric_(fabric), world_size_(world_size) {}
  Communicator(const Communicator&) = delete;
  Communicator& operator=(const Communicator&) = delete;
  ~Communicator() {
    controller_.Release();
    for (auto& arena : events_)
      for (auto e : arena) B::EventDestroy(e);
    for (auto t : timers_) B::TimerDestroy(t);
  }

  // PrepareMemoryPool (ibcomm/ibverbs_communicator_cuda.cpp:26-37) plus this build's knobs.
  int Init(size_t pool_block_bytes = 0) {
    if (world_size_ < 1 || world_size_ != fabric_->world_size())
      return Fail(kInvalidArgument, "world size %d does not match the fabric's %d", world_size_, fabric_->world_size());
    IBCOMM_RETURN_IF_ERROR(pool_.Init(pool_block_bytes));
    const char* v = getenv("IBCOMM_HIP_MAX_FUSE");
    max_fuse_ = v ? atoi(v) : kMaxSegments;
    if (max_fuse_ < 1 || max_fuse_ > kMaxSegments)
      return Fail(kInvalidArgument, "IBCOMM_HIP_MAX_FUSE must be in [1, %d]", kMaxSegments);
    v = getenv("IBCOMM_HIP_LANDING");
    if (!v || !strcmp(v, "staged")) landing_ = kLandStaged;
    else if (!strcmp(v, "kernel")) landing_ = kLandKernel;
    else if (!strcmp(v, "memcpy")) landing_ = kLandMemcpy;
    else if (!strcmp(v, "direct")) landing_ = kLandDirect;
    else return Fail(kInvalidArgument, "IBCOMM_HIP_LANDING must be memcpy, kernel, direct or staged, not '%s'", v);
    // The working GPU buffer (IBCOMM_WORK_GPU_MEMORY_SIZE, ibverbs_communicator_cuda.cpp:12-37) held
    // the second operand of the Rabenseifner kernel.  Here that kernel reads the incoming message
    // where it lies, so no such buffer is allocated.  The variable keeps its meaning as far as a
    // caller can observe it: read with atoi, unset or -1 is 32 MiB, anything else is taken as given
    // (text that is no number reads as 0), a size no allocation could satisfy fails as the
    // reference's cudaMalloc does (CUDA_ERROR), and a size below the chunk size draws the
    // reference's warning at the first Rabenseifner call (Begin) instead of an error.
    v = getenv("IBCOMM_WORK_GPU_MEMORY_SIZE");
    work_gpu_memory_size_ = v ? atoi(v) : -1;
    if (work_gpu_memory_size_ == -1) work_gpu_memory_size_ = 32ll << 20;
    if (work_gpu_memory_size_ < 0)
      return Fail(kDeviceError, "IBCOMM_WORK_GPU_MEMORY_SIZE=%s: no working buffer of that size can be allocated", v);
    v = getenv("IBCOMM_HIP_TRACE");
    trace_.Enable(v && atoi(v) != 0);
    return kOk;
  }

  Trace& trace() { return trace_; }
  // DumpTrace (ibverbs_communicator.cpp:183-212): ${IBCOMM_TRACE_FILE:-ibcomm_trace}_<rank>.dat
  bool DumpTrace() const {
    const char* base = getenv("IBCOMM_TRACE_FILE");
    return trace_.Dump(std::string(base ? base : "ibcomm_trace") + "_" + std::to_string(rank_) + ".dat");
  }

  void RegisterMyself(int rank) {  // ibverbs_communicator.cpp:355-357
    rank_ = rank;
    plan_cached_ = false;
  }
  int rank() const { return rank_; }
  int world_size() const { return world_size_; }
  MemoryPool<B>& pool() { return pool_; }
  Fabric<B>* fabric() { return fabric_; }
  // While set, launches go to the collector instead of the stream (merge.hpp): for the recording of a
  // whole world, where every rank issues on the one recording stream.
  void set_collector(LaunchCollector<B>* c) { collector_ = c; }
  void set_max_fuse(int f) { max_fuse_ = f < 1 ? 1 : (f > kMaxSegments ? kMaxSegments : f); }
  void set_landing(int mode) { landing_ = mode; }
  int landing() const { return landing_; }
  int max_fuse() const { return max_fuse_; }
  long long work_gpu_memory_size() const { return work_gpu_memory_size_; }

  EngineStats stats() {
    EngineStats s = stats_;
    s.streams_created = pool_.streams_created();
    s.pool_blocks = pool_.blocks();
    s.pool_bytes = pool_.bytes_allocated();
    return s;
  }
  void reset_stats() { stats_ = EngineStats(); }

  // ---- one collective: Begin, Progress until finished, Finish ------------------------------------

  int Begin(int algo, int dtype, const void* sendbuf, void* recvbuf, size_t len_elements) {
    TraceScope scope(&trace_, Trace::kOther);
    if (active_) return Fail(kNotSupported, "an allreduce is already in progress on this communicator");
    if (fabric_->poisoned())
      return Fail(kTransportError, "this loopback world was abandoned after an earlier failure (%s); create a new one", fabric_->poison_reason());
    if (rank_ < 0 || rank_ >= world_size_) return Fail(kInvalidArgument, "RegisterMyself has not been called");
    es_ = DTypeSize(dtype);
    if (es_ == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
    if (!sendbuf || !recvbuf) return Fail(kInvalidArgument, "sendbuf and recvbuf must not be null");
    dtype_ = dtype;
    sendbuf_ = static_cast<const char*>(sendbuf);
    recvbuf_ = static_cast<char*>(recvbuf);
    const size_t bytes = len_elements * es_;
    // The reference's ring cannot run in place (its landing copy overwrites the operand it still
    // has to add, allreduce_cuda_impl.h:129-133).  This engine can, as long as the two buffers
    // are the very same range; anything in between is refused.
    in_place_ = (sendbuf_ == recvbuf_);
    if (!in_place_ && sendbuf_ < recvbuf_ + bytes && recvbuf_ < sendbuf_ + bytes)
      return Fail(kInvalidArgument, "sendbuf and recvbuf overlap partially");

    // IBCOMM_CHUNKSIZE is read on every call (ibverbs_communicator.cpp:619-634); the plan it leads to
    // is kept for as long as the call shape stays the same.
    const char* chunk_env = getenv("IBCOMM_CHUNKSIZE");
    const std::string chunk_text = chunk_env ? std::string("=") + chunk_env : std::string();
    if (!(plan_cached_ && plan_.algo == algo && plan_len_ == len_elements && plan_es_ == es_ && plan_chunk_env_ == chunk_text)) {
      plan_cached_ = false;
      IBCOMM_RETURN_IF_ERROR(BuildPlan(algo, world_size_, rank_, len_elements, es_, chunk_env, &plan_));
      plan_len_ = len_elements;
      plan_es_ = es_;
      plan_chunk_env_ = chunk_text;
      plan_cached_ = true;
    }
    stats_.calls++;
    // Events of the call before last are free again: a peer trails this rank by at most one
    // collective, because finishing a collective needs every peer to have taken part in it.
    arena_ ^= 1;
    event_cursor_ = 0;
    pool_.RewindStreams();
    next_send_ = next_recv_ = 0;
    outstanding_sends_ = 0;
    finished_ = false;
    pull_events_.clear();

    if (world_size_ == 1) {  // allreduce_cuda_impl.h:40-46
      if (!in_place_ && bytes) {
        Stream s;
        IBCOMM_RETURN_IF_ERROR(pool_.NextStream(&s));
        IBCOMM_RETURN_IF_ERROR(DeviceCopy(recvbuf_, sendbuf_, bytes, s));
        stats_.gather_copies++;
        stats_.gather_bytes += bytes;
      }
      finished_ = true;
      active_ = true;
      return kOk;
    }

    const size_t chunks = plan_.part.ranges.size();
    recv_done_.assign(plan_.recvs.size(), OpState());
    staged_.assign(plan_.recvs.size(), nullptr);
    chunk_last_.assign(chunks, OpState());
    chunk_unconsumed_.assign(chunks, 0);
    chunk_pulled_.assign(chunks, OpState());
    chunk_in_batch_.assign(chunks, 0);
    // per-peer queues are kept from call to call (a deque that is cleared keeps its first block)
    posted_.resize(world_size_);
    arrived_.resize(world_size_);
    for (auto& q : posted_) q.clear();
    for (auto& q : arrived_) q.clear();
    pending_reduce_.clear();
    pending_gather_.clear();
    // A slot needs spare bytes only if some chunk of recvbuf starts off a 16-byte boundary.  Without
    // them, slots of a chunk size that is a multiple of 256 bytes lie back to back, so chunks that are
    // neighbours in the buffers are neighbours in the pool too and merge into one kernel segment.
    const size_t chunk_bytes = plan_.part.ranges[0].size() * es_;
    if (algo == kRabenseifner && static_cast<size_t>(work_gpu_memory_size_) < chunk_bytes) {
      // allreduce_cuda_impl.h:372-385: warn, grow the working buffer to one chunk, carry on
      Warn("IBCOMM_GPU_WORK_MEMORY_SIZE is smaller than chunk size.\nruntime-reallocation is occured.");
      work_gpu_memory_size_ = static_cast<long long>(chunk_bytes);
    }
    const bool phase_margin = (reinterpret_cast<uintptr_t>(recvbuf_) & 15) != 0 || (chunk_bytes & 15) != 0;
    // The ring's queues visit the chunks of a group from the last to the first, the halving windows
    // from the first to the last; the pool hands out its slots in the same direction.
    IBCOMM_RETURN_IF_ERROR(pool_.GetController(chunk_bytes, phase_margin, Descending(plan_), &controller_));
    reduce_runs_ = gather_runs_ = 0;
    active_ = true;
    return kOk;
  }

  // Issues everything that can be issued now.  Never waits for the device or for a peer.
  int Progress(bool* progressed, bool* finished) {
    *progressed = false;
    *finished = finished_;
    if (!active_) return Fail(kInvalidArgument, "Progress without Begin");
    if (finished_) return kOk;
    stats_.progress_passes++;
    for (;;) {
      bool moved = false;
      IBCOMM_RETURN_IF_ERROR(DrainSendCompletions(&moved));
      IBCOMM_RETURN_IF_ERROR(PostSends(&moved));
      IBCOMM_RETURN_IF_ERROR(TakeMessages(&moved));
      IBCOMM_RETURN_IF_ERROR(FlushGathers());
      IBCOMM_RETURN_IF_ERROR(FlushReduces());
      if (!moved) break;
      *progressed = true;
    }
    finished_ = next_send_ == plan_.sends.size() && next_recv_ == plan_.recvs.size() && outstanding_sends_ == 0;
    *finished = finished_;
    return kOk;
  }

  // Waits for this rank's device work (and, with wait_pulls, for the peers' reads of this rank's
  // buffers) and releases the pool controller.  The collective is complete for the caller when
  // this returns, as in the reference (allreduce_cuda_impl.h:280-299, :709-715).
  int Finish(bool wait_pulls) {
    if (!active_) return kOk;
    TraceScope scope(&trace_, Trace::kOther);
    int rc = pool_.SynchronizeStreams();
    if (rc == kOk && wait_pulls) {
      for (const PullEvent& p : pull_events_) {
        rc = B::EventSynchronize(p.event);
        if (rc != kOk) break;
      }
    }
    if (rc == kOk) rc = ResolveDeviceSpans();
    ReleaseCall();
    return rc;
  }

  // Same as Finish but without touching the device: for a caller that has synchronised already
  // (or is recording a graph and will synchronise the replay).
  void FinishNoSync() {
    if (active_) ReleaseCall();
  }

  void Abort() {
    if (!active_) return;
    pool_.SynchronizeStreams();
    ReleaseCall();
  }

  // Per-rank blocking call: the shape of AllreduceRingCuda / AllreduceRabenseifnerCuda.  Every
  // emulated rank must be inside the same collective on a thread of its own.
  int AllreduceBlocking(int algo, int dtype, const void* sendbuf, void* recvbuf, size_t len_elements) {
    IBCOMM_RETURN_IF_ERROR(Begin(algo, dtype, sendbuf, recvbuf, len_elements));
    const char* t = getenv("IBCOMM_HIP_TIMEOUT_S");
    const double limit = t ? atof(t) : 120.0;
    auto last_progress = std::chrono::steady_clock::now();
    bool progressed = false, finished = false;
    for (;;) {
      const int rc = Progress(&progressed, &finished);
      if (rc != kOk) {
        // What this rank has posted stays in the channels: no later collective may run on them.
        fabric_->Poison("a rank failed inside an allreduce");
        Abort();
        return rc;
      }
      if (finished) break;
      if (progressed) {
        last_progress = std::chrono::steady_clock::now();
        continue;
      }
      if (fabric_->poisoned()) {
        Abort();
        return Fail(kTransportError, "rank %d: a peer gave up on this allreduce (%s)", rank_, fabric_->poison_reason());
      }
      std::this_thread::yield();
      const double idle = std::chrono::duration<double>(std::chrono::steady_clock::now() - last_progress).count();
      if (idle > limit) {
        fabric_->Poison("a rank saw no peer progress within IBCOMM_HIP_TIMEOUT_S");
        Abort();
        return Fail(kTransportError, "rank %d: no peer progress for %.0f s (recv %zu/%zu, send %zu/%zu)", rank_, limit,
                    next_recv_, plan_.recvs.size(), next_send_, plan_.sends.size());
      }
    }
    return Finish(true);
  }

  // Bytes of log a recording of this rank's side of the given collective needs, and whether that
  // collective visits neighbouring chunks downwards.
  int RecordingBytes(int algo, int dtype, size_t len_elements, size_t* out, bool* descending = nullptr) {
    Plan p;
    const size_t es = DTypeSize(dtype);
    if (es == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
    IBCOMM_RETURN_IF_ERROR(BuildPlan(algo, world_size_, rank_, len_elements, es, getenv("IBCOMM_CHUNKSIZE"), &p));
    size_t total = 0;
    for (const RecvOp& r : p.recvs) total += (p.part.ranges[r.chunk].size() * es + 255) & ~size_t(255);
    *out = total;
    if (descending) *descending = Descending(p);
    return kOk;
  }

  // ---- point-to-point messaging over the loopback -------------------------------------------------
  // IBVerbsCommunicator::Send / Recv / SendPoll / RecvPoll / SendWait / RecvWait / Bcast
  // (ibcomm/ibverbs_communicator.cpp:371-384, 486-499, 416-473, 529-606).  Buffers may be host or
  // device memory.  As in the reference, one non-blocking send and one non-blocking receive per peer
  // may be outstanding; posting another before its Wait is NOT_SUPPORTED (cpp:375-378, 490-493).
  // The receiver moves the data when it polls.

  int Send(int dest, const void* buf, size_t len, bool blocking) {
    IBCOMM_RETURN_IF_ERROR(CheckPeer(dest));
    if (p2p_send_pending_[dest]) return Fail(kNotSupported, "SendWait must be called before next non-blocking send.");
    fabric_->PostSend(rank_, dest, buf, len, Event{}, false);
    p2p_send_pending_[dest] = 1;
    return blocking ? SendWait(dest) : kOk;
  }
  int Recv(int src, void* buf, size_t len, bool blocking) {
    IBCOMM_RETURN_IF_ERROR(CheckPeer(src));
    if (p2p_recv_[src].active) return Fail(kNotSupported, "RecvWait must be called before next non-blocking send.");
    p2p_recv_[src].buf = buf;
    p2p_recv_[src].len = len;
    p2p_recv_[src].active = true;
    return blocking ? RecvWait(src) : kOk;
  }
  int SendPoll(int dest, bool* completed) {
    IBCOMM_RETURN_IF_ERROR(CheckPeer(dest));
    typename Fabric<B>::Completion c;
    *completed = fabric_->PollSendCompletion(rank_, dest, &c);
    if (*completed) p2p_send_pending_[dest] = 0;
    return kOk;
  }
  int RecvPoll(int src, bool* completed) {
    IBCOMM_RETURN_IF_ERROR(CheckPeer(src));
    *completed = false;
    if (!p2p_recv_[src].active) return kOk;
    Message m;
    if (!fabric_->Take(rank_, src, &m)) return kOk;
    if (m.bytes > p2p_recv_[src].len)
      return Fail(kTransportError, "message of %zu bytes from rank %d does not fit the posted buffer of %zu", m.bytes, src,
                  p2p_recv_[src].len);
    const int rc = B::CopySync(p2p_recv_[src].buf, m.src, m.bytes);
    fabric_->Complete(rank_, src, m.ticket, Event{}, false);
    p2p_recv_[src].active = false;
    *completed = true;
    return rc;
  }
  int SendWait(int dest) { return SpinUntil([&](bool* ok) { return SendPoll(dest, ok); }, "SendWait", dest); }
  int RecvWait(int src) { return SpinUntil([&](bool* ok) { return RecvPoll(src, ok); }, "RecvWait", src); }
  // Naive broadcast (cpp:586-606): the root sends to everyone, then waits for every send.
  int Bcast(void* buf, size_t len, int root) {
    IBCOMM_RETURN_IF_ERROR(CheckPeer(root));
    if (rank_ != root) return Recv(root, buf, len, true);
    for (int i = 0; i < world_size_; i++)
      if (i != rank_) IBCOMM_RETURN_IF_ERROR(Send(i, buf, len, false));
    for (int i = 0; i < world_size_; i++)
      if (i != rank_) IBCOMM_RETURN_IF_ERROR(SendWait(i));
    return kOk;
  }

  const Plan& plan() const { return plan_; }
  bool active() const { return active_; }
  size_t recv_cursor() const { return next_recv_; }
  size_t send_cursor() const { return next_send_; }
  size_t recv_total() const { return plan_.recvs.size(); }
  size_t send_total() const { return plan_.sends.size(); }

 private:
  struct OpState {
    bool issued = false;     // the device work has been enqueued
    bool has_event = false;  // ... and `event` completes with it
    Event event{};
    Stream stream{};         // stream the event was recorded on (ours), or Stream{} for a peer's
  };
  struct PendingRecv {
    int op = 0;              // index into plan_.recvs
    Message msg;
    Memory<B>* slot = nullptr;   // landing slot; null for gathers and when the message is read in place
    Memory<B>* stage = nullptr;  // send-staging slot the result goes to; null when it goes to recvbuf
    int joins = 0;               // +1 / -1: its operands continue those of the pending entry before it,
                                 // upwards / downwards in memory, so both share a kernel segment; 0: new segment
  };
  struct PostedSend {
    uint64_t ticket;
    int send_index;
  };
  struct PostedRecv {
    void* buf = nullptr;
    size_t len = 0;
    bool active = false;
  };
  struct PullEvent {
    Stream stream;
    Event event;
  };
  struct DeviceSpan {
    typename B::Timer start{}, stop{};
    Trace::DeviceCategory category = Trace::kDeviceReduce;
  };
  // A later event on a stream covers the earlier ones, so one event per peer stream is all that
  // Finish() has to wait for, however many messages the peers pulled.
  void NotePull(Event e, Stream s) {
    for (PullEvent& p : pull_events_) {
      if (p.stream == s) {
        p.event = e;
        return;
      }
    }
    pull_events_.push_back(PullEvent{s, e});
  }

  static bool Descending(const Plan& p) { return p.recvs.size() > 1 && p.recvs[1].chunk < p.recvs[0].chunk; }

  bool ZeroCopyReceive() const { return landing_ == kLandDirect || landing_ == kLandStaged; }

  char* RecvPtr(int chunk) const { return recvbuf_ + plan_.part.ranges[chunk].begin * es_; }
  const char* SendPtr(int chunk) const { return sendbuf_ + plan_.part.ranges[chunk].begin * es_; }
  size_t ChunkElems(int chunk) const { return plan_.part.ranges[chunk].size(); }
  size_t ChunkBytes(int chunk) const { return plan_.part.ranges[chunk].size() * es_; }

  // The three pointers of the reduction of one pending partial sum.
  const void* IncomingOf(const PendingRecv& p) const {
    return ZeroCopyReceive() ? p.msg.src : p.slot->LandingFor(RecvPtr(plan_.recvs[p.op].chunk));
  }
  const void* OwnOf(const PendingRecv& p) const {
    const RecvOp& r = plan_.recvs[p.op];
    return r.kind == kReduceWithSendbuf ? SendPtr(r.chunk) : static_cast<const char*>(RecvPtr(r.chunk));
  }
  void* ResultOf(const PendingRecv& p) const {
    const int c = plan_.recvs[p.op].chunk;
    return p.stage ? p.stage->LandingFor(RecvPtr(c)) : RecvPtr(c);
  }
  // +1 if `next` starts where `prev` ends, -1 if it ends where `prev` starts, else 0.
  static int Adjacent(const void* prev, size_t prev_bytes, const void* next, size_t next_bytes) {
    const char* p = static_cast<const char*>(prev);
    const char* n = static_cast<const char*>(next);
    if (p + prev_bytes == n) return 1;
    if (n + next_bytes == p) return -1;
    return 0;
  }
  // Does the reduction of `next` continue the reduction of `prev` in all three operands, in the
  // direction `run` the segment has grown in so far (0 = either)?  Returns the direction or 0.
  int ReduceJoins(const PendingRecv& prev, const PendingRecv& next, int run) const {
    const size_t pb = ChunkBytes(plan_.recvs[prev.op].chunk), nb = ChunkBytes(plan_.recvs[next.op].chunk);
    const int d = Adjacent(ResultOf(prev), pb, ResultOf(next), nb);
    if (d == 0 || (run != 0 && d != run)) return 0;
    if (Adjacent(IncomingOf(prev), pb, IncomingOf(next), nb) != d || Adjacent(OwnOf(prev), pb, OwnOf(next), nb) != d) return 0;
    return d;
  }
  int GatherJoins(const PendingRecv& prev, const PendingRecv& next, int run) const {
    const int pc = plan_.recvs[prev.op].chunk, nc = plan_.recvs[next.op].chunk;
    const int d = Adjacent(RecvPtr(pc), ChunkBytes(pc), RecvPtr(nc), ChunkBytes(nc));
    if (d == 0 || (run != 0 && d != run)) return 0;
    return Adjacent(prev.msg.src, ChunkBytes(pc), next.msg.src, ChunkBytes(nc)) == d ? d : 0;
  }
  // Adds a segment to a launch: a new entry, or (joins = +1 / -1) grown onto the end / the front of the last one.
  static void AppendSegment(SegmentBatch* batch, const Segment& seg, int joins) {
    if (joins == 0 || batch->count == 0) {
      batch->seg[batch->count++] = seg;
      return;
    }
    Segment& last = batch->seg[batch->count - 1];
    if (joins < 0) {
      last.dst = seg.dst;
      last.a = seg.a;
      last.b = seg.b;
    }
    last.n += seg.n;
  }
  // Chunks one launch may carry: the knob, or any number when the knob is at its ceiling (then only
  // the number of kernel segments, after merging, bounds a launch).
  size_t ChunkLimit() const { return max_fuse_ >= kMaxSegments ? SIZE_MAX : static_cast<size_t>(max_fuse_); }

  void ReleaseCall() {
    stats_.slots_high_water = std::max<uint64_t>(stats_.slots_high_water, controller_.high_water());
    if (controller_.active()) stats_.slot_count = controller_.slot_count();
    controller_.Release();
    pull_events_.clear();
    spans_.clear();
    timer_cursor_ = 0;
    active_ = false;
  }

  int RecordEvent(Stream s, OpState* st) {
    std::vector<Event>& arena = events_[arena_];
    if (event_cursor_ == arena.size()) {
      Event e;
      IBCOMM_RETURN_IF_ERROR(B::EventCreate(&e));
      arena.push_back(e);
    }
    st->event = arena[event_cursor_++];
    st->stream = s;
    st->has_event = true;
    st->issued = true;
    stats_.events_recorded++;
    return B::EventRecord(st->event, s);
  }

  // The messages of a batch usually carry one and the same event (their sender produced them with one
  // launch), and so do the chunks of a group: within one flush a stream waits for an event once.
  bool WaitedAlready(Stream s, Event e) {
    for (const auto& w : waited_)
      if (w.first == s && w.second == e) return true;
    waited_.emplace_back(s, e);
    return false;
  }
  // Orders stream s after `st` unless it already is (same stream) or there is nothing to wait for.
  int WaitOn(Stream s, const OpState& st) {
    if (!st.has_event || st.stream == s || WaitedAlready(s, st.event)) return kOk;
    stats_.stream_waits++;
    return B::StreamWaitEvent(s, st.event);
  }
  int WaitOnMessage(Stream s, const Message& m) {
    if (!m.has_ready || m.ready_stream == s || WaitedAlready(s, m.ready)) return kOk;
    stats_.stream_waits++;
    return B::StreamWaitEvent(s, m.ready);
  }

  // ---- device durations for the trace -------------------------------------------------------------
  // Only when tracing, only on a backend that keeps time, and never while the launches are being
  // recorded into a graph (a replay is timed as a whole by its caller).
  bool DeviceTiming() const { return B::kHasTimers && trace_.enabled() && !pool_.has_override(); }
  int NextTimer(typename B::Timer* out) {
    if (timer_cursor_ == timers_.size()) {
      typename B::Timer t;
      IBCOMM_RETURN_IF_ERROR(B::TimerCreate(&t));
      timers_.push_back(t);
    }
    *out = timers_[timer_cursor_++];
    return kOk;
  }
  int SpanBegin(Stream s, Trace::DeviceCategory category) {
    if (!DeviceTiming()) return kOk;
    DeviceSpan span;
    span.category = category;
    IBCOMM_RETURN_IF_ERROR(NextTimer(&span.start));
    IBCOMM_RETURN_IF_ERROR(NextTimer(&span.stop));
    if (spans_.empty()) span_origin_ms_ = trace_.NowMs();
    IBCOMM_RETURN_IF_ERROR(B::TimerRecord(span.start, s));
    spans_.push_back(span);
    return kOk;
  }
  int SpanEnd(Stream s) {
    if (!DeviceTiming()) return kOk;
    return B::TimerRecord(spans_.back().stop, s);
  }
  // A kernel launch takes the span's two timers itself and leaves its own begin and end times in
  // them: the span is then the kernel's duration, without the few microseconds it costs the
  // device to process a marker before and after it.
  int LaunchTimed(const SegmentBatch& batch, Stream s, int role, Trace::DeviceCategory category) {
    if (collector_) return collector_->Add(batch, dtype_, s);
    if (!DeviceTiming()) return B::LaunchSegments(batch, dtype_, s, role);
    DeviceSpan span;
    span.category = category;
    IBCOMM_RETURN_IF_ERROR(NextTimer(&span.start));
    IBCOMM_RETURN_IF_ERROR(NextTimer(&span.stop));
    if (spans_.empty()) span_origin_ms_ = trace_.NowMs();
    spans_.push_back(span);
    return B::LaunchSegments(batch, dtype_, s, role, span.start, span.stop);
  }
  // After the streams have drained: turn the timer pairs of this call into trace entries.
  int ResolveDeviceSpans() {
    for (const DeviceSpan& span : spans_) {
      float since_first = 0, duration = 0;
      IBCOMM_RETURN_IF_ERROR(B::TimerElapsedMs(spans_.front().start, span.start, &since_first));
      IBCOMM_RETURN_IF_ERROR(B::TimerElapsedMs(span.start, span.stop, &duration));
      trace_.AddDevice(span.category, span_origin_ms_ + since_first, duration);
    }
    spans_.clear();
    timer_cursor_ = 0;
    return kOk;
  }

  int DrainSendCompletions(bool* moved) {
    for (int peer = 0; peer < world_size_; peer++) {
      if (posted_[peer].empty()) continue;
      completions_.clear();
      fabric_->PollSendCompletions(rank_, peer, &completions_);
      for (const typename Fabric<B>::Completion& c : completions_) {
        if (posted_[peer].empty())
          return Fail(kTransportError, "rank %d: completion for ticket %llu from rank %d with no send outstanding", rank_,
                      (unsigned long long)c.ticket, peer);
        const PostedSend ps = posted_[peer].front();
        posted_[peer].pop_front();
        if (ps.ticket != c.ticket)
          return Fail(kTransportError, "rank %d: completion for ticket %llu from rank %d while %llu is the oldest send", rank_,
                      (unsigned long long)c.ticket, peer, (unsigned long long)ps.ticket);
        const SendOp& s = plan_.sends[ps.send_index];
        outstanding_sends_--;
        if (c.has_done) NotePull(c.done, c.done_stream);
        if (s.dep >= 0 && staged_[s.dep] != nullptr) {
          // the peer has fetched the staged partial sum: the slot is free once its read completes.  A
          // peer that reads nothing (a ghost in a replay) hands back no event; the slot's next user
          // must then at least follow the launch that wrote it.
          const OpState& wrote = recv_done_[s.dep];
          if (c.has_done) controller_.returnMemory(staged_[s.dep], c.done, c.done_stream);
          else if (wrote.has_event) controller_.returnMemory(staged_[s.dep], wrote.event, wrote.stream);
          else controller_.returnMemory(staged_[s.dep]);
          staged_[s.dep] = nullptr;
        } else if (s.dep >= 0 || in_place_) {
          chunk_unconsumed_[s.chunk]--;
          OpState& p = chunk_pulled_[s.chunk];
          p.issued = true;
          p.has_event = c.has_done;
          p.event = c.done;
          p.stream = c.done_stream;
        }
        *moved = true;
      }
    }
    return kOk;
  }

  // Hands the sends collected for one peer to the loopback under one lock.
  void PostCollected(int peer) {
    if (out_msgs_.empty()) return;
    const uint64_t first = fabric_->PostSendBatch(rank_, peer, out_msgs_.data(), out_msgs_.size());
    for (size_t i = 0; i < out_msgs_.size(); i++) posted_[peer].push_back(PostedSend{first + i, out_index_[i]});
    out_msgs_.clear();
    out_index_.clear();
  }

  int PostSends(bool* moved) {
    int batch_peer = -1;
    while (next_send_ < plan_.sends.size()) {
      const SendOp& s = plan_.sends[next_send_];
      Message m;
      if (s.dep < 0) {
        m.src = SendPtr(s.chunk);
      } else {
        const OpState& d = recv_done_[s.dep];
        if (!d.issued) break;  // the data has not been enqueued yet
        m.src = staged_[s.dep] ? staged_[s.dep]->LandingFor(RecvPtr(s.chunk)) : RecvPtr(s.chunk);
        m.ready = d.event;
        m.ready_stream = d.stream;
        m.has_ready = d.has_event;
      }
      TraceScope scope(&trace_, Trace::kIssueSend);
      m.bytes = ChunkBytes(s.chunk);
      if (s.peer != batch_peer) {
        PostCollected(batch_peer);
        batch_peer = s.peer;
      }
      out_msgs_.push_back(m);
      out_index_.push_back(static_cast<int>(next_send_));
      const bool from_staging = s.dep >= 0 && staged_[s.dep] != nullptr;
      if (!from_staging && (s.dep >= 0 || in_place_)) chunk_unconsumed_[s.chunk]++;
      outstanding_sends_++;
      stats_.messages_sent++;
      next_send_++;
      *moved = true;
    }
    PostCollected(batch_peer);
    return kOk;
  }

  // Reports the pulls of a list of messages, all completing with `done`, peer by peer in the order taken.
  void CompleteAll(const std::vector<PendingRecv>& list, const OpState& done) {
    size_t i = 0;
    while (i < list.size()) {
      const int peer = plan_.recvs[list[i].op].peer;
      tickets_.clear();
      while (i < list.size() && plan_.recvs[list[i].op].peer == peer) tickets_.push_back(list[i++].msg.ticket);
      fabric_->CompleteBatch(rank_, peer, tickets_.data(), tickets_.size(), done.event, true, done.stream);
    }
  }

  int TakeMessages(bool* moved) {
    while (next_recv_ < plan_.recvs.size()) {
      const RecvOp& r = plan_.recvs[next_recv_];
      // A gather overwrites recvbuf[chunk]; a send of ours out of that range must have been read first.
      if (r.kind == kGather && chunk_unconsumed_[r.chunk] > 0) break;
      PendingRecv p;
      trace_.Mark(Trace::kReceived);
      std::deque<Message>& arrived = arrived_[r.peer];  // taken from the loopback, not yet consumed by the plan
      if (arrived.empty()) fabric_->TakeAll(rank_, r.peer, &arrived, next_send_);
      const bool got = !arrived.empty();
      if (!got) trace_.Unmark(Trace::kReceived);
      if (!got) break;
      p.msg = arrived.front();
      arrived.pop_front();
      trace_.Mark(Trace::kReceived);
      if (p.msg.bytes != ChunkBytes(r.chunk))
        return Fail(kTransportError, "rank %d: message of %zu bytes from rank %d where chunk %d has %zu", rank_, p.msg.bytes,
                    r.peer, r.chunk, ChunkBytes(r.chunk));
      p.op = static_cast<int>(next_recv_);
      // Completions of a channel go back in the order taken, so the two pending lists never hold
      // messages at the same time.
      if (r.kind == kGather) {
        IBCOMM_RETURN_IF_ERROR(FlushReduces());
        if (!pending_gather_.empty()) p.joins = GatherJoins(pending_gather_.back(), p, pending_gather_.back().joins);
        if (p.joins == 0 && gather_runs_ == kMaxSegments) IBCOMM_RETURN_IF_ERROR(FlushGathers());
        if (p.joins == 0) gather_runs_++;
        pending_gather_.push_back(p);
        if (pending_gather_.size() >= ChunkLimit()) IBCOMM_RETURN_IF_ERROR(FlushGathers());
      } else {
        IBCOMM_RETURN_IF_ERROR(FlushGathers());
        // Segments of one launch run concurrently: a chunk whose previous partial sum is still
        // waiting in this batch must go into the next launch.
        if (chunk_in_batch_[r.chunk]) IBCOMM_RETURN_IF_ERROR(FlushReduces());
        {
          // One entry per partial sum accepted, whether or not it needs a landing slot of its own.
          TraceScope scope(&trace_, Trace::kIssueRecv);
          if (!ZeroCopyReceive() && !controller_.TryGetMemory(&p.slot)) {
            // Every slot is taken by a message waiting in this pass: launch what has been collected,
            // which hands its landing slots back (their next use is ordered on the device), and go
            // on with those.  Only a pool whose blocks hold no slot of this size at all grows.
            IBCOMM_RETURN_IF_ERROR(FlushReduces());
            IBCOMM_RETURN_IF_ERROR(controller_.getMemory(&p.slot));
          }
        }
        // Nobody on this rank reads a partial sum that is only forwarded: it is produced where the
        // next rank will fetch it, in a staging slot.  Staging slots come back when the next rank has
        // taken the message, which this rank cannot hurry; when none is left the sum goes to recvbuf
        // and is forwarded from there, as every sum is in the `direct` mode.
        if (landing_ == kLandStaged && plan_.forward_only[p.op] >= 0) (void)controller_.TryGetMemory(&p.stage);
        if (!pending_reduce_.empty()) p.joins = ReduceJoins(pending_reduce_.back(), p, pending_reduce_.back().joins);
        if (p.joins == 0 && reduce_runs_ == kMaxSegments) IBCOMM_RETURN_IF_ERROR(FlushReduces());
        if (p.joins == 0) reduce_runs_++;
        chunk_in_batch_[r.chunk] = 1;
        pending_reduce_.push_back(p);
        if (pending_reduce_.size() >= ChunkLimit()) IBCOMM_RETURN_IF_ERROR(FlushReduces());
      }
      next_recv_++;
      stats_.messages_received++;
      *moved = true;
    }
    return kOk;
  }

  // Issues the copies a pass has collected on stream s: one copy-kernel launch for all of them, or, in
  // the `memcpy` mode, one device copy per segment (a run of chunks that follow one another at both
  // ends).  *issued counts launches or copies.
  int IssueCopies(const SegmentBatch& batch, Stream s, int role, uint64_t* issued) {
    if (batch.count == 0) return kOk;
    if (landing_ != kLandMemcpy) {
      IBCOMM_RETURN_IF_ERROR(LaunchTimed(batch, s, role, Trace::kDeviceCopy));
      (*issued)++;
      return kOk;
    }
    for (int i = 0; i < batch.count; i++) {
      const Segment& seg = batch.seg[i];
      IBCOMM_RETURN_IF_ERROR(SpanBegin(s, Trace::kDeviceCopy));
      IBCOMM_RETURN_IF_ERROR(DeviceCopy(seg.dst, seg.a, seg.n * es_, s));
      IBCOMM_RETURN_IF_ERROR(SpanEnd(s));
      (*issued)++;
    }
    return kOk;
  }

  // Finished chunks: recvbuf[c] <- message.  All copies of a pass go to one stream and share one
  // event and one batch of completions (a stream, an event and a cross-stream wait per message cost
  // the host twice what an 8 MiB copy takes on the device).
  int FlushGathers() {
    if (pending_gather_.empty()) return kOk;
    waited_.clear();
    TraceScope scope(&trace_, Trace::kIssueCopyKernel);
    Stream s;
    IBCOMM_RETURN_IF_ERROR(pool_.NextStream(&s));
    SegmentBatch batch;
    batch.count = 0;
    for (const PendingRecv& p : pending_gather_) {
      const int c = plan_.recvs[p.op].chunk;
      IBCOMM_RETURN_IF_ERROR(WaitOnMessage(s, p.msg));
      IBCOMM_RETURN_IF_ERROR(WaitOn(s, chunk_pulled_[c]));
      IBCOMM_RETURN_IF_ERROR(WaitOn(s, chunk_last_[c]));
      IBCOMM_RETURN_IF_ERROR(RecordPayload(p.msg, s));
      AppendSegment(&batch, Segment{RecvPtr(c), p.msg.src, nullptr, ChunkElems(c)}, p.joins);
      stats_.gather_bytes += ChunkBytes(c);
    }
    IBCOMM_RETURN_IF_ERROR(IssueCopies(batch, s, 2, &stats_.gather_copies));
    OpState done;
    IBCOMM_RETURN_IF_ERROR(RecordEvent(s, &done));
    CompleteAll(pending_gather_, done);
    for (const PendingRecv& p : pending_gather_) {
      recv_done_[p.op] = done;
      chunk_last_[plan_.recvs[p.op].chunk] = done;
    }
    pending_gather_.clear();
    gather_runs_ = 0;
    return kOk;
  }

  // Partial sums: land every pending message, then one launch adds them all.
  int FlushReduces() {
    if (pending_reduce_.empty()) return kOk;
    waited_.clear();
    const size_t n = pending_reduce_.size();
    Stream s{};

    trace_.Mark(Trace::kIssueCopyKernel);
    IBCOMM_RETURN_IF_ERROR(pool_.NextStream(&s));
    for (size_t i = 0; i < n; i++) {
      IBCOMM_RETURN_IF_ERROR(WaitOnMessage(s, pending_reduce_[i].msg));
      IBCOMM_RETURN_IF_ERROR(RecordPayload(pending_reduce_[i].msg, s));
    }
    if (!ZeroCopyReceive()) {
      // Land every message in its pool slot, on the stream of the reduction that follows: one event
      // and one batch of completions for the pass.
      SegmentBatch copy;
      copy.count = 0;
      for (size_t i = 0; i < n; i++) {
        PendingRecv& p = pending_reduce_[i];
        const int c = plan_.recvs[p.op].chunk;
        IBCOMM_RETURN_IF_ERROR(WaitOnSlot(s, p.slot));
        // the slots of a run continue one another; the sources may or may not
        int joins = 0;
        if (p.joins != 0 && copy.count > 0) {
          const PendingRecv& q = pending_reduce_[i - 1];
          const int qc = plan_.recvs[q.op].chunk;
          if (Adjacent(q.msg.src, ChunkBytes(qc), p.msg.src, ChunkBytes(c)) == p.joins) joins = p.joins;
        }
        if (joins == 0 && copy.count == kMaxSegments) {
          IBCOMM_RETURN_IF_ERROR(IssueCopies(copy, s, 1, &stats_.landing_copies));
          copy.count = 0;
        }
        AppendSegment(&copy, Segment{p.slot->LandingFor(RecvPtr(c)), p.msg.src, nullptr, ChunkElems(c)}, joins);
        stats_.landing_bytes += ChunkBytes(c);
      }
      IBCOMM_RETURN_IF_ERROR(IssueCopies(copy, s, 1, &stats_.landing_copies));
      OpState done;
      IBCOMM_RETURN_IF_ERROR(RecordEvent(s, &done));
      CompleteAll(pending_reduce_, done);
    }

    trace_.Mark(Trace::kIssueCopyKernel);
    trace_.Mark(Trace::kIssueReduKernel);
    SegmentBatch batch;
    batch.count = 0;
    for (size_t i = 0; i < n; i++) {
      const PendingRecv& p = pending_reduce_[i];
      const RecvOp& r = plan_.recvs[p.op];
      const int c = r.chunk;
      if (r.kind != kReduceWithSendbuf) IBCOMM_RETURN_IF_ERROR(WaitOn(s, chunk_last_[c]));  // the previous halving step's sum
      if (p.stage) {
        IBCOMM_RETURN_IF_ERROR(WaitOnSlot(s, p.stage));
        staged_[p.op] = p.stage;
      }
      AppendSegment(&batch, Segment{ResultOf(p), IncomingOf(p), OwnOf(p), ChunkElems(c)}, p.joins);
      stats_.reduce_elements += ChunkElems(c);
    }
    IBCOMM_RETURN_IF_ERROR(LaunchTimed(batch, s, 0, Trace::kDeviceReduce));
    stats_.reduce_launches++;
    stats_.reduce_segments += n;
    stats_.reduce_kernel_segments += batch.count;
    uint64_t launch_elements = 0;
    for (int i = 0; i < batch.count; i++) launch_elements += batch.seg[i].n;
    if (launch_elements > stats_.largest_reduce_elements) {
      stats_.largest_reduce_elements = launch_elements;
      stats_.largest_reduce_kernel_segments = batch.count;
      stats_.largest_reduce_launches = 0;
    }
    if (launch_elements == stats_.largest_reduce_elements) stats_.largest_reduce_launches++;
    OpState done;
    IBCOMM_RETURN_IF_ERROR(RecordEvent(s, &done));
    trace_.Mark(Trace::kIssueReduKernel);
    TraceScope reduced(&trace_, Trace::kReduced);
    for (size_t i = 0; i < n; i++) {
      const PendingRecv& p = pending_reduce_[i];
      const RecvOp& r = plan_.recvs[p.op];
      recv_done_[p.op] = done;
      chunk_last_[r.chunk] = done;
      if (p.slot) controller_.returnMemory(p.slot, done.event, s);
      chunk_in_batch_[r.chunk] = 0;
    }
    if (ZeroCopyReceive()) CompleteAll(pending_reduce_, done);
    pending_reduce_.clear();
    reduce_runs_ = 0;
    return kOk;
  }

  // While this rank's traffic is being recorded for replay, keep a copy of the message's payload.
  int RecordPayload(const Message& m, Stream s) {
    if (!m.record_to) return kOk;
    return DeviceCopy(m.record_to, m.src, m.bytes, s);
  }

  // A device copy goes straight to the stream: whatever a collector still holds was issued before it
  // and has to be on the stream first.
  int DeviceCopy(void* dst, const void* src, size_t bytes, Stream s) {
    if (collector_) IBCOMM_RETURN_IF_ERROR(collector_->Flush());
    return B::CopyAsync(dst, src, bytes, s);
  }

  int CheckPeer(int peer) {
    if (rank_ < 0) return Fail(kInvalidArgument, "RegisterMyself has not been called");
    if (peer < 0 || peer >= world_size_) return Fail(kInvalidArgument, "rank %d outside world of %d", peer, world_size_);
    if (active_) return Fail(kNotSupported, "point-to-point calls cannot be mixed into a running allreduce");
    if (p2p_send_pending_.empty()) {
      p2p_send_pending_.assign(world_size_, 0);
      p2p_recv_.assign(world_size_, PostedRecv());
    }
    return kOk;
  }

  template <class Poll>
  int SpinUntil(Poll poll, const char* what, int peer) {
    const char* t = getenv("IBCOMM_HIP_TIMEOUT_S");
    const double limit = t ? atof(t) : 120.0;
    const auto t0 = std::chrono::steady_clock::now();
    for (;;) {
      bool ok = false;
      IBCOMM_RETURN_IF_ERROR(poll(&ok));
      if (ok) return kOk;
      std::this_thread::yield();
      if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > limit)
        return Fail(kTransportError, "rank %d: %s(%d) saw no completion for %.0f s", rank_, what, peer, limit);
    }
  }

  int WaitOnSlot(Stream s, const Memory<B>* slot) {
    if (!slot->has_free_event || slot->free_stream == s || WaitedAlready(s, slot->free_event)) return kOk;
    stats_.stream_waits++;
    return B::StreamWaitEvent(s, slot->free_event);
  }

  Fabric<B>* fabric_;
  int world_size_;
  int rank_ = -1;
  MemoryPool<B> pool_;
  MemoryController<B> controller_;
  LaunchCollector<B>* collector_ = nullptr;
  int max_fuse_ = kMaxSegments;
  int landing_ = kLandStaged;
  long long work_gpu_memory_size_ = 0;

  bool active_ = false;
  bool finished_ = false;
  bool in_place_ = false;
  Plan plan_;
  bool plan_cached_ = false;       // plan_ is the plan of (plan_.algo, plan_len_, plan_es_, plan_chunk_env_) for this rank
  size_t plan_len_ = 0, plan_es_ = 0;
  std::string plan_chunk_env_;     // "" = IBCOMM_CHUNKSIZE unset, else "=" + its text
  int dtype_ = kF32;
  size_t es_ = 4;
  const char* sendbuf_ = nullptr;
  char* recvbuf_ = nullptr;
  size_t next_send_ = 0, next_recv_ = 0;
  size_t outstanding_sends_ = 0;
  std::vector<OpState> recv_done_;        // per receive op: result enqueued (+ completion event)
  std::vector<Memory<B>*> staged_;        // per receive op: the send-staging slot holding its result, if any
  std::vector<OpState> chunk_last_;       // per chunk: our last device op that wrote recvbuf[chunk]
  std::vector<int> chunk_unconsumed_;     // per chunk: our sends out of recvbuf[chunk] no peer has taken yet
  std::vector<OpState> chunk_pulled_;     // per chunk: the peer's latest read of recvbuf[chunk]
  std::vector<char> chunk_in_batch_;      // per chunk: a reduction of it sits in pending_reduce_
  std::vector<std::deque<PostedSend>> posted_;  // per peer: sends awaiting completion, oldest first
  std::vector<PendingRecv> pending_reduce_, pending_gather_;
  int reduce_runs_ = 0, gather_runs_ = 0;  // kernel segments the pending lists will merge into
  std::vector<std::deque<Message>> arrived_;  // per peer: messages taken from the loopback in one go, oldest first
  std::vector<typename Fabric<B>::Completion> completions_;  // scratch of DrainSendCompletions
  std::vector<Message> out_msgs_;         // sends collected for one peer, posted together
  std::vector<int> out_index_;            // ... and their indices in plan_.sends
  std::vector<uint64_t> tickets_;         // scratch of CompleteAll
  std::vector<std::pair<Stream, Event>> waited_;  // (stream, event) pairs already ordered in the current flush
  std::vector<PullEvent> pull_events_;    // per peer stream: the latest read of this rank's memory enqueued on it
  std::vector<Event> events_[2];
  int arena_ = 0;
  size_t event_cursor_ = 0;
  EngineStats stats_;
  Trace trace_;
  std::vector<typename B::Timer> timers_;  // created on demand, reused by every traced call
  size_t timer_cursor_ = 0;
  std::vector<DeviceSpan> spans_;          // the traced launches of the call in progress
  double span_origin_ms_ = 0;              // host time at which the first of them was issued
  std::vector<char> p2p_send_pending_;   // per peer: a non-blocking Send awaits its SendPoll/SendWait
  std::vector<PostedRecv> p2p_recv_;     // per peer: the buffer a non-blocking Recv posted
};

}  // namespace ibcomm_hip
