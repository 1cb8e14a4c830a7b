// A host-side stand-in for the device runtime, for testing the engine's logic without a GPU.
//
// TEST INFRASTRUCTURE ONLY -- it is compiled into tests/support/libibcomm_sim.so and never into
// the shipped library, which has no host execution path.
//
// Streams, events, copies and segment launches are recorded as nodes of a dependency graph exactly
// as a GPU would see them (a stream is a FIFO; a stream-wait adds an edge from the event's last
// record).  Nothing runs when it is enqueued.  At a synchronisation point the recorded nodes run in
// a RANDOM topological order, so an ordering the engine forgot to express shows up as a wrong
// result, and CheckRaces() proves the absence of such gaps outright: every pair of nodes with a
// conflicting memory access must be connected by a dependency path.
#pragma once

#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <random>
#include <string>
#include <vector>

#include "segments.hpp"
#include "status.hpp"

namespace ibcomm_sim {

using ibcomm_hip::Segment;
using ibcomm_hip::SegmentBatch;

struct SimStream {
  int id = 0;
  int last = -1;            // last node enqueued on this stream
  std::vector<int> waits;   // nodes the next enqueued node must also follow
};
struct SimEvent {
  int node = -1;            // node of the most recent record, -1 = never recorded
};

struct Access {
  uintptr_t begin, end;
  bool write;
  int part;  // segment index inside a launch: segments of one launch run concurrently
};

struct SimNode {
  int kind = 0;  // 0 marker (event record), 1 copy, 2 segment launch
  int stream = 0;
  int epoch = 0;
  std::vector<int> deps;
  void* dst = nullptr;
  const void* src = nullptr;
  size_t bytes = 0;
  SegmentBatch batch;
  int dtype = 0;
  bool executed = false;
};

class Sim {
 public:
  static Sim& Get() {
    static Sim s;
    return s;
  }

  void Reset(unsigned seed) {
    std::lock_guard<std::mutex> lock(mu_);
    nodes_.clear();
    rng_.seed(seed);
    unrecorded_waits_ = 0;
    epoch_ = 0;
    streams_made_ = 0;
  }

  int AddNode(SimStream* s, SimNode&& n) {
    std::lock_guard<std::mutex> lock(mu_);
    n.stream = s->id;
    n.epoch = epoch_;
    if (s->last >= 0) n.deps.push_back(s->last);
    for (int w : s->waits) n.deps.push_back(w);
    s->waits.clear();
    nodes_.push_back(std::move(n));
    s->last = static_cast<int>(nodes_.size()) - 1;
    return s->last;
  }

  void Wait(SimStream* s, SimEvent* e) {
    std::lock_guard<std::mutex> lock(mu_);
    if (e->node < 0) {
      unrecorded_waits_++;  // on a GPU this wait would silently be a no-op
      return;
    }
    s->waits.push_back(e->node);
  }

  int NewStreamId() {
    std::lock_guard<std::mutex> lock(mu_);
    return ++streams_made_;
  }

  // Runs every recorded node that has not run yet, in a random order that respects the edges.
  void RunAll() {
    std::lock_guard<std::mutex> lock(mu_);
    const int n = static_cast<int>(nodes_.size());
    std::vector<int> indeg(n, 0);
    std::vector<std::vector<int>> out(n);
    std::vector<int> ready;
    for (int i = 0; i < n; i++) {
      if (nodes_[i].executed) continue;
      for (int d : nodes_[i].deps) {
        if (!nodes_[d].executed) {
          indeg[i]++;
          out[d].push_back(i);
        }
      }
      if (indeg[i] == 0) ready.push_back(i);
    }
    while (!ready.empty()) {
      const size_t k = std::uniform_int_distribution<size_t>(0, ready.size() - 1)(rng_);
      const int i = ready[k];
      ready[k] = ready.back();
      ready.pop_back();
      Execute(nodes_[i]);
      nodes_[i].executed = true;
      for (int j : out[i])
        if (--indeg[j] == 0) ready.push_back(j);
    }
    epoch_++;
  }

  // Number of node pairs that touch overlapping memory (at least one writing) without being
  // ordered by a dependency path.  -1 if the graph is too large to check.
  long CheckRaces(std::string* first) {
    std::lock_guard<std::mutex> lock(mu_);
    const size_t n = nodes_.size();
    if (n > 40000) return -1;
    const size_t words = (n + 63) / 64;
    std::vector<uint64_t> anc(n * words, 0);
    for (size_t i = 0; i < n; i++) {
      uint64_t* ai = &anc[i * words];
      for (int d : nodes_[i].deps) {
        const uint64_t* ad = &anc[static_cast<size_t>(d) * words];
        for (size_t w = 0; w <= static_cast<size_t>(d) / 64; w++) ai[w] |= ad[w];
        ai[d / 64] |= uint64_t(1) << (d % 64);
      }
    }
    struct Rec { uintptr_t begin, end; int node; bool write; int part; };
    std::vector<Rec> recs;
    for (size_t i = 0; i < n; i++) {
      std::vector<Access> acc;
      Accesses(nodes_[i], &acc);
      for (const Access& a : acc)
        if (a.end > a.begin) recs.push_back(Rec{a.begin, a.end, static_cast<int>(i), a.write, a.part});
    }
    std::sort(recs.begin(), recs.end(), [](const Rec& x, const Rec& y) { return x.begin < y.begin; });
    long races = 0;
    for (size_t i = 0; i < recs.size(); i++) {
      for (size_t j = i + 1; j < recs.size() && recs[j].begin < recs[i].end; j++) {
        if (!recs[i].write && !recs[j].write) continue;
        int lo = std::min(recs[i].node, recs[j].node), hi = std::max(recs[i].node, recs[j].node);
        if (lo == hi) {
          if (recs[i].part == recs[j].part) continue;  // one segment may update in place
        } else {
          if (nodes_[lo].epoch < nodes_[hi].epoch) continue;  // separated by a full synchronisation
          if (anc[static_cast<size_t>(hi) * words + lo / 64] >> (lo % 64) & 1) continue;
        }
        if (races == 0 && first) {
          char buf[256];
          snprintf(buf, sizeof buf, "node %d (kind %d, stream %d) and node %d (kind %d, stream %d) overlap at %p without ordering",
                   lo, nodes_[lo].kind, nodes_[lo].stream, hi, nodes_[hi].kind, nodes_[hi].stream,
                   reinterpret_cast<void*>(std::max(recs[i].begin, recs[j].begin)));
          *first = buf;
        }
        races++;
      }
    }
    return races;
  }

  long unrecorded_waits() const { return unrecorded_waits_; }
  long node_count() const { return static_cast<long>(nodes_.size()); }

 private:
  static void Accesses(const SimNode& n, std::vector<Access>* out) {
    if (n.kind == 1) {
      out->push_back(Access{reinterpret_cast<uintptr_t>(n.src), reinterpret_cast<uintptr_t>(n.src) + n.bytes, false, 0});
      out->push_back(Access{reinterpret_cast<uintptr_t>(n.dst), reinterpret_cast<uintptr_t>(n.dst) + n.bytes, true, 0});
    } else if (n.kind == 2) {
      const size_t es = ibcomm_hip::DTypeSize(n.dtype);
      for (int i = 0; i < n.batch.count; i++) {
        const Segment& s = n.batch.seg[i];
        const size_t b = s.n * es;
        out->push_back(Access{reinterpret_cast<uintptr_t>(s.a), reinterpret_cast<uintptr_t>(s.a) + b, false, i});
        if (s.b) out->push_back(Access{reinterpret_cast<uintptr_t>(s.b), reinterpret_cast<uintptr_t>(s.b) + b, false, i});
        out->push_back(Access{reinterpret_cast<uintptr_t>(s.dst), reinterpret_cast<uintptr_t>(s.dst) + b, true, i});
      }
    }
  }

  template <typename T>
  static void RunSegment(const Segment& s) {
    T* d = static_cast<T*>(s.dst);
    const T* a = static_cast<const T*>(s.a);
    const T* b = static_cast<const T*>(s.b);
    for (uint64_t i = 0; i < s.n; i++) {
      T v = a[i];
      if (b) v = v + b[i];
      d[i] = v;
    }
  }

  static void Execute(const SimNode& n) {
    if (n.kind == 1) {
      memmove(n.dst, n.src, n.bytes);
    } else if (n.kind == 2) {
      // last segment first: a batch must not depend on its segments running in list order
      for (int i = n.batch.count - 1; i >= 0; i--) {
        switch (n.dtype) {
          case ibcomm_hip::kF32: RunSegment<float>(n.batch.seg[i]); break;
          case ibcomm_hip::kI32: RunSegment<uint32_t>(n.batch.seg[i]); break;
          case ibcomm_hip::kF64: RunSegment<double>(n.batch.seg[i]); break;
          case ibcomm_hip::kI64: RunSegment<uint64_t>(n.batch.seg[i]); break;
        }
      }
    }
  }

  std::mutex mu_;
  std::vector<SimNode> nodes_;
  std::mt19937 rng_;
  long unrecorded_waits_ = 0;
  int epoch_ = 0;
  int streams_made_ = 0;
};

struct SimBackend {
  using Stream = SimStream*;
  using Event = SimEvent*;

  static int Malloc(void** p, size_t bytes) {
    *p = aligned_alloc(256, (bytes + 255) & ~size_t(255));
    if (!*p) return ibcomm_hip::Fail(ibcomm_hip::kDeviceError, "host allocation of %zu bytes failed", bytes);
    memset(*p, 0xEE, bytes);
    return 0;
  }
  static int Free(void* p) {
    free(p);
    return 0;
  }
  static int StreamCreate(Stream* s) {
    *s = new SimStream();
    (*s)->id = Sim::Get().NewStreamId();
    return 0;
  }
  static int StreamDestroy(Stream s) {
    delete s;
    return 0;
  }
  static int StreamSynchronize(Stream) {
    Sim::Get().RunAll();
    return 0;
  }
  static int EventCreate(Event* e) {
    *e = new SimEvent();
    return 0;
  }
  static int EventDestroy(Event e) {
    delete e;
    return 0;
  }
  static int EventRecord(Event e, Stream s) {
    SimNode n;
    n.kind = 0;
    e->node = Sim::Get().AddNode(s, std::move(n));
    return 0;
  }
  static int StreamWaitEvent(Stream s, Event e) {
    Sim::Get().Wait(s, e);
    return 0;
  }
  static int EventSynchronize(Event) {
    Sim::Get().RunAll();
    return 0;
  }
  using Timer = int;  // the simulated device keeps no time
  static constexpr bool kHasTimers = false;
  static int TimerCreate(Timer*) { return 0; }
  static int TimerDestroy(Timer) { return 0; }
  static int TimerRecord(Timer, Stream) { return 0; }
  static int TimerElapsedMs(Timer, Timer, float* ms) {
    *ms = 0;
    return 0;
  }
  static int CopySync(void* dst, const void* src, size_t bytes) {
    memmove(dst, src, bytes);
    return 0;
  }
  static int CopyAsync(void* dst, const void* src, size_t bytes, Stream s) {
    SimNode n;
    n.kind = 1;
    n.dst = dst;
    n.src = src;
    n.bytes = bytes;
    Sim::Get().AddNode(s, std::move(n));
    return 0;
  }
  static int LaunchSegments(const SegmentBatch& batch, int dtype, Stream s, int role = 0, Timer = 0, Timer = 0) {
    SimNode n;
    n.kind = 2;
    n.batch = batch;
    n.dtype = dtype;
    Sim::Get().AddNode(s, std::move(n));
    return 0;
  }
};

}  // namespace ibcomm_sim
