// Cooperative driver: one host thread steps every emulated rank of a loopback world.
//
// The reference runs one process per rank and lets each spin in its own polling loop.  With all
// ranks on one GPU a single thread can do the same job deterministically: call Progress() on each
// rank in turn until all have issued their whole plan.  Progress() never waits, so a full sweep in
// which no rank moved means the plans do not fit together; that is reported instead of spinning.
//
// Sweeps are lockstep: during a sweep a rank can take only the messages that had been posted when
// the sweep began (Fabric::BeginSweep).  Without that, the rank visited last would find its
// upstream's entire reduce-scatter already posted and the emulated ranks would run one after the
// other; with it every sweep is one step of the algorithm on all ranks at once, and their launches
// are independent and overlap on the GPU the way N devices would work side by side.
#pragma once

#include <vector>

#include "engine.hpp"

namespace ibcomm_hip {

// Issues one allreduce on every rank.  With `synchronize` the call returns when all results are in
// place (the reference's blocking semantics); without it only the host-side issue is done and the
// caller synchronises (used while recording a graph).
// With a `collector` (only where all ranks issue on one stream, i.e. while a world is being recorded) the
// ranks' launches are merged as far as their memory accesses allow (merge.hpp); everything
// collected is on the stream when the call returns.
template <class B>
int RunWorld(Communicator<B>* const* comms, int n, int algo, int dtype, const void* const* sendbufs,
             void* const* recvbufs, size_t len_elements, bool synchronize, LaunchCollector<B>* collector = nullptr) {
  if (n < 1) return Fail(kInvalidArgument, "empty world");
  for (int r = 0; r < n; r++) {
    if (comms[r]->world_size() != n || comms[r]->rank() != r)
      return Fail(kInvalidArgument, "communicator %d is rank %d of %d, expected rank %d of %d", r, comms[r]->rank(),
                  comms[r]->world_size(), r, n);
  }
  int rc = kOk;
  int begun = 0;
  for (int r = 0; r < n; r++) comms[r]->set_collector(collector);
  for (; begun < n; begun++) {
    rc = comms[begun]->Begin(algo, dtype, sendbufs[begun], recvbufs[begun], len_elements);
    if (rc != kOk) break;
  }
  if (rc == kOk) {
    std::vector<char> done(n, 0);
    int remaining = n;
    Fabric<B>* fabric = comms[0]->fabric();
    static const bool lockstep = !(getenv("IBCOMM_HIP_LOCKSTEP") && atoi(getenv("IBCOMM_HIP_LOCKSTEP")) == 0);
    while (remaining > 0 && rc == kOk) {
      bool any = false;
      if (lockstep) fabric->BeginSweep();
      for (int r = 0; r < n && rc == kOk; r++) {
        if (done[r]) continue;
        bool progressed = false, finished = false;
        rc = comms[r]->Progress(&progressed, &finished);
        any = any || progressed || finished;
        if (finished) {
          done[r] = 1;
          remaining--;
        }
      }
      // a sweep sees everything posted before it began, so one idle sweep is conclusive
      if (rc == kOk && remaining > 0 && !any) {
        int stuck = 0;
        while (done[stuck]) stuck++;
        rc = Fail(kTransportError, "loopback world made no progress: rank %d stopped at receive %zu/%zu, send %zu/%zu", stuck,
                  comms[stuck]->recv_cursor(), comms[stuck]->recv_total(), comms[stuck]->send_cursor(),
                  comms[stuck]->send_total());
      }
    }
  }
  comms[0]->fabric()->EndLockstep();
  for (int r = 0; r < n; r++) comms[r]->set_collector(nullptr);
  if (collector) {
    if (rc == kOk) rc = collector->Flush();
    else collector->Discard();
  }
  if (rc != kOk) {
    // keep the message of the first failure
    char saved[512];
    strncpy(saved, LastErrorBuffer(), sizeof saved);
    saved[sizeof saved - 1] = 0;
    for (int r = 0; r < begun; r++) comms[r]->Abort();
    comms[0]->fabric()->Reset();
    strncpy(LastErrorBuffer(), saved, 512);
    return rc;
  }
  for (int r = 0; r < n; r++) {
    if (synchronize) {
      const int f = comms[r]->Finish(false);  // every rank's streams are drained below or here
      if (f != kOk && rc == kOk) rc = f;
    } else {
      comms[r]->FinishNoSync();
    }
  }
  return rc;
}

// One rank on its own against recorded peers (Fabric::StartReplay must be in effect for it).
template <class B>
int RunAlone(Communicator<B>* comm, int algo, int dtype, const void* sendbuf, void* recvbuf, size_t len_elements,
             bool synchronize) {
  comm->fabric()->RewindReplay();
  IBCOMM_RETURN_IF_ERROR(comm->Begin(algo, dtype, sendbuf, recvbuf, len_elements));
  for (;;) {
    bool progressed = false, finished = false;
    const int rc = comm->Progress(&progressed, &finished);
    if (rc != kOk) {
      comm->Abort();
      comm->fabric()->Reset();  // completions of sends to the ghosts must not leak into the next call
      return rc;
    }
    if (finished) break;
    if (!progressed) {
      comm->Abort();
      comm->fabric()->Reset();
      return Fail(kTransportError, "replay of rank %d stalled at receive %zu/%zu, send %zu/%zu: the recording is of a different call",
                  comm->rank(), comm->recv_cursor(), comm->recv_total(), comm->send_cursor(), comm->send_total());
    }
  }
  if (!comm->fabric()->ReplayDrained()) {
    comm->Abort();
    comm->fabric()->Reset();
    return Fail(kTransportError, "replay of rank %d left recorded messages unused: the recording is of a different call", comm->rank());
  }
  if (synchronize) return comm->Finish(false);
  comm->FinishNoSync();
  return kOk;
}

}  // namespace ibcomm_hip
