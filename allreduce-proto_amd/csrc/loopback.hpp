// In-process loopback transport: what the allreduce engines see of the network.
//
// The reference moves every chunk with two-sided InfiniBand verbs over one
// reliable-connection queue pair per peer (ibcomm/ibverbs_communicator.cpp:
// 386-414 SendRegistered, 501-527 RecvRegistered, 416-461 SendPoll, 529-572
// RecvPoll).  The engines depend on four properties only: posting never
// blocks; the k-th message from A to B is delivered into the k-th buffer B
// provides for A; a message with no buffer yet simply waits; each completion
// is reported once.  This class gives emulated ranks that share one GPU the
// same contract with device-side ordering instead of host polling:
//
//   sender    PostSend(src pointer, bytes, `ready` event after which the data
//             is valid)                                   -> ticket
//   receiver  Take() the oldest message a peer has posted, enqueue its own copy
//             (after `ready`) on one of its streams, then Complete() it,
//             handing back a `done` event that completes when the copy has
//             read the source
//   sender    PollSendCompletion() yields tickets in order with their `done`
//             event; the source may be overwritten after it.
//
// The receiver pulls, so all device work that touches a rank's memory is
// issued by that rank.  On a multi-GPU system the pull becomes a peer-to-peer
// read over xGMI and the events become IPC events; nothing here models a wire.
#pragma once

#include <stdint.h>

#include <deque>
#include <memory>
#include <mutex>
#include <vector>

namespace ibcomm_hip {

template <class B>
class Fabric {
 public:
  struct Message {
    const void* src = nullptr;
    size_t bytes = 0;
    typename B::Event ready{};
    bool has_ready = false;
    typename B::Stream ready_stream{};  // stream `ready` was recorded on (a wait from that same stream is redundant)
    uint64_t ticket = 0;
  };
  struct Completion {
    uint64_t ticket = 0;
    typename B::Event done{};
    bool has_done = false;
    typename B::Stream done_stream{};
  };

  explicit Fabric(int world_size) : n_(world_size), channels_(static_cast<size_t>(world_size) * world_size) {
    for (auto& c : channels_) c.reset(new Channel());
  }

  int world_size() const { return n_; }

  uint64_t PostSend(int from, int to, const void* src, size_t bytes, typename B::Event ready, bool has_ready,
                    typename B::Stream ready_stream = typename B::Stream{}) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    Message m;
    m.src = src;
    m.bytes = bytes;
    m.ready = ready;
    m.has_ready = has_ready;
    m.ready_stream = ready_stream;
    m.ticket = c.next_ticket++;
    c.inbox.push_back(m);
    c.posted++;
    return m.ticket;
  }

  // Receiver: remove and return the oldest message `from` has posted for `to`.  The receiver now
  // owes exactly one Complete() for it, and must complete a channel's messages in the order taken.
  bool Take(int to, int from, Message* out) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.inbox.empty() || c.inbox.front().ticket >= c.visible_below) return false;
    *out = c.inbox.front();
    c.inbox.pop_front();
    c.taken++;
    return true;
  }

  // Lockstep emulation for a single-threaded driver.  Real ranks run at the same time, so what a
  // rank can receive at some instant does not depend on the order a driver happens to visit the
  // ranks in.  BeginSweep() freezes, for every channel, the set of receivable messages to those
  // posted so far; messages posted during the sweep become receivable at the next BeginSweep().
  // EndLockstep() lifts the limit (the threaded, one-thread-per-rank use never sets it).
  void BeginSweep() {
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      c->visible_below = c->next_ticket;
    }
  }
  void EndLockstep() {
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      c->visible_below = UINT64_MAX;
    }
  }

  // Receiver: the pull of message `ticket` has been enqueued; `done` completes when it has read the source.
  void Complete(int to, int from, uint64_t ticket, typename B::Event done, bool has_done,
                typename B::Stream done_stream = typename B::Stream{}) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    Completion k;
    k.ticket = ticket;
    k.done = done;
    k.has_done = has_done;
    k.done_stream = done_stream;
    c.completions.push_back(k);
    c.delivered++;
  }

  bool PollSendCompletion(int from, int to, Completion* out) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.completions.empty()) return false;
    *out = c.completions.front();
    c.completions.pop_front();
    return true;
  }

  // Messages posted but not yet taken, over all channels (0 when idle).
  uint64_t InFlight() {
    uint64_t t = 0;
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      t += c->inbox.size();
    }
    return t;
  }
  uint64_t Delivered() {
    uint64_t t = 0;
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      t += c->delivered;
    }
    return t;
  }

  // Drops everything queued; used when a collective is abandoned after an error.
  void Reset() {
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      c->inbox.clear();
      c->completions.clear();
    }
  }

 private:
  struct Channel {
    std::mutex mu;
    std::deque<Message> inbox;
    std::deque<Completion> completions;
    uint64_t next_ticket = 0;
    uint64_t visible_below = UINT64_MAX;
    uint64_t posted = 0;
    uint64_t taken = 0;
    uint64_t delivered = 0;
  };
  Channel& chan(int from, int to) { return *channels_[static_cast<size_t>(from) * n_ + to]; }

  int n_;
  std::vector<std::unique_ptr<Channel>> channels_;
};

}  // namespace ibcomm_hip
