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

#include <atomic>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
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
    char* record_to = nullptr;          // while recording: where the receiver must also copy the payload
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
    Message m;
    m.src = src;
    m.bytes = bytes;
    m.ready = ready;
    m.has_ready = has_ready;
    m.ready_stream = ready_stream;
    return PostSendBatch(from, to, &m, 1);
  }

  // Posts n messages (src, bytes and the ready fields filled in) to one peer in one go; their tickets
  // are consecutive and the first is returned.  One lock per batch instead of one per message matters
  // when sender and receiver are threads of their own: a receiver that polls takes the same lock.
  uint64_t PostSendBatch(int from, int to, const Message* msgs, size_t n) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    const uint64_t first = c.next_ticket;
    if (from == replay_rank_) {
      // The peer is a ghost: nobody will read the data, the sends are complete at once.
      for (size_t i = 0; i < n; i++) {
        Completion k;
        k.ticket = c.next_ticket++;
        c.completions.push_back(k);
      }
      return first;
    }
    for (size_t i = 0; i < n; i++) {
      Message m = msgs[i];
      m.ticket = c.next_ticket++;
      m.record_to = nullptr;
      c.inbox.push_back(m);
    }
    c.posted += n;
    return first;
  }

  // Receiver: remove and return the oldest message `from` has posted for `to`.  The receiver now
  // owes exactly one Complete() for it, and must complete a channel's messages in the order taken.
  // `sends_posted` is how many messages the receiver itself has emitted so far in this collective;
  // it only matters for recording and replay (below).
  bool Take(int to, int from, Message* out, size_t sends_posted = 0) {
    if (to == replay_rank_) return GhostTake(from, out, sends_posted);
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.inbox.empty() || c.inbox.front().ticket >= c.visible_below) return false;
    *out = c.inbox.front();
    c.inbox.pop_front();
    c.taken++;
    if (to == record_rank_) {
      // Remember the message for replay: its size, its sender, and how far the receiver had got with
      // its own sends when the message was there to take.  The receiver copies the payload to
      // out->record_to (a range of the log) when it lands the message.
      LogEntry e;
      e.from = from;
      e.bytes = out->bytes;
      e.gate = sends_posted;
      const size_t rounded = (out->bytes + 255) & ~size_t(255);
      const bool fits = log_used_ + rounded <= log_need_;
      // The log is filled in the direction the chunks are visited in, so that payloads of chunks
      // that are neighbours in the buffers are neighbours in the log, as they are in the pool.
      e.offset = !fits ? 0 : (log_descending_ ? log_need_ - log_used_ - rounded : log_used_);
      log_used_ += rounded;
      out->record_to = fits ? log_base_ + e.offset : nullptr;
      log_.push_back(e);
    }
    return true;
  }

  // Receiver: all messages `from` has posted for `to` that may be taken now, appended to *out in
  // order, under one lock (one at a time while recording or replaying, where each message is tied to
  // the receiver's own progress).  Returns how many were appended.
  size_t TakeAll(int to, int from, std::deque<Message>* out, size_t sends_posted = 0) {
    if (to == replay_rank_ || to == record_rank_) {
      Message m;
      if (!Take(to, from, &m, sends_posted)) return 0;
      out->push_back(m);
      return 1;
    }
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    size_t n = 0;
    while (!c.inbox.empty() && c.inbox.front().ticket < c.visible_below) {
      out->push_back(c.inbox.front());
      c.inbox.pop_front();
      n++;
    }
    c.taken += n;
    return n;
  }

  // Lockstep emulation for a single-threaded driver.  Real ranks run at the same time, so what a
  // rank can receive at some instant does not depend on the order a driver happens to visit the
  // ranks in.  BeginSweep() freezes, for every channel, the set of receivable messages to those
  // posted so far; messages posted during the sweep become receivable at the next BeginSweep().
  // EndLockstep() lifts the limit (the threaded, one-thread-per-rank use never sets it).
  // Completions are frozen the same way: a rank learns that a peer has taken its message at the
  // next sweep, not from a peer the driver happened to visit earlier in this one.  (Otherwise the
  // rank visited last would get its staging slots back a step before everybody else and write, in
  // this step, into slots the first rank's launch of this step reads; correct on an in-order
  // stream, but it keeps the two launches from being merged.)
  void BeginSweep() {
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      c->visible_below = c->next_ticket;
      c->completions_visible = c->completions.size();
    }
  }
  void EndLockstep() {
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      c->visible_below = UINT64_MAX;
      c->completions_visible = SIZE_MAX;
    }
  }

  // Receiver: the pull of message `ticket` has been enqueued; `done` completes when it has read the source.
  void Complete(int to, int from, uint64_t ticket, typename B::Event done, bool has_done,
                typename B::Stream done_stream = typename B::Stream{}) {
    CompleteBatch(to, from, &ticket, 1, done, has_done, done_stream);
  }
  // The same for n messages of one channel whose pulls share one completion event.
  void CompleteBatch(int to, int from, const uint64_t* tickets, size_t n, typename B::Event done, bool has_done,
                     typename B::Stream done_stream = typename B::Stream{}) {
    if (to == replay_rank_) return;  // recorded messages have no sender waiting for them
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    for (size_t i = 0; i < n; i++) {
      Completion k;
      k.ticket = tickets[i];
      k.done = done;
      k.has_done = has_done;
      k.done_stream = done_stream;
      c.completions.push_back(k);
    }
    c.delivered += n;
  }

  bool PollSendCompletion(int from, int to, Completion* out) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    if (c.completions.empty() || c.completions_visible == 0) return false;
    *out = c.completions.front();
    c.completions.pop_front();
    if (c.completions_visible != SIZE_MAX) c.completions_visible--;
    return true;
  }

  // Sender: every completion that is there, appended to *out in order, under one lock.
  size_t PollSendCompletions(int from, int to, std::vector<Completion>* out) {
    Channel& c = chan(from, to);
    std::lock_guard<std::mutex> lock(c.mu);
    const size_t n = c.completions.size() < c.completions_visible ? c.completions.size() : c.completions_visible;
    out->insert(out->end(), c.completions.begin(), c.completions.begin() + n);
    c.completions.erase(c.completions.begin(), c.completions.begin() + n);
    if (c.completions_visible != SIZE_MAX) c.completions_visible -= n;
    return n;
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

  // ---- recording one rank's incoming traffic, and replaying it -------------------------------
  //
  // Measuring one rank's share of a collective needs that rank to run alone, yet every message it
  // consumes is a partial sum produced by the others.  So one ordinary run of the whole world is
  // recorded: each message `rank` takes is copied into a device-resident log together with the
  // number of sends `rank` had posted when the message was available.  In a replay the other ranks
  // are ghosts: `rank` finds the logged messages in its channels, each visible once it has itself
  // posted as many sends as it had in the recorded run (which paces the replay the way the real
  // dependency on upstream ranks does), and its own sends complete immediately.

  // Arms recording for the next collective.  log_bytes must cover the payload of every message
  // `rank` will take (each rounded up to 256 bytes); `descending` says that the collective visits
  // neighbouring chunks from the higher address to the lower.
  int StartRecording(int rank, size_t log_bytes, bool descending = false) {
    StopReplay();
    if (log_base_ && log_bytes_ < log_bytes) {
      B::Free(log_base_);
      log_base_ = nullptr;
    }
    if (!log_base_) {
      void* p = nullptr;
      const int rc = B::Malloc(&p, log_bytes);
      if (rc != 0) return rc;
      log_base_ = static_cast<char*>(p);
      log_bytes_ = log_bytes;
    }
    log_.clear();
    log_used_ = 0;
    log_need_ = log_bytes;
    log_descending_ = descending;
    record_rank_ = rank;
    recorded_rank_ = -1;
    return 0;
  }
  // Ends recording; the log now describes `rank`'s side of the collective just run.
  void StopRecording() {
    if (record_rank_ >= 0 && log_used_ <= log_need_) recorded_rank_ = record_rank_;
    record_rank_ = -1;
  }
  int recording_rank() const { return record_rank_; }
  int recorded_rank() const { return recorded_rank_; }
  size_t recorded_messages() const { return log_.size(); }

  // From now on `rank` runs alone against the recorded messages.  False if nothing was recorded for it.
  bool StartReplay(int rank) {
    if (recorded_rank_ != rank) return false;
    replay_rank_ = rank;
    RewindReplay();
    return true;
  }
  void RewindReplay() { log_cursor_ = 0; }
  void StopReplay() { replay_rank_ = -1; }
  int replay_rank() const { return replay_rank_; }
  bool ReplayDrained() const { return log_cursor_ == log_.size(); }

  void FreeLog() {
    if (log_base_) B::Free(log_base_);
    log_base_ = nullptr;
    log_bytes_ = 0;
    log_.clear();
    recorded_rank_ = -1;
  }
  ~Fabric() { FreeLog(); }

  // A rank that gives up inside a collective while its peers may still be in it (one thread per
  // rank) leaves messages and completions behind that no later collective could tell from its own.
  // It marks the world instead: peers that are waiting stop with a clear error, and every later
  // collective on this world is refused.
  void Poison(const char* reason) {
    std::lock_guard<std::mutex> lock(poison_mu_);
    if (!poisoned_.load()) {
      poison_reason_ = reason;
      poisoned_.store(true);
    }
  }
  bool poisoned() const { return poisoned_.load(); }
  const char* poison_reason() {
    std::lock_guard<std::mutex> lock(poison_mu_);
    return poison_reason_.c_str();
  }

  // Drops everything queued and lifts the mark above; for the owner of the world, once every rank
  // has left the collective that was abandoned.
  void Reset() {
    for (auto& c : channels_) {
      std::lock_guard<std::mutex> lock(c->mu);
      c->inbox.clear();
      c->completions.clear();
      if (c->completions_visible != SIZE_MAX) c->completions_visible = 0;
    }
    std::lock_guard<std::mutex> lock(poison_mu_);
    poisoned_.store(false);
    poison_reason_.clear();
  }

 private:
  struct LogEntry {
    int from;
    size_t bytes;
    size_t gate;    // sends the recorded rank had posted when this message was available
    size_t offset;  // of the payload in the log
  };

  bool GhostTake(int from, Message* out, size_t sends_posted) {
    if (log_cursor_ >= log_.size()) return false;
    const LogEntry& e = log_[log_cursor_];
    if (e.from != from || sends_posted < e.gate) return false;
    *out = Message();
    out->src = log_base_ + e.offset;
    out->bytes = e.bytes;
    out->ticket = log_cursor_;
    log_cursor_++;
    return true;
  }

  struct Channel {
    std::mutex mu;
    std::deque<Message> inbox;
    std::deque<Completion> completions;
    uint64_t next_ticket = 0;
    uint64_t visible_below = UINT64_MAX;
    size_t completions_visible = SIZE_MAX;  // how many of `completions`, from the front, the sender may see (lockstep sweeps)
    uint64_t posted = 0;
    uint64_t taken = 0;
    uint64_t delivered = 0;
  };
  Channel& chan(int from, int to) { return *channels_[static_cast<size_t>(from) * n_ + to]; }

  int n_;
  std::vector<std::unique_ptr<Channel>> channels_;
  std::atomic<bool> poisoned_{false};
  std::mutex poison_mu_;
  std::string poison_reason_;
  int record_rank_ = -1;    // rank whose incoming messages are being logged
  int recorded_rank_ = -1;  // rank the finished log belongs to
  int replay_rank_ = -1;    // rank currently running against the log
  char* log_base_ = nullptr;
  size_t log_bytes_ = 0, log_need_ = 0, log_used_ = 0, log_cursor_ = 0;
  bool log_descending_ = false;
  std::vector<LogEntry> log_;
};

}  // namespace ibcomm_hip
