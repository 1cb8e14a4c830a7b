// Meeting point of the blocking per-rank allreduce calls of one loopback world.
//
// The reference's surface is one blocking call per rank, AllreduceRingCuda<T> /
// AllreduceRabenseifnerCuda<T> (ibcomm/ibverbs_communicator.h:108-115), entered by every process of
// the job at about the same time (examples/allreduce.cpp:107-118).  Here the ranks are threads of one
// process on one GPU, and the cheapest way to run the collective they all ask for is the
// single-thread driver with its recorded graph: so the calls meet.  Each rank leaves its arguments;
// the rank that arrives last drives the whole world with everybody's buffers (one eager run, one
// recording, graph replays from then on) while the others wait for its verdict; all return the same
// status.  The ranks' pipelines, their wire order and every sum are those of the per-rank engine:
// only who issues the device work changes.
//
// A rank that waits longer than its time limit for its peers takes its arguments back, marks the
// world as abandoned and fails with a transport error; the others see the mark and stop waiting.
// Once the last rank has arrived nobody gives up any more: the driver works for all and finishes.
#pragma once

#include <stdint.h>
#include <string.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>

#include "status.hpp"

namespace ibcomm_hip {

// What one rank passes to its blocking call.
struct RankCall {
  void* comm = nullptr;  // the rank's communicator, as the driver's callback wants it
  int algo = 0;
  int dtype = 0;
  const void* sendbuf = nullptr;
  void* recvbuf = nullptr;
  size_t len = 0;
  bool present = false;
};

class Rendezvous {
 public:
  explicit Rendezvous(int world_size) : n_(world_size), calls_(static_cast<size_t>(world_size)) {}
  Rendezvous(const Rendezvous&) = delete;
  Rendezvous& operator=(const Rendezvous&) = delete;

  uint64_t rounds() const { return generation_.load(std::memory_order_relaxed); }

  // Blocks until every rank of the world has arrived with its call and the last of them has run
  // `drive(calls)` (calls[r] = rank r's arguments), then returns what drive returned, with its
  // message in this thread's error buffer.  `world` is the loopback world the ranks share: it
  // carries the mark a rank leaves when it gives up (poisoned / Poison / poison_reason).
  template <class World, class Drive>
  int Arrive(int rank, const RankCall& call, double limit_s, World* world, Drive&& drive) {
    if (rank < 0 || rank >= n_) return Fail(kInvalidArgument, "RegisterMyself has not been called");
    std::unique_lock<std::mutex> lock(mu_);
    if (world->poisoned())
      return Fail(kTransportError, "this loopback world was abandoned after an earlier failure (%s); create a new one",
                  world->poison_reason());
    if (calls_[rank].present) return Fail(kNotSupported, "rank %d is already inside an allreduce", rank);
    calls_[rank] = call;
    calls_[rank].present = true;
    arrived_++;
    const uint64_t my_round = generation_.load(std::memory_order_relaxed);

    if (arrived_ == n_) {
      driving_ = true;
      lock.unlock();
      int rc = CheckAgreement();
      if (rc == kOk) rc = drive(calls_.data());
      lock.lock();
      result_ = rc;
      if (rc != kOk) {
        strncpy(message_, LastErrorBuffer(), sizeof message_);
        message_[sizeof message_ - 1] = 0;
      }
      for (RankCall& c : calls_) c.present = false;
      arrived_ = 0;
      driving_ = false;
      generation_.store(my_round + 1, std::memory_order_release);
      lock.unlock();
      done_.notify_all();
      return rc;
    }
    lock.unlock();

    // Wait for the driver's verdict: a short spin (a replayed collective takes tens of microseconds
    // to a few milliseconds and the reference's ranks busy-poll as well), then yields, then sleeps
    // on the condition variable in slices, looking at the clock and at the world's mark in between.
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t spins = 1;; spins++) {
      if (generation_.load(std::memory_order_acquire) != my_round) break;
      if (spins < 4096) {
        __builtin_ia32_pause();
        continue;
      }
      const double waited = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      if (waited < 0.002) {
        std::this_thread::yield();
        continue;
      }
      lock.lock();
      if (generation_.load(std::memory_order_relaxed) != my_round) {
        lock.unlock();
        break;
      }
      if (!driving_ && (world->poisoned() || waited > limit_s)) {
        calls_[rank].present = false;
        arrived_--;
        const int missing = n_ - arrived_ - 1;
        lock.unlock();
        if (world->poisoned())
          return Fail(kTransportError, "rank %d: a peer gave up on this allreduce (%s)", rank, world->poison_reason());
        world->Poison("a rank saw no peer progress within IBCOMM_HIP_TIMEOUT_S");
        return Fail(kTransportError, "rank %d: no peer progress for %.0f s (%d of %d ranks never entered the allreduce)", rank,
                    limit_s, missing, n_);
      }
      // (a wait against the system clock is pthread_cond_timedwait, which ThreadSanitizer follows;
      // the steady-clock form is a newer call that gcc 11's does not)
      done_.wait_until(lock, std::chrono::system_clock::now() + std::chrono::milliseconds(driving_ ? 1 : 20));
      lock.unlock();
    }
    // The next round cannot start before this rank has arrived again, so the verdict is still there.
    const int rc = result_;
    if (rc != kOk) strncpy(LastErrorBuffer(), message_, 512);
    return rc;
  }

 private:
  // Every process of the reference passes the same algorithm, element type and length; ranks that
  // do not are told so instead of being left to trip over each other's messages.
  int CheckAgreement() const {
    for (int r = 1; r < n_; r++) {
      if (calls_[r].algo != calls_[0].algo || calls_[r].dtype != calls_[0].dtype || calls_[r].len != calls_[0].len)
        return Fail(kInvalidArgument, "rank %d entered the allreduce with algorithm %d, element type %d, %zu elements; rank 0 with %d, %d, %zu",
                    r, calls_[r].algo, calls_[r].dtype, calls_[r].len, calls_[0].algo, calls_[0].dtype, calls_[0].len);
    }
    return kOk;
  }

  const int n_;
  std::mutex mu_;
  std::condition_variable done_;
  std::vector<RankCall> calls_;
  int arrived_ = 0;
  bool driving_ = false;
  std::atomic<uint64_t> generation_{0};
  int result_ = kOk;
  char message_[512] = "";
};

}  // namespace ibcomm_hip
