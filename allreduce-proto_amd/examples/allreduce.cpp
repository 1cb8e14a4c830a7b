// Loopback counterpart of PFNProto's example program (examples/allreduce.cpp).
//
//   allreduce_example [np [algorithm [elements [timed_runs]]]]        defaults: 8 ring 67108864 1
//
// The reference runs one MPI process per rank; here the <np> ranks are threads of one process that
// share the GPU, each with its own IBVerbsCommunicator and its own device buffers.  What each rank
// does follows the reference: fill a float vector with integers drawn from [-1000, 1000] (:87-94;
// seeded per rank here so that the ranks differ), run the collective WARMUP + 1 times and time the
// last run (:28-29, :107-118), compare every element with the exact sum within 1e-6 (:130-140,
// where the reference takes the answer from MPI_Allreduce), print "rank: r OK" or "rank: r FAIL"
// and, once, "elapsed time : ... [s]" of rank 0.  The exit status is the number of failed ranks.
// With timed_runs > 1 the collective runs that many more times after the warm-ups; the reference's
// line still reports the first timed run and a second line lists rank 0's time for every one of them.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <thread>
#include <vector>

#include "ibcomm/ibverbs_communicator.h"

namespace {

constexpr int kWarmup = 3;

double Now() {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC_RAW, &ts);
  return ts.tv_sec + 1e-9 * ts.tv_nsec;
}

void HipOrDie(hipError_t e, int line) {
  if (e == hipSuccess) return;
  util::IbcommError(__FILE__, line, util::IBCOMM_ERROR_CODE::CUDA_ERROR, "%s", hipGetErrorString(e));
}

struct Rank {
  std::unique_ptr<IBVerbsCommunicator> comm;
  std::vector<float> send, recv;
  std::vector<double> elapsed;  // per timed run
  bool ok = false;
};

}  // namespace

int main(int argc, char* argv[]) {
  const int np = argc > 1 ? atoi(argv[1]) : 8;
  const bool ring = argc > 2 ? strcmp(argv[2], "rabenseifner") != 0 : true;
  const size_t n = argc > 3 ? strtoull(argv[3], nullptr, 10) : 67108864ull;
  const int timed_runs = argc > 4 ? atoi(argv[4]) : 1;
  if (np < 1 || n == 0 || timed_runs < 1 || (argc > 2 && strcmp(argv[2], "ring") && strcmp(argv[2], "rabenseifner"))) {
    fprintf(stderr, "usage: %s [np [ring|rabenseifner [elements [timed_runs]]]]\n", argv[0]);
    return 1;
  }

  std::vector<Rank> ranks(np);
  for (int r = 0; r < np; r++) {
    ranks[r].comm.reset(new IBVerbsCommunicator(np));
    ranks[r].comm->PrepareMemoryPool();  // public in the reference (ibverbs_communicator.h:116); nothing left to do here
    for (int i = 0; i < np; i++) {  // the bring-up sequence of the reference (:52-77); nothing to exchange here
      if (i == r) ranks[r].comm->RegisterMyself(i);
      else ranks[r].comm->RegisterQueuePair(i, ranks[r].comm->CreateQueuePair(i));
    }
    std::mt19937 mt(r);
    std::uniform_int_distribution<int> dist(-1000, 1000);
    ranks[r].send.resize(n);
    ranks[r].recv.resize(n);
    for (size_t i = 0; i < n; i++) ranks[r].send[i] = static_cast<float>(dist(mt));
  }

  std::vector<float> answer(n);  // |sum| <= 1000 * np: exact in float, whatever the order
  for (size_t i = 0; i < n; i++) {
    long sum = 0;
    for (int r = 0; r < np; r++) sum += static_cast<long>(ranks[r].send[i]);
    answer[i] = static_cast<float>(sum);
  }

  std::vector<std::thread> threads;
  for (int r = 0; r < np; r++) {
    threads.emplace_back([&, r] {
      Rank& me = ranks[r];
      float *dev_send = nullptr, *dev_recv = nullptr;
      HipOrDie(hipSetDevice(0), __LINE__);
      HipOrDie(hipMalloc(reinterpret_cast<void**>(&dev_send), n * sizeof(float)), __LINE__);
      HipOrDie(hipMalloc(reinterpret_cast<void**>(&dev_recv), n * sizeof(float)), __LINE__);
      HipOrDie(hipMemcpy(dev_send, me.send.data(), n * sizeof(float), hipMemcpyHostToDevice), __LINE__);
      for (int it = 0; it < kWarmup + timed_runs; it++) {
        const double start = Now();
        if (ring) me.comm->AllreduceRingCuda(dev_send, dev_recv, n);
        else me.comm->AllreduceRabenseifnerCuda(dev_send, dev_recv, n);
        if (it >= kWarmup) me.elapsed.push_back(Now() - start);
      }
      HipOrDie(hipMemcpy(me.recv.data(), dev_recv, n * sizeof(float), hipMemcpyDeviceToHost), __LINE__);
      HipOrDie(hipFree(dev_send), __LINE__);
      HipOrDie(hipFree(dev_recv), __LINE__);
      me.ok = true;
      int reported = 0;
      for (size_t i = 0; i < n; i++) {
        if (std::fabs(answer[i] - me.recv[i]) > 1e-6) {
          me.ok = false;
          if (reported++ < 10)
            printf("wrong at %d rank %zu element %g:%g\n", r, i, static_cast<double>(answer[i]), static_cast<double>(me.recv[i]));
        }
      }
    });
  }
  for (auto& t : threads) t.join();

  int failed = 0;
  for (int r = 0; r < np; r++) {
    printf("rank: %d%s\n", r, ranks[r].ok ? " OK" : " FAIL");
    failed += ranks[r].ok ? 0 : 1;
  }
  printf("elapsed time : %e [s]\n", ranks[0].elapsed[0]);
  if (timed_runs > 1) {
    printf("elapsed times of %d timed runs [s] :", timed_runs);
    for (double t : ranks[0].elapsed) printf(" %e", t);
    printf("\n");
  }
  ranks.clear();
  return failed;
}
