// Stand-alone driver that runs the allreduce engine on the simulated device under the host
// sanitizers (built by tests/test_engine_sanitizers.py with -fsanitize=address,undefined or
// -fsanitize=thread; no GPU, no Python in the process).  Random worlds, lengths, chunk sizes, fusion
// limits, landing modes and pool sizes, single-threaded lockstep, one thread per rank with an engine of
// its own, and one thread per rank whose blocking calls meet (every other threaded world), plus the
// record/replay, failure-handling, meeting and point-to-point cases of sim_world.cpp.
//
//   sanitize_main <iterations> <all_threaded 0|1> [<extras 0|1>]    exit status 0 if every run returned success
// (extras, default 1: the failure-handling and point-to-point cases)
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

extern "C" {
int sim_world_allreduce(int algo, int dtype, int world, const void* const* sendbufs, void* const* recvbufs, size_t len,
                        int max_fuse, int landing, unsigned seed, int threaded, int repeats, void* rep);
int sim_record_replay(int algo, int dtype, int world, const void* const* sendbufs, void* const* recvbufs, size_t len,
                      int rank, int max_fuse, int landing, unsigned seed, void* replay_out, int replays, void* rep);
int sim_failures(void);
int sim_rendezvous(void);
int sim_p2p(void);
}

int main(int argc, char** argv) {
  const int iterations = argc > 1 ? atoi(argv[1]) : 100;
  const bool all_threaded = argc > 2 && atoi(argv[2]) != 0;
  const bool extras = !(argc > 3 && atoi(argv[3]) == 0);
  std::mt19937 rng(7);
  int bad = 0, runs = 0;
  static char report[1 << 16];  // sim_report, larger than needed
  for (int it = 0; it < iterations; it++) {
    const int algo = rng() % 2;
    const int ring_worlds[] = {2, 3, 4, 5, 8}, halving_worlds[] = {2, 4, 8, 16};
    const int world = algo ? halving_worlds[rng() % 4] : ring_worlds[rng() % 5];
    size_t n;
    if (rng() % 2) {  // 256-byte chunks in aligned buffers: pool slots lie back to back and chunks merge
      n = static_cast<size_t>(world) * (2 + rng() % 40) * 64 + (rng() % 3 ? 0 : 5);
      setenv("IBCOMM_CHUNKSIZE", "256", 1);
    } else {
      n = world + rng() % 5000;
      unsetenv("IBCOMM_CHUNKSIZE");
    }
    setenv("IBCOMM_MEMORY_POOL_PRE_ALLOC", (rng() % 2) ? "4096" : "1048576", 1);
    std::vector<std::vector<float>> send(world, std::vector<float>(n)), recv(world, std::vector<float>(n));
    for (auto& v : send)
      for (auto& x : v) x = static_cast<float>(rng() % 1000) / 7.0f;
    std::vector<const void*> sp(world);
    std::vector<void*> rp(world);
    for (int i = 0; i < world; i++) {
      sp[i] = send[i].data();
      rp[i] = recv[i].data();
    }
    const int fuse = (rng() % 2) ? 64 : 1 + rng() % 64, landing = rng() % 4;
    // single-threaded worlds: every third one issues on one stream with its ranks' launches merged, as a recording does
    const int threaded = (all_threaded || rng() % 5 == 0) ? 1 + it % 2 : (it % 3 == 0 ? 3 : 0);
    int rc = sim_world_allreduce(algo, 0, world, sp.data(), rp.data(), n, fuse, landing, it, threaded, 1 + rng() % 2, report);
    runs++;
    if (rc != 0) {
      bad++;
      printf("allreduce returned %d (algo %d, world %d, n %zu, fuse %d, landing %d)\n", rc, algo, world, n, fuse, landing);
    }
    if (it % 4 == 0) {
      std::vector<float> out(n);
      rc = sim_record_replay(algo, 0, world, sp.data(), rp.data(), n, rng() % world, fuse, landing, it, out.data(), 2, report);
      runs++;
      if (rc != 0) {
        bad++;
        printf("record/replay returned %d (algo %d, world %d, n %zu)\n", rc, algo, world, n);
      }
    }
  }
  unsetenv("IBCOMM_CHUNKSIZE");
  unsetenv("IBCOMM_MEMORY_POOL_PRE_ALLOC");
  const int failures_held = extras ? sim_failures() : 4095, p2p_held = extras ? sim_p2p() : 2047;
  const int meeting_held = sim_rendezvous();  // threads by nature: also in the run that skips the other extras
  if (failures_held != 4095 || p2p_held != 2047 || meeting_held != 255) {
    bad++;
    printf("failure-handling checks %d of 4095, point-to-point checks %d of 2047, meeting checks %d of 255\n", failures_held, p2p_held,
           meeting_held);
  }
  printf("runs %d bad %d\n", runs, bad);
  return bad != 0;
}
