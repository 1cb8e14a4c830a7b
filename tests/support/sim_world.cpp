// C entry points that run the allreduce engine on the simulated device (see sim_backend.hpp).
// TEST INFRASTRUCTURE ONLY.
#include <memory>
#include <string>
#include <thread>
#include <vector>

#include "sim_backend.hpp"
#include "engine.hpp"
#include "world.hpp"

using namespace ibcomm_hip;
using ibcomm_sim::Sim;
using ibcomm_sim::SimBackend;

extern "C" {

struct sim_report {
  int rc;
  long nodes;
  long races;             // -1: graph too large to check
  long unrecorded_waits;
  EngineStats rank0;
  char error[512];
  char first_race[256];
};

// threaded = 0: one thread steps all ranks (RunWorld); 1: one thread per rank (AllreduceBlocking).
// repeats > 1 runs the same collective again on the same communicators (event/slot reuse).
int sim_world_allreduce(int algo, int dtype, int world, const void* const* sendbufs, void* const* recvbufs, size_t len,
                        int max_fuse, int landing, unsigned seed, int threaded, int repeats, sim_report* rep) {
  *rep = sim_report();
  Sim::Get().Reset(seed);
  Fabric<SimBackend> fabric(world);
  std::vector<std::unique_ptr<Communicator<SimBackend>>> comms;
  std::vector<Communicator<SimBackend>*> raw;
  int rc = kOk;
  for (int r = 0; r < world && rc == kOk; r++) {
    comms.emplace_back(new Communicator<SimBackend>(&fabric, world));
    rc = comms.back()->Init();
    comms.back()->RegisterMyself(r);
    comms.back()->set_max_fuse(max_fuse);
    comms.back()->set_landing(landing);
    raw.push_back(comms.back().get());
  }
  for (int k = 0; k < repeats && rc == kOk; k++) {
    if (!threaded) {
      rc = RunWorld<SimBackend>(raw.data(), world, algo, dtype, sendbufs, recvbufs, len, true);
      if (rc != kOk) snprintf(rep->error, sizeof rep->error, "%s", LastErrorBuffer());
    } else {
      std::vector<int> rcs(world, 0);
      std::vector<std::string> msgs(world);
      std::vector<std::thread> th;
      for (int r = 0; r < world; r++) {
        th.emplace_back([&, r]() {
          rcs[r] = raw[r]->AllreduceBlocking(algo, dtype, sendbufs[r], recvbufs[r], len);
          if (rcs[r]) msgs[r] = LastErrorBuffer();
        });
      }
      for (auto& t : th) t.join();
      for (int r = 0; r < world; r++) {
        if (rcs[r] && rc == kOk) {
          rc = rcs[r];
          snprintf(rep->error, sizeof rep->error, "%s", msgs[r].c_str());
        }
      }
    }
  }
  if (rc != kOk && !rep->error[0]) snprintf(rep->error, sizeof rep->error, "%s", LastErrorBuffer());
  std::string first;
  rep->rc = rc;
  rep->nodes = Sim::Get().node_count();
  rep->races = threaded ? -1 : Sim::Get().CheckRaces(&first);
  rep->unrecorded_waits = Sim::Get().unrecorded_waits();
  if (!raw.empty()) rep->rank0 = raw[0]->stats();
  snprintf(rep->first_race, sizeof rep->first_race, "%s", first.c_str());
  return rc;
}

// Runs one world allreduce with tracing on and dumps rank 0's trace to `path`.
int sim_trace(int algo, int world, const void* const* sendbufs, void* const* recvbufs, size_t len, int max_fuse,
              const char* path, unsigned long long* pairs /* 7 */) {
  Sim::Get().Reset(3);
  Fabric<SimBackend> fabric(world);
  std::vector<std::unique_ptr<Communicator<SimBackend>>> comms;
  std::vector<Communicator<SimBackend>*> raw;
  for (int r = 0; r < world; r++) {
    comms.emplace_back(new Communicator<SimBackend>(&fabric, world));
    if (comms.back()->Init() != kOk) return 1;
    comms.back()->RegisterMyself(r);
    comms.back()->set_max_fuse(max_fuse);
    comms.back()->trace().Enable(true);
    comms.back()->trace().SetTimerBase();
    raw.push_back(comms.back().get());
  }
  const int rc = RunWorld<SimBackend>(raw.data(), world, algo, kF32, sendbufs, recvbufs, len, true);
  if (rc != kOk) return rc;
  for (int c = 0; c < Trace::kCategories; c++) pairs[c] = raw[0]->trace().pairs(static_cast<Trace::Category>(c));
  return raw[0]->trace().Dump(path) ? kOk : 1;
}

// Pool knobs and controller rules (memory_pool.h:111-121, 139-173): returns the status of creating a
// communicator under the current environment, and in *second_controller the status of asking the
// pool for a second controller while one is live.
int sim_pool_rules(int* second_controller, unsigned long long* block_bytes, int* max_streams, int* slots_for_chunk,
                   unsigned long long chunk_bytes) {
  Sim::Get().Reset(1);
  Fabric<SimBackend> fabric(2);
  Communicator<SimBackend> c(&fabric, 2);
  const int rc = c.Init();
  if (rc != kOk) return rc;
  *block_bytes = c.pool().block_bytes();
  *max_streams = c.pool().max_streams();
  MemoryController<SimBackend> a, b;
  int rc2 = c.pool().GetController(chunk_bytes, &a);
  if (rc2 != kOk) return rc2;
  *slots_for_chunk = static_cast<int>(a.slot_count());
  *second_controller = c.pool().GetController(chunk_bytes, &b);
  a.Release();
  rc2 = c.pool().GetController(chunk_bytes, &b);  // free again after release
  b.Release();
  return rc2;
}

// Records `rank`'s incoming traffic during one world run, then runs that rank alone `replays` times
// against the recording, writing its result to replay_out.
int sim_record_replay(int algo, int dtype, int world, const void* const* sendbufs, void* const* recvbufs, size_t len,
                      int rank, int max_fuse, int landing, unsigned seed, void* replay_out, int replays, sim_report* rep) {
  *rep = sim_report();
  Sim::Get().Reset(seed);
  Fabric<SimBackend> fabric(world);
  std::vector<std::unique_ptr<Communicator<SimBackend>>> comms;
  std::vector<Communicator<SimBackend>*> raw;
  int rc = kOk;
  for (int r = 0; r < world && rc == kOk; r++) {
    comms.emplace_back(new Communicator<SimBackend>(&fabric, world));
    rc = comms.back()->Init();
    comms.back()->RegisterMyself(r);
    comms.back()->set_max_fuse(max_fuse);
    comms.back()->set_landing(landing);
    raw.push_back(comms.back().get());
  }
  size_t log_bytes = 0;
  if (rc == kOk) rc = raw[rank]->RecordingBytes(algo, dtype, len, &log_bytes);
  if (rc == kOk) rc = fabric.StartRecording(rank, log_bytes);
  if (rc == kOk) rc = RunWorld<SimBackend>(raw.data(), world, algo, dtype, sendbufs, recvbufs, len, true);
  fabric.StopRecording();
  raw[rank]->reset_stats();
  for (int k = 0; k < replays && rc == kOk; k++) {
    if (!fabric.StartReplay(rank)) rc = Fail(kInvalidArgument, "nothing recorded");
    if (rc == kOk) rc = RunAlone<SimBackend>(raw[rank], algo, dtype, sendbufs[rank], replay_out, len, true);
    fabric.StopReplay();
  }
  if (rc != kOk) snprintf(rep->error, sizeof rep->error, "%s", LastErrorBuffer());
  std::string first;
  rep->rc = rc;
  rep->nodes = Sim::Get().node_count();
  rep->races = Sim::Get().CheckRaces(&first);
  rep->unrecorded_waits = Sim::Get().unrecorded_waits();
  rep->rank0 = raw[rank]->stats();
  snprintf(rep->first_race, sizeof rep->first_race, "%s", first.c_str());
  return rc;
}

}  // extern "C"
