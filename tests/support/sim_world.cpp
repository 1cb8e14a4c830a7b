// C entry points that run the allreduce engine on the simulated device (see sim_backend.hpp).
// TEST INFRASTRUCTURE ONLY.
#include <string.h>

#include <chrono>
#include <memory>
#include <string>
#include <thread>
#include <vector>

#include "sim_backend.hpp"
#include "engine.hpp"
#include "rendezvous.hpp"
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
  long launches_collected;  // threaded == 3: launches the ranks handed to the collector ...
  long launches_issued;     // ... and launches it put on the stream
};

// threaded = 0: one thread steps all ranks (RunWorld); 1: one thread per rank, each running its own
// engine (AllreduceBlocking); 2: one thread per rank, the calls meet and the last to arrive steps all
// ranks (Rendezvous, what the library's blocking per-rank entry points do); 3: one thread steps all ranks, all
// of them issuing on ONE stream with their launches merged across ranks (what a recording of a world does).
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
  Rendezvous meet(world);
  LaunchCollector<SimBackend> collector;
  SimBackend::Stream one = nullptr;
  for (int k = 0; k < repeats && rc == kOk; k++) {
    if (threaded == 3) {
      if (!one) SimBackend::StreamCreate(&one);
      for (auto* c : raw) c->pool().OverrideStream(one);
      rc = RunWorld<SimBackend>(raw.data(), world, algo, dtype, sendbufs, recvbufs, len, false, &collector);
      for (auto* c : raw) c->pool().ClearOverride();
      SimBackend::StreamSynchronize(one);
      if (rc != kOk) snprintf(rep->error, sizeof rep->error, "%s", LastErrorBuffer());
    } else if (!threaded) {
      rc = RunWorld<SimBackend>(raw.data(), world, algo, dtype, sendbufs, recvbufs, len, true);
      if (rc != kOk) snprintf(rep->error, sizeof rep->error, "%s", LastErrorBuffer());
    } else {
      std::vector<int> rcs(world, 0);
      std::vector<std::string> msgs(world);
      std::vector<std::thread> th;
      for (int r = 0; r < world; r++) {
        th.emplace_back([&, r]() {
          if (threaded == 2) {
            RankCall call;
            call.comm = raw[r];
            call.algo = algo;
            call.dtype = dtype;
            call.sendbuf = sendbufs[r];
            call.recvbuf = recvbufs[r];
            call.len = len;
            rcs[r] = meet.Arrive(r, call, 60.0, &fabric, [&](const RankCall* calls) {
              std::vector<Communicator<SimBackend>*> cs(world);
              std::vector<const void*> sp(world);
              std::vector<void*> rp(world);
              for (int i = 0; i < world; i++) {
                cs[i] = static_cast<Communicator<SimBackend>*>(calls[i].comm);
                sp[i] = calls[i].sendbuf;
                rp[i] = calls[i].recvbuf;
              }
              return RunWorld<SimBackend>(cs.data(), world, calls[0].algo, calls[0].dtype, sp.data(), rp.data(), calls[0].len, true);
            });
          } else {
            rcs[r] = raw[r]->AllreduceBlocking(algo, dtype, sendbufs[r], recvbufs[r], len);
          }
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
  rep->races = threaded == 1 ? -1 : Sim::Get().CheckRaces(&first);
  rep->unrecorded_waits = Sim::Get().unrecorded_waits();
  if (!raw.empty()) rep->rank0 = raw[0]->stats();
  snprintf(rep->first_race, sizeof rep->first_race, "%s", first.c_str());
  rep->launches_collected = static_cast<long>(collector.collected());
  rep->launches_issued = static_cast<long>(collector.issued());
  if (one) SimBackend::StreamDestroy(one);
  return rc;
}

// Failure handling, forced from the host; returns a bit per check that held.
int sim_failures(void) {
  Sim::Get().Reset(9);
  int held = 0;
  std::vector<float> a(4096, 1.0f), b(4096, 2.0f), ra(4096), rb(4096);
  {
    // a rank whose peer never shows up gives up after IBCOMM_HIP_TIMEOUT_S with a transport error
    Fabric<SimBackend> fabric(2);
    Communicator<SimBackend> c0(&fabric, 2), c1(&fabric, 2);
    c0.Init(); c1.Init();
    c0.RegisterMyself(0); c1.RegisterMyself(1);
    setenv("IBCOMM_HIP_TIMEOUT_S", "0.2", 1);
    const int rc = c0.AllreduceBlocking(kRing, kF32, a.data(), ra.data(), a.size());
    unsetenv("IBCOMM_HIP_TIMEOUT_S");
    if (rc == kTransportError && !c0.active()) held |= 1;
    // what that rank had posted is still in the channels: the world refuses further collectives ...
    if (fabric.poisoned() && c1.Begin(kRing, kF32, b.data(), rb.data(), a.size()) == kTransportError &&
        strstr(LastErrorBuffer(), "abandoned") != nullptr)
      held |= 1024;
    fabric.Reset();
    // ... until its owner resets it; then the communicators are usable again
    const void* sends[2] = {a.data(), b.data()};
    void* recvs[2] = {ra.data(), rb.data()};
    Communicator<SimBackend>* cs[2] = {&c0, &c1};
    if (RunWorld<SimBackend>(cs, 2, kRing, kF32, sends, recvs, a.size(), true) == kOk && ra[7] == 3.0f && rb[4095] == 3.0f) held |= 2;
  }
  {
    // three ranks, one never joins: the first to lose patience (0.3 s) marks the world, and the other
    // stops waiting at once instead of sitting out its own, much longer, time limit (30 s)
    Fabric<SimBackend> fabric(3);
    Communicator<SimBackend> c0(&fabric, 3), c1(&fabric, 3);
    c0.Init(); c1.Init();
    c0.RegisterMyself(0); c1.RegisterMyself(1);
    std::vector<float> rc_buf(4096);
    int r0 = 0, r1 = 0;
    std::string m1;
    const auto t0 = std::chrono::steady_clock::now();
    setenv("IBCOMM_HIP_TIMEOUT_S", "0.3", 1);
    std::thread t([&]() { r0 = c0.AllreduceBlocking(kRing, kF32, a.data(), ra.data(), a.size()); });
    std::this_thread::sleep_for(std::chrono::milliseconds(100));  // rank 0 has read its limit by now
    setenv("IBCOMM_HIP_TIMEOUT_S", "30", 1);
    r1 = c1.AllreduceBlocking(kRing, kF32, b.data(), rb.data(), b.size());
    m1 = LastErrorBuffer();
    t.join();
    unsetenv("IBCOMM_HIP_TIMEOUT_S");
    const double took = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (r0 == kTransportError && r1 == kTransportError && took < 5.0 && m1.find("gave up") != std::string::npos) held |= 2048;
  }
  {
    // ranks that disagree about the buffer length: the first mismatching message is a transport error
    Fabric<SimBackend> fabric(2);
    Communicator<SimBackend> c0(&fabric, 2), c1(&fabric, 2);
    c0.Init(); c1.Init();
    c0.RegisterMyself(0); c1.RegisterMyself(1);
    int rc = c0.Begin(kRing, kF32, a.data(), ra.data(), 4096);
    if (rc == kOk) rc = c1.Begin(kRing, kF32, b.data(), rb.data(), 2048);
    bool p = false, f = false;
    int r0 = kOk, r1 = kOk;
    for (int k = 0; k < 8 && r0 == kOk && r1 == kOk; k++) {
      r0 = c0.Progress(&p, &f);
      if (r0 == kOk) r1 = c1.Progress(&p, &f);
    }
    if (rc == kOk && (r0 == kTransportError || r1 == kTransportError)) held |= 4;
    c0.Abort(); c1.Abort();
  }
  {
    // a second collective on a communicator that is still inside one is refused (NOT_SUPPORTED)
    Fabric<SimBackend> fabric(2);
    Communicator<SimBackend> c0(&fabric, 2);
    c0.Init(); c0.RegisterMyself(0);
    if (c0.Begin(kRing, kF32, a.data(), ra.data(), 4096) == kOk &&
        c0.Begin(kRing, kF32, a.data(), ra.data(), 4096) == kNotSupported) held |= 8;
    // point-to-point calls are refused while it runs
    if (c0.Send(1, a.data(), 4, false) == kNotSupported) held |= 16;
    c0.Abort();
    // partially overlapping buffers and null pointers are invalid arguments
    if (c0.Begin(kRing, kF32, a.data(), a.data() + 8, 2048) == kInvalidArgument &&
        c0.Begin(kRing, kF32, nullptr, ra.data(), 2048) == kInvalidArgument &&
        c0.Begin(kRing, 99, a.data(), ra.data(), 2048) == kInvalidArgument) held |= 32;
  }
  {
    // a replay needs a recording of the same rank and the same call
    Fabric<SimBackend> fabric(2);
    Communicator<SimBackend> c0(&fabric, 2), c1(&fabric, 2);
    c0.Init(); c1.Init();
    c0.RegisterMyself(0); c1.RegisterMyself(1);
    Communicator<SimBackend>* cs[2] = {&c0, &c1};
    const void* sends[2] = {a.data(), b.data()};
    void* recvs[2] = {ra.data(), rb.data()};
    if (!fabric.StartReplay(0)) held |= 64;  // nothing recorded yet
    size_t bytes = 0;
    c0.RecordingBytes(kRing, kF32, 4096, &bytes);
    fabric.StartRecording(0, bytes);
    int rc = RunWorld<SimBackend>(cs, 2, kRing, kF32, sends, recvs, 4096, true);
    fabric.StopRecording();
    if (rc == kOk && !fabric.StartReplay(1)) held |= 128;  // recorded rank 0, not rank 1
    if (fabric.StartReplay(0)) {
      std::vector<float> out(4096);
      // a different length: the first recorded message does not fit the plan
      rc = RunAlone<SimBackend>(&c0, kRing, kF32, a.data(), out.data(), 2048, true);
      if (rc == kTransportError && !c0.active()) held |= 256;
      // the right call still replays afterwards
      rc = RunAlone<SimBackend>(&c0, kRing, kF32, a.data(), out.data(), 4096, true);
      if (rc == kOk && out[100] == 3.0f) held |= 512;
      fabric.StopReplay();
    }
  }
  return held;
}

// The meeting of blocking per-rank calls, forced from the host; returns a bit per check that held.
int sim_rendezvous(void) {
  Sim::Get().Reset(11);
  int held = 0;
  std::vector<float> a(4096, 1.0f), b(4096, 2.0f), c(4096, 4.0f), ra(4096), rb(4096), rc_buf(4096);
  auto call_of = [](void* comm, int algo, const void* s, void* r, size_t n) {
    RankCall k;
    k.comm = comm;
    k.algo = algo;
    k.dtype = kF32;
    k.sendbuf = s;
    k.recvbuf = r;
    k.len = n;
    return k;
  };
  Fabric<SimBackend> fabric(3);
  Communicator<SimBackend> c0(&fabric, 3), c1(&fabric, 3), c2(&fabric, 3);
  Communicator<SimBackend>* cs[3] = {&c0, &c1, &c2};
  for (int r = 0; r < 3; r++) {
    cs[r]->Init();
    cs[r]->RegisterMyself(r);
  }
  Rendezvous meet(3);
  int drives = 0;
  auto drive = [&](const RankCall* calls) {
    drives++;
    Communicator<SimBackend>* w[3];
    const void* sp[3];
    void* rp[3];
    for (int i = 0; i < 3; i++) {
      w[i] = static_cast<Communicator<SimBackend>*>(calls[i].comm);
      sp[i] = calls[i].sendbuf;
      rp[i] = calls[i].recvbuf;
    }
    return RunWorld<SimBackend>(w, 3, calls[0].algo, calls[0].dtype, sp, rp, calls[0].len, true);
  };
  {
    // three ranks meet, five rounds in a row; one thread drives each round, all get its status
    int r[3] = {-1, -1, -1};
    bool ok = true;
    for (int round = 0; round < 5 && ok; round++) {
      std::thread t1([&]() { r[1] = meet.Arrive(1, call_of(&c1, kRing, b.data(), rb.data(), 4096), 30.0, &fabric, drive); });
      std::thread t2([&]() { r[2] = meet.Arrive(2, call_of(&c2, kRing, c.data(), rc_buf.data(), 4096), 30.0, &fabric, drive); });
      r[0] = meet.Arrive(0, call_of(&c0, kRing, a.data(), ra.data(), 4096), 30.0, &fabric, drive);
      t1.join();
      t2.join();
      ok = r[0] == kOk && r[1] == kOk && r[2] == kOk && ra[5] == 7.0f && rb[4095] == 7.0f && rc_buf[0] == 7.0f;
    }
    if (ok && drives == 5 && meet.rounds() == 5) held |= 1;
  }
  {
    // ranks that disagree about the length are all told so, with the message in each thread's buffer
    int r[3] = {-1, -1, -1};
    std::string m1;
    const int before = drives;
    std::thread t1([&]() {
      r[1] = meet.Arrive(1, call_of(&c1, kRing, b.data(), rb.data(), 2048), 30.0, &fabric, drive);
      m1 = LastErrorBuffer();
    });
    std::thread t2([&]() { r[2] = meet.Arrive(2, call_of(&c2, kRing, c.data(), rc_buf.data(), 4096), 30.0, &fabric, drive); });
    r[0] = meet.Arrive(0, call_of(&c0, kRing, a.data(), ra.data(), 4096), 30.0, &fabric, drive);
    t1.join();
    t2.join();
    if (r[0] == kInvalidArgument && r[1] == kInvalidArgument && r[2] == kInvalidArgument && drives == before &&
        m1.find("rank 1 entered") != std::string::npos)
      held |= 2;
  }
  {
    // a failure inside the collective (a world the algorithm does not support) reaches every rank, and
    // the world stays usable: the driver cleans up after itself
    int r[3] = {-1, -1, -1};
    std::thread t1([&]() { r[1] = meet.Arrive(1, call_of(&c1, kRabenseifner, b.data(), rb.data(), 4096), 30.0, &fabric, drive); });
    std::thread t2([&]() { r[2] = meet.Arrive(2, call_of(&c2, kRabenseifner, c.data(), rc_buf.data(), 4096), 30.0, &fabric, drive); });
    r[0] = meet.Arrive(0, call_of(&c0, kRabenseifner, a.data(), ra.data(), 4096), 30.0, &fabric, drive);
    t1.join();
    t2.join();
    if (r[0] == kNotSupported && r[1] == kNotSupported && r[2] == kNotSupported && !fabric.poisoned() && !c0.active()) held |= 4;
  }
  {
    // the same rank twice in one round is refused
    std::thread t1([&]() { (void)meet.Arrive(1, call_of(&c1, kRing, b.data(), rb.data(), 4096), 0.5, &fabric, drive); });
    std::this_thread::sleep_for(std::chrono::milliseconds(100));
    if (meet.Arrive(1, call_of(&c1, kRing, b.data(), rb.data(), 4096), 0.5, &fabric, drive) == kNotSupported) held |= 8;
    t1.join();  // gives up after its 0.5 s and marks the world
    if (fabric.poisoned()) held |= 16;
    // an abandoned world refuses further meetings until its owner resets it
    if (meet.Arrive(0, call_of(&c0, kRing, a.data(), ra.data(), 4096), 0.5, &fabric, drive) == kTransportError &&
        strstr(LastErrorBuffer(), "abandoned") != nullptr)
      held |= 32;
    fabric.Reset();
  }
  {
    // one rank never comes: the first to lose patience (0.3 s) marks the world and the other stops
    // waiting at once instead of sitting out its own limit (30 s); nothing was driven
    int r0 = -1, r1 = -1;
    std::string m1;
    const int before = drives;
    const auto t0 = std::chrono::steady_clock::now();
    std::thread t([&]() { r0 = meet.Arrive(0, call_of(&c0, kRing, a.data(), ra.data(), 4096), 0.3, &fabric, drive); });
    r1 = meet.Arrive(1, call_of(&c1, kRing, b.data(), rb.data(), 4096), 30.0, &fabric, drive);
    m1 = LastErrorBuffer();
    t.join();
    const double took = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (r0 == kTransportError && r1 == kTransportError && took < 5.0 && m1.find("gave up") != std::string::npos && drives == before)
      held |= 64;
    fabric.Reset();
    // after the reset the three meet again
    int r[3] = {-1, -1, -1};
    std::thread t1([&]() { r[1] = meet.Arrive(1, call_of(&c1, kRing, b.data(), rb.data(), 4096), 30.0, &fabric, drive); });
    std::thread t2([&]() { r[2] = meet.Arrive(2, call_of(&c2, kRing, c.data(), rc_buf.data(), 4096), 30.0, &fabric, drive); });
    r[0] = meet.Arrive(0, call_of(&c0, kRing, a.data(), ra.data(), 4096), 30.0, &fabric, drive);
    t1.join();
    t2.join();
    if (r[0] == kOk && r[1] == kOk && r[2] == kOk && ra[9] == 7.0f) held |= 128;
  }
  return held;
}

// Point-to-point scenarios on host buffers; returns a bit per check that held.
int sim_p2p(void) {
  Sim::Get().Reset(5);
  const int world = 4;
  Fabric<SimBackend> fabric(world);
  std::vector<std::unique_ptr<Communicator<SimBackend>>> comms;
  for (int r = 0; r < world; r++) {
    comms.emplace_back(new Communicator<SimBackend>(&fabric, world));
    if (comms.back()->Init() != kOk) return -1;
    comms.back()->RegisterMyself(r);
  }
  int held = 0;
  // ping-pong as in tests/sendrecv_test.cpp: non-blocking Send, blocking Recv, SendWait
  int value = 10, value2 = -1;
  bool ok = false;
  if (comms[0]->Send(1, &value, sizeof value, false) == kOk && comms[1]->Recv(0, &value2, sizeof value2, true) == kOk &&
      comms[0]->SendWait(1) == kOk && value2 == 10)
    held |= 1;
  value2 = -7;
  if (comms[1]->Send(0, &value2, sizeof value2, false) == kOk && comms[0]->Recv(1, &value, sizeof value, true) == kOk &&
      comms[1]->SendWait(0) == kOk && value == -7)
    held |= 2;
  // a second non-blocking send before SendWait is refused with NOT_SUPPORTED; so is a second Recv
  int a = 1, b = 2, c = 0, d = 0;
  if (comms[2]->Send(3, &a, sizeof a, false) == kOk && comms[2]->Send(3, &b, sizeof b, false) == kNotSupported) held |= 4;
  if (comms[3]->Recv(2, &c, sizeof c, false) == kOk && comms[3]->Recv(2, &d, sizeof d, false) == kNotSupported) held |= 8;
  // polls: nothing before the data has been moved, exactly one completion afterwards
  if (comms[2]->SendPoll(3, &ok) == kOk && !ok) held |= 16;
  if (comms[3]->RecvPoll(2, &ok) == kOk && ok && c == 1 && comms[3]->RecvPoll(2, &ok) == kOk && !ok) held |= 32;
  if (comms[2]->SendPoll(3, &ok) == kOk && ok && comms[2]->SendPoll(3, &ok) == kOk && !ok) held |= 64;
  // messages between a pair are delivered in order
  int seq[3] = {5, 6, 7}, got[3] = {0, 0, 0};
  bool fifo = true;
  for (int k = 0; k < 3; k++) {
    fifo = fifo && comms[0]->Send(2, &seq[k], sizeof(int), false) == kOk && comms[2]->Recv(0, &got[k], sizeof(int), true) == kOk &&
           comms[0]->SendWait(2) == kOk;
  }
  if (fifo && got[0] == 5 && got[1] == 6 && got[2] == 7) held |= 128;
  // a message larger than the posted buffer is a transport error; bad ranks are invalid arguments
  long big = 1;
  char small_buf = 0;
  if (comms[0]->Send(1, &big, sizeof big, false) == kOk && comms[1]->Recv(0, &small_buf, 1, false) == kOk &&
      comms[1]->RecvPoll(0, &ok) == kTransportError)
    held |= 256;
  if (comms[0]->Send(9, &a, 4, false) == kInvalidArgument && comms[0]->Recv(-1, &a, 4, false) == kInvalidArgument) held |= 512;
  // broadcast from rank 1 with one thread per rank
  std::vector<int> vals(world, 0);
  vals[1] = 4242;
  Fabric<SimBackend> fabric2(world);
  std::vector<std::unique_ptr<Communicator<SimBackend>>> c2;
  for (int r = 0; r < world; r++) {
    c2.emplace_back(new Communicator<SimBackend>(&fabric2, world));
    c2.back()->Init();
    c2.back()->RegisterMyself(r);
  }
  std::vector<std::thread> th;
  std::vector<int> rcs(world, -1);
  for (int r = 0; r < world; r++) th.emplace_back([&, r]() { rcs[r] = c2[r]->Bcast(&vals[r], sizeof(int), 1); });
  for (auto& t : th) t.join();
  bool bc = true;
  for (int r = 0; r < world; r++) bc = bc && rcs[r] == kOk && vals[r] == 4242;
  if (bc) held |= 1024;
  return held;
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
  int rc2 = c.pool().GetController(chunk_bytes, true, false, &a);
  if (rc2 != kOk) return rc2;
  *slots_for_chunk = static_cast<int>(a.slot_count());
  *second_controller = c.pool().GetController(chunk_bytes, true, false, &b);
  a.Release();
  rc2 = c.pool().GetController(chunk_bytes, true, false, &b);  // free again after release
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
  bool descending = false;
  if (rc == kOk) rc = raw[rank]->RecordingBytes(algo, dtype, len, &log_bytes, &descending);
  if (rc == kOk) rc = fabric.StartRecording(rank, log_bytes, descending);
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
