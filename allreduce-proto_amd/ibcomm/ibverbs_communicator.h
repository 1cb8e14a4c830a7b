// Drop-in for PFNProto's ibcomm/ibverbs_communicator.h on one MI355X.
//
// Same class name, constructor, connection-management calls and allreduce member templates as the
// reference (ibcomm/ibverbs_communicator.h:59-123), implemented over the C ABI of libibcomm_hip.so.
// The InfiniBand network is replaced by an in-process loopback: every communicator constructed with
// the same world size in one process joins the same loopback world, and each emulated rank calls the
// blocking allreduce from a thread of its own, the way each process does in the reference.
//
//   IBVerbsCommunicator comm(world_size);          // ibverbs_communicator.cpp:24-99
//   comm.RegisterMyself(rank);                     // :355-357
//   comm.AllreduceRingCuda(send_dev, recv_dev, n); // allreduce_cuda_impl.h:35-301
//
// Failures behave as in the reference: a message on stderr and exit(code) with the codes of
// ibcomm/util.h:32-42.  Element types: float, double, 32- and 64-bit integers.
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <map>
#include <mutex>
#include <type_traits>
#include <vector>

#include "ibcomm/util.h"
#include "ibcomm_hip.h"

struct ProcessInfo {  // ibverbs_communicator.h:23-27; carries nothing over the loopback
  uint16_t lid;
  uint32_t qp_n;
  uint32_t psn;
};

class IBVerbsCommunicator {
 public:
  IBVerbsCommunicator() {}
  explicit IBVerbsCommunicator(int world_size) { Init(world_size); }
  IBVerbsCommunicator(const IBVerbsCommunicator&) = delete;
  IBVerbsCommunicator& operator=(const IBVerbsCommunicator&) = delete;
  IBVerbsCommunicator(IBVerbsCommunicator&&) = delete;
  IBVerbsCommunicator& operator=(IBVerbsCommunicator&&) = delete;

  ~IBVerbsCommunicator() {
    for (ibcomm_hip_comm* c : loop_comms_) ibcomm_hip_comm_destroy(c);
    if (loop_fabric_) ibcomm_hip_fabric_destroy(loop_fabric_);
    if (!comm_) return;
    Registry& reg = registry();
    std::lock_guard<std::mutex> lock(reg.mu);
    ibcomm_hip_comm_destroy(comm_);
    World& w = reg.worlds[world_size_];
    if (--w.users == 0) {
      ibcomm_hip_fabric_destroy(w.fabric);
      reg.worlds.erase(world_size_);
    }
  }

  void Init(int world_size) {
    if (comm_) {
      util::IbcommWarning(__FILE__, __LINE__, "IBVerbsCommunicator is already initialized.");
      return;
    }
    Registry& reg = registry();
    std::lock_guard<std::mutex> lock(reg.mu);
    World& w = reg.worlds[world_size];
    if (!w.fabric) Check(ibcomm_hip_fabric_create(world_size, &w.fabric), __LINE__);
    Check(ibcomm_hip_comm_create(w.fabric, world_size, &comm_), __LINE__);
    w.users++;
    world_size_ = world_size;
    static std::atomic<uint16_t> next_id{1};
    id_ = next_id++;
    wired_to_.assign(world_size, -1);
  }

  // Queue-pair bring-up (ibverbs_communicator.cpp:286-353).  Between communicators of one process there
  // is nothing to exchange: ranks find each other through the loopback world.  The information
  // returned still names the endpoint (this communicator, the peer index the pair stands for), so
  // that the one wiring the loopback cannot provide by itself keeps working: a communicator
  // connecting two of its own queue pairs to each other, as the reference's tests/sendrecv_test.cpp
  // does (pair 1 to pair 0 of the same object: what is sent "to 0" is received "from 1").
  struct ProcessInfo CreateQueuePair(int dest_rank) {
    return ProcessInfo{id_, static_cast<uint32_t>(dest_rank), 0};
  }
  struct ProcessInfo RegisterProcess(int dest_rank, struct ProcessInfo pinfo) {
    RegisterQueuePair(dest_rank, pinfo);
    return CreateQueuePair(dest_rank);
  }
  void RegisterQueuePair(int dest_rank, struct ProcessInfo pinfo) {
    if (pinfo.lid != id_) return;  // a pair of another communicator: the loopback world connects the two
    if (dest_rank < 0 || dest_rank >= world_size_ || pinfo.qp_n >= static_cast<uint32_t>(world_size_))
      util::IbcommError(__FILE__, __LINE__, util::IBCOMM_ERROR_CODE::INVALID_ARGUMENT, "queue pair index outside the world");
    wired_to_[dest_rank] = static_cast<int>(pinfo.qp_n);
    wired_to_[pinfo.qp_n] = dest_rank;
  }
  void RegisterMyself(int my_rank) {
    my_rank_ = my_rank;
    Check(ibcomm_hip_comm_register_myself(comm_, my_rank), __LINE__);
  }

  // Point-to-point messaging over the loopback (ibverbs_communicator.cpp:371-606); host or device buffers.
  void Send(int dest_rank, const void* buf, size_t len, bool blocking = true) {
    Check(ibcomm_hip_send(Endpoint(dest_rank), dest_rank, buf, len, blocking ? 1 : 0), __LINE__);
  }
  void Recv(int src_rank, void* buf, size_t len, bool blocking = true) {
    Check(ibcomm_hip_recv(Endpoint(src_rank), src_rank, buf, len, blocking ? 1 : 0), __LINE__);
  }
  bool SendPoll(int dest_rank) {
    int done = 0;
    Check(ibcomm_hip_send_poll(Endpoint(dest_rank), dest_rank, &done), __LINE__);
    return done != 0;
  }
  bool RecvPoll(int src_rank) {
    int done = 0;
    Check(ibcomm_hip_recv_poll(Endpoint(src_rank), src_rank, &done), __LINE__);
    return done != 0;
  }
  void SendWait(int dest_rank) { Check(ibcomm_hip_send_wait(Endpoint(dest_rank), dest_rank), __LINE__); }
  void RecvWait(int src_rank) { Check(ibcomm_hip_recv_wait(Endpoint(src_rank), src_rank), __LINE__); }
  void Bcast(void* buf, size_t len, int root) { Check(ibcomm_hip_bcast(comm_, buf, len, root), __LINE__); }

  // Device buffers.  Blocking; every rank of the world must be inside the same call.
  template <typename T>
  void AllreduceRingCuda(const T* sendbuf, T* recvbuf, size_t len_elements) {
    Check(ibcomm_hip_allreduce_ring(comm_, DType<T>(), sendbuf, recvbuf, len_elements), __LINE__);
  }
  template <typename T>
  void AllreduceRabenseifnerCuda(const T* sendbuf, T* recvbuf, size_t len_elements) {
    Check(ibcomm_hip_allreduce_rabenseifner(comm_, DType<T>(), sendbuf, recvbuf, len_elements), __LINE__);
  }

  // Host buffers (ibcomm/allreduce_cpu_impl.h:23-244, 246-372): staged through the device, same sums in
  // the same order as the reference's CPU path.
  template <typename T>
  void AllreduceRing(const T* sendbuf, T* recvbuf, size_t len_elements) {
    Check(ibcomm_hip_allreduce_ring_host(comm_, DType<T>(), sendbuf, recvbuf, len_elements), __LINE__);
  }
  template <typename T>
  void AllreduceRabenseifner(const T* sendbuf, T* recvbuf, size_t len_elements) {
    Check(ibcomm_hip_allreduce_rabenseifner_host(comm_, DType<T>(), sendbuf, recvbuf, len_elements), __LINE__);
  }

  // ibverbs_communicator.h:116-118, ibverbs_communicator_cuda.cpp:26-37.  The reference's Init calls it
  // to build the staging pool and the working GPU buffer; here the communicator's constructor has
  // already built the pool (ibcomm_hip_comm_create), so a caller that names it finds nothing left to do.
  void PrepareMemoryPool() {}

  // ibverbs_communicator.cpp:157-216; the trace is recorded when IBCOMM_HIP_TRACE=1.
  void SetTimerBase() { ibcomm_hip_comm_set_timer_base(comm_); }
  void DumpTrace() const { ibcomm_hip_comm_dump_trace(comm_); }

  ibcomm_hip_comm* handle() { return comm_; }

 private:
  struct World {
    ibcomm_hip_fabric* fabric = nullptr;
    int users = 0;
  };
  struct Registry {
    std::mutex mu;
    std::map<int, World> worlds;
  };
  static Registry& registry() {
    static Registry r;
    return r;
  }

  template <typename T>
  static constexpr int DType() {
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value ||
                      (std::is_integral<T>::value && (sizeof(T) == 4 || sizeof(T) == 8)),
                  "allreduce element type must be float, double or a 32/64-bit integer");
    return std::is_same<T, float>::value ? IBCOMM_HIP_F32
           : std::is_same<T, double>::value ? IBCOMM_HIP_F64
           : sizeof(T) == 4 ? IBCOMM_HIP_I32
                            : IBCOMM_HIP_I64;
  }

  // The communicator a point-to-point call naming `peer` runs on: this one, or, when this object's
  // queue pair for `peer` is wired to another queue pair of the same object, the private
  // communicator that plays the rank at the other end of that wire.
  ibcomm_hip_comm* Endpoint(int peer) {
    if (my_rank_ >= 0 || peer < 0 || peer >= world_size_ || wired_to_[peer] < 0) return comm_;
    if (loop_comms_.empty()) {
      Check(ibcomm_hip_fabric_create(world_size_, &loop_fabric_), __LINE__);
      for (int r = 0; r < world_size_; r++) {
        ibcomm_hip_comm* c = nullptr;
        Check(ibcomm_hip_comm_create(loop_fabric_, world_size_, &c), __LINE__);
        loop_comms_.push_back(c);
        Check(ibcomm_hip_comm_register_myself(c, r), __LINE__);
      }
    }
    return loop_comms_[wired_to_[peer]];
  }

  static void Check(int rc, int line) {
    if (rc == 0) return;
    util::IbcommError(__FILE__, line, static_cast<util::IBCOMM_ERROR_CODE>(rc), "%s", ibcomm_hip_last_error());
  }

  ibcomm_hip_comm* comm_ = nullptr;
  int my_rank_ = -1;
  int world_size_ = 0;
  uint16_t id_ = 0;                          // names this communicator in the ProcessInfo it hands out
  std::vector<int> wired_to_;                // per queue pair: the queue pair of this object it is connected to, or -1
  ibcomm_hip_fabric* loop_fabric_ = nullptr; // private world for self-wired queue pairs
  std::vector<ibcomm_hip_comm*> loop_comms_;
};
