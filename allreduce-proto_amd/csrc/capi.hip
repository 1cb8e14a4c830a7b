// extern "C" surface of libibcomm_hip.so; declarations and reference citations are in
// include/ibcomm_hip.h.
#include "ibcomm_hip.h"

#include <new>
#include <vector>

#include "backend_hip.hpp"
#include "engine.hpp"
#include "world.hpp"

using namespace ibcomm_hip;

static_assert(sizeof(ibcomm_hip_stats) == sizeof(EngineStats), "ibcomm_hip_stats must mirror EngineStats");
static_assert(IBCOMM_HIP_F32 == kF32 && IBCOMM_HIP_I32 == kI32 && IBCOMM_HIP_F64 == kF64 && IBCOMM_HIP_I64 == kI64,
              "dtype codes");
static_assert(IBCOMM_HIP_RING == kRing && IBCOMM_HIP_RABENSEIFNER == kRabenseifner, "algorithm codes");

struct ibcomm_hip_fabric {
  explicit ibcomm_hip_fabric(int n) : fabric(n) {}
  Fabric<HipBackend> fabric;
  int live_comms = 0;
};

struct ibcomm_hip_comm {
  ibcomm_hip_comm(ibcomm_hip_fabric* f, int n) : owner(f), comm(&f->fabric, n) {}
  ibcomm_hip_fabric* owner;
  Communicator<HipBackend> comm;
};

struct ibcomm_hip_plan {
  Plan plan;
};

extern "C" {

const char* ibcomm_hip_last_error(void) { return LastErrorBuffer(); }

int ibcomm_hip_fabric_create(int world_size, ibcomm_hip_fabric** out) {
  if (!out) return Fail(kInvalidArgument, "out is null");
  if (world_size < 1 || world_size > 4096) return Fail(kInvalidArgument, "world_size %d out of range", world_size);
  *out = new (std::nothrow) ibcomm_hip_fabric(world_size);
  return *out ? kOk : Fail(kInvalidArgument, "out of host memory");
}

int ibcomm_hip_fabric_destroy(ibcomm_hip_fabric* fabric) {
  if (!fabric) return kOk;
  if (fabric->live_comms) return Fail(kInvalidArgument, "%d communicators still use this fabric", fabric->live_comms);
  delete fabric;
  return kOk;
}

int ibcomm_hip_comm_create(ibcomm_hip_fabric* fabric, int world_size, ibcomm_hip_comm** out) {
  if (!fabric || !out) return Fail(kInvalidArgument, "fabric or out is null");
  ibcomm_hip_comm* c = new (std::nothrow) ibcomm_hip_comm(fabric, world_size);
  if (!c) return Fail(kInvalidArgument, "out of host memory");
  const int rc = c->comm.Init();
  if (rc != kOk) {
    delete c;
    return rc;
  }
  fabric->live_comms++;
  *out = c;
  return kOk;
}

int ibcomm_hip_comm_destroy(ibcomm_hip_comm* comm) {
  if (!comm) return kOk;
  comm->comm.Abort();
  comm->owner->live_comms--;
  delete comm;
  return kOk;
}

int ibcomm_hip_comm_register_myself(ibcomm_hip_comm* comm, int my_rank) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (my_rank < 0 || my_rank >= comm->comm.world_size())
    return Fail(kInvalidArgument, "rank %d outside world of %d", my_rank, comm->comm.world_size());
  comm->comm.RegisterMyself(my_rank);
  return kOk;
}

int ibcomm_hip_allreduce_ring(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.AllreduceBlocking(kRing, dtype, sendbuf, recvbuf, len);
}

int ibcomm_hip_allreduce_rabenseifner(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf, size_t len) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  return comm->comm.AllreduceBlocking(kRabenseifner, dtype, sendbuf, recvbuf, len);
}

int ibcomm_hip_allreduce_ring_f32(ibcomm_hip_comm* c, const float* s, float* r, size_t n) {
  return ibcomm_hip_allreduce_ring(c, kF32, s, r, n);
}
int ibcomm_hip_allreduce_ring_i32(ibcomm_hip_comm* c, const int32_t* s, int32_t* r, size_t n) {
  return ibcomm_hip_allreduce_ring(c, kI32, s, r, n);
}
int ibcomm_hip_allreduce_rabenseifner_f32(ibcomm_hip_comm* c, const float* s, float* r, size_t n) {
  return ibcomm_hip_allreduce_rabenseifner(c, kF32, s, r, n);
}
int ibcomm_hip_allreduce_rabenseifner_i32(ibcomm_hip_comm* c, const int32_t* s, int32_t* r, size_t n) {
  return ibcomm_hip_allreduce_rabenseifner(c, kI32, s, r, n);
}

int ibcomm_hip_world_allreduce(ibcomm_hip_comm* const* comms, int world_size, int algo, int dtype,
                               const void* const* sendbufs, void* const* recvbufs, size_t len) {
  if (!comms || !sendbufs || !recvbufs || world_size < 1) return Fail(kInvalidArgument, "null argument");
  std::vector<Communicator<HipBackend>*> cs(world_size);
  for (int r = 0; r < world_size; r++) {
    if (!comms[r]) return Fail(kInvalidArgument, "comms[%d] is null", r);
    if (comms[r]->owner != comms[0]->owner) return Fail(kInvalidArgument, "communicators belong to different fabrics");
    cs[r] = &comms[r]->comm;
  }
  return RunWorld<HipBackend>(cs.data(), world_size, algo, dtype, sendbufs, recvbufs, len, true);
}

int ibcomm_hip_reduce(int dtype, void* dst, const void* a, const void* b, size_t n, void* stream) {
  if (DTypeSize(dtype) == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (n && (!dst || !a || !b)) return Fail(kInvalidArgument, "null operand");
  IBCOMM_HIP_CHECK(LaunchReduce2(dst, a, b, n, dtype, static_cast<hipStream_t>(stream)));
  return kOk;
}

int ibcomm_hip_max_segments(void) { return kMaxSegments; }

int ibcomm_hip_reduce_segments(int dtype, int n_segments, void* const* dst, const void* const* a, const void* const* b,
                               const size_t* len, void* stream) {
  if (DTypeSize(dtype) == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);
  if (n_segments < 0 || n_segments > kMaxSegments) return Fail(kInvalidArgument, "at most %d segments per launch", kMaxSegments);
  SegmentBatch batch;
  batch.count = n_segments;
  for (int i = 0; i < n_segments; i++) {
    if (len[i] && (!dst[i] || !a[i] || !b[i])) return Fail(kInvalidArgument, "null operand in segment %d", i);
    batch.seg[i] = Segment{dst[i], nullptr, a[i], b[i], len[i]};
  }
  IBCOMM_HIP_CHECK(LaunchSegments(batch, dtype, DefaultTuning(), static_cast<hipStream_t>(stream)));
  return kOk;
}

int ibcomm_hip_split_buffer(size_t len, size_t sizeof_element, int world_size, const char* env_chunksize, size_t* starts,
                            size_t* ends, int cap, int* n_ranges) {
  if (!n_ranges || sizeof_element == 0 || world_size < 1) return Fail(kInvalidArgument, "bad argument");
  std::vector<Range> ranges;
  *n_ranges = 0;
  IBCOMM_RETURN_IF_ERROR(SplitBuffer(len, sizeof_element, world_size, env_chunksize, &ranges));
  *n_ranges = static_cast<int>(ranges.size());
  for (int i = 0; i < *n_ranges && i < cap; i++) {
    starts[i] = ranges[i].begin;
    ends[i] = ranges[i].end;
  }
  return kOk;
}

int ibcomm_hip_rank_to_chunk(int n_ranges, int world_size, int* first_chunk, int* n_chunks) {
  if (n_ranges < 0 || world_size < 1 || !first_chunk || !n_chunks) return Fail(kInvalidArgument, "bad argument");
  std::vector<int> first, count;
  GetRankToChunk(static_cast<size_t>(n_ranges), world_size, &first, &count);
  for (int r = 0; r < world_size; r++) {
    first_chunk[r] = first[r];
    n_chunks[r] = count[r];
  }
  return kOk;
}

int ibcomm_hip_get_exp_of_two(int n) { return GetExpOfTwo(n); }

int ibcomm_hip_plan_create(int algo, int world_size, int rank, size_t len, size_t sizeof_element, const char* env_chunksize,
                           ibcomm_hip_plan** out) {
  if (!out || sizeof_element == 0) return Fail(kInvalidArgument, "bad argument");
  ibcomm_hip_plan* p = new (std::nothrow) ibcomm_hip_plan();
  if (!p) return Fail(kInvalidArgument, "out of host memory");
  const int rc = BuildPlan(algo, world_size, rank, len, sizeof_element, env_chunksize, &p->plan);
  if (rc != kOk) {
    delete p;
    return rc;
  }
  *out = p;
  return kOk;
}

void ibcomm_hip_plan_destroy(ibcomm_hip_plan* plan) { delete plan; }

int ibcomm_hip_plan_counts(const ibcomm_hip_plan* plan, int* n_chunks, int* n_recvs, int* n_sends) {
  if (!plan) return Fail(kInvalidArgument, "plan is null");
  if (n_chunks) *n_chunks = static_cast<int>(plan->plan.part.ranges.size());
  if (n_recvs) *n_recvs = static_cast<int>(plan->plan.recvs.size());
  if (n_sends) *n_sends = static_cast<int>(plan->plan.sends.size());
  return kOk;
}

int ibcomm_hip_plan_range(const ibcomm_hip_plan* plan, int chunk, size_t* begin, size_t* end) {
  if (!plan || chunk < 0 || chunk >= static_cast<int>(plan->plan.part.ranges.size())) return Fail(kInvalidArgument, "bad chunk");
  *begin = plan->plan.part.ranges[chunk].begin;
  *end = plan->plan.part.ranges[chunk].end;
  return kOk;
}

int ibcomm_hip_plan_recv(const ibcomm_hip_plan* plan, int k, int* chunk, int* peer, int* kind) {
  if (!plan || k < 0 || k >= static_cast<int>(plan->plan.recvs.size())) return Fail(kInvalidArgument, "bad index");
  *chunk = plan->plan.recvs[k].chunk;
  *peer = plan->plan.recvs[k].peer;
  *kind = plan->plan.recvs[k].kind;
  return kOk;
}

int ibcomm_hip_plan_send(const ibcomm_hip_plan* plan, int k, int* chunk, int* peer, int* dep) {
  if (!plan || k < 0 || k >= static_cast<int>(plan->plan.sends.size())) return Fail(kInvalidArgument, "bad index");
  *chunk = plan->plan.sends[k].chunk;
  *peer = plan->plan.sends[k].peer;
  *dep = plan->plan.sends[k].dep;
  return kOk;
}

int ibcomm_hip_comm_set_max_fuse(ibcomm_hip_comm* comm, int f) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (f < 1 || f > kMaxSegments) return Fail(kInvalidArgument, "max fuse must be in [1, %d]", kMaxSegments);
  comm->comm.set_max_fuse(f);
  return kOk;
}

int ibcomm_hip_comm_set_landing(ibcomm_hip_comm* comm, int mode) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  if (mode < kLandMemcpy || mode > kLandDirect) return Fail(kInvalidArgument, "landing mode must be 0, 1 or 2");
  comm->comm.set_landing(mode);
  return kOk;
}

int ibcomm_hip_comm_stats(ibcomm_hip_comm* comm, ibcomm_hip_stats* out) {
  if (!comm || !out) return Fail(kInvalidArgument, "null argument");
  const EngineStats s = comm->comm.stats();
  memcpy(out, &s, sizeof s);
  return kOk;
}

int ibcomm_hip_comm_reset_stats(ibcomm_hip_comm* comm) {
  if (!comm) return Fail(kInvalidArgument, "comm is null");
  comm->comm.reset_stats();
  return kOk;
}

}  // extern "C"
