/*
 * C ABI of the MI355X allreduce hot path (libibcomm_hip.so).
 *
 * This is the boundary a binding of PFNProto's IBVerbsCommunicator would call
 * for the device allreduce path.  The reference exposes that path as C++
 * member templates instantiated in the caller's translation unit
 * (ibcomm/ibverbs_communicator.h:101-115, bodies in
 * ibcomm/allreduce_cuda_impl.h); there is no exported symbol per element type.
 * Each entry point below names the reference interface it stands for.
 *
 * Conventions
 *   - Plain pointers and sizes only.  Buffers passed to the allreduce and
 *     reduce calls are DEVICE pointers on the current HIP device.  The
 *     allreduce calls work on streams of their own that do not synchronise
 *     with the caller's (the reference creates its streams with
 *     cudaStreamNonBlocking, ibcomm/memory_pool.h:96): whatever produces
 *     sendbuf, and any earlier use of recvbuf's memory, must have completed
 *     before the call, as the calls themselves complete before they return.
 *   - Every function returns 0 on success or one of the reference's exit codes
 *     (ibcomm/util.h:32-42): 1 invalid argument, 2 transport error, 3 HIP
 *     error, 4 not supported.  Where the reference prints a message and calls
 *     exit(code) (util.h:44-52) this library returns the code and keeps the
 *     message for ibcomm_hip_last_error(); the C++ facade
 *     (allreduce-proto_amd/ibcomm/ibverbs_communicator.h) prints and exits.
 *   - The network is an in-process loopback: all ranks of a world live in one
 *     process on one GPU and exchange chunks through device memory.
 *   - Environment knobs keep the reference's names: IBCOMM_CHUNKSIZE (read on
 *     every allreduce), IBCOMM_NUM_CUDA_STREAM, IBCOMM_MEMORY_POOL_PRE_ALLOC,
 *     IBCOMM_WORK_GPU_MEMORY_SIZE (read when a communicator is created).
 */
#ifndef IBCOMM_HIP_H_
#define IBCOMM_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ibcomm_hip_fabric ibcomm_hip_fabric; /* the loopback "network" of one world */
typedef struct ibcomm_hip_comm ibcomm_hip_comm;     /* one rank's IBVerbsCommunicator */
typedef struct ibcomm_hip_plan ibcomm_hip_plan;     /* read-only view of one rank's message plan */

/* ibcomm/util.h:32-42 */
enum {
  IBCOMM_HIP_OK = 0,
  IBCOMM_HIP_INVALID_ARGUMENT = 1,
  IBCOMM_HIP_TRANSPORT_ERROR = 2, /* IBVERBS_ERROR */
  IBCOMM_HIP_DEVICE_ERROR = 3,    /* CUDA_ERROR */
  IBCOMM_HIP_NOT_SUPPORTED = 4
};

/* element types the templates are instantiated with: float (examples/allreduce.cpp:103-111),
 * int (ibcomm/allreduce_tester.cpp:416); double and 64-bit integers come for free */
enum { IBCOMM_HIP_F32 = 0, IBCOMM_HIP_I32 = 1, IBCOMM_HIP_F64 = 2, IBCOMM_HIP_I64 = 3 };

enum { IBCOMM_HIP_RING = 0, IBCOMM_HIP_RABENSEIFNER = 1 };

/* Message of the last failure on the calling thread (what util::IbcommError would have printed). */
const char* ibcomm_hip_last_error(void);

/* ---- bring-up ----------------------------------------------------------------------------- */

/* Stands for the queue-pair wiring the reference does with CreateQueuePair / RegisterQueuePair
 * and an out-of-band MPI_Alltoall (examples/allreduce.cpp:50-77): creates the channels between
 * world_size emulated ranks. */
int ibcomm_hip_fabric_create(int world_size, ibcomm_hip_fabric** out);
int ibcomm_hip_fabric_destroy(ibcomm_hip_fabric* fabric);

/* IBVerbsCommunicator::IBVerbsCommunicator(int world_size) + Init + PrepareMemoryPool
 * (ibcomm/ibverbs_communicator.cpp:24-99, ibcomm/ibverbs_communicator_cuda.cpp:26-37):
 * allocates the HBM staging pool and reads the pool knobs. */
int ibcomm_hip_comm_create(ibcomm_hip_fabric* fabric, int world_size, ibcomm_hip_comm** out);
/* IBVerbsCommunicator::~IBVerbsCommunicator (ibcomm/ibverbs_communicator.cpp:101-155) */
int ibcomm_hip_comm_destroy(ibcomm_hip_comm* comm);
/* IBVerbsCommunicator::RegisterMyself (ibcomm/ibverbs_communicator.cpp:355-357) */
int ibcomm_hip_comm_register_myself(ibcomm_hip_comm* comm, int my_rank);

/* ---- the hot path ------------------------------------------------------------------------- */

/* IBVerbsCommunicator::AllreduceRingCuda<T>(const T* sendbuf, T* recvbuf, size_t len_elements)
 * (ibcomm/allreduce_cuda_impl.h:35-301).  Blocking; every rank of the world must be inside the
 * same call on a thread of its own, as every process is in the reference.  On return recvbuf
 * holds, for each element, the left fold of the ranks' values starting at the rank that owns the
 * element's chunk group. */
int ibcomm_hip_allreduce_ring(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf,
                              size_t len_elements);
/* IBVerbsCommunicator::AllreduceRabenseifnerCuda<T> (ibcomm/allreduce_cuda_impl.h:326-717).
 * Power-of-two worlds only (returns 4 otherwise); the result is the balanced pairwise tree over
 * rank index. */
int ibcomm_hip_allreduce_rabenseifner(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf,
                                      size_t len_elements);

/* IBVerbsCommunicator::AllreduceRing<T> and AllreduceRabenseifner<T> on HOST buffers
 * (ibcomm/allreduce_cpu_impl.h:23-244, 246-372).  The reference computes these on the CPU; here
 * the data is copied to the device, reduced by the device path above and copied back.  The sums and
 * their order are the same (ring: left fold from the owner of the chunk group under
 * SplitBuffer; Rabenseifner: balanced tree, which does not depend on how the buffer is cut), so the
 * results are bit-identical to the reference's.  Two differences, both from the reference's CPU
 * Rabenseifner cutting the buffer into world_size ranges of ceilDiv(len, world_size) elements instead
 * of going through SplitBuffer (allreduce_cpu_impl.h:264-271): it accepts len_elements < world_size,
 * which returns 4 here; and when (world_size - 1) * ceilDiv(len, world_size) > len (5 elements on 4
 * ranks) one of its ranges is inverted and its size_t lengths wrap, whereas every
 * len_elements >= world_size works here. */
int ibcomm_hip_allreduce_ring_host(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf,
                                   size_t len_elements);
int ibcomm_hip_allreduce_rabenseifner_host(ibcomm_hip_comm* comm, int dtype, const void* sendbuf, void* recvbuf,
                                           size_t len_elements);

/* Typed spellings of the two device-buffer calls, one per template instantiation the reference's own
 * programs use. */
int ibcomm_hip_allreduce_ring_f32(ibcomm_hip_comm* comm, const float* sendbuf, float* recvbuf, size_t len_elements);
int ibcomm_hip_allreduce_ring_i32(ibcomm_hip_comm* comm, const int32_t* sendbuf, int32_t* recvbuf, size_t len_elements);
int ibcomm_hip_allreduce_rabenseifner_f32(ibcomm_hip_comm* comm, const float* sendbuf, float* recvbuf,
                                          size_t len_elements);
int ibcomm_hip_allreduce_rabenseifner_i32(ibcomm_hip_comm* comm, const int32_t* sendbuf, int32_t* recvbuf,
                                          size_t len_elements);

/* The same collectives for a whole loopback world driven from ONE host thread: comms[r],
 * sendbufs[r], recvbufs[r] belong to rank r, r = 0 .. world_size-1.  Equivalent to world_size
 * concurrent calls of the per-rank functions (which is how mpiexec runs the reference,
 * tests/allreduce_test.py:91), without needing the threads. */
int ibcomm_hip_world_allreduce(ibcomm_hip_comm* const* comms, int world_size, int algo, int dtype,
                               const void* const* sendbufs, void* const* recvbufs, size_t len_elements);

/* ibcomm_hip_world_allreduce for callers that cannot allocate device memory or create streams and
 * events at the time of the call: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  Same arguments without the
 * communicators, same results bit for bit, and `stream` (a hipStream_t, NULL = default stream): all
 * device work of all world_size ranks is enqueued on that one stream and the call returns without
 * waiting for it.  Staging slots come out of a 64 MiB array that is part of the library's code
 * object (one copy per GPU, held until the process ends): a call whose ranks could need more, i.e.
 * world_size * 2 * (chunks per buffer) * (chunk bytes + 16, rounded up to 256) > 64 MiB, returns 1 with a
 * message and enqueues nothing.  Calls on one GPU share the array: they must not overlap in time
 * (enqueue them on one stream, or synchronise in between).  The first call on a device looks up the
 * array's address and should be made outside a capture. */
int ibcomm_hip_world_allreduce_noalloc(int world_size, int algo, int dtype, const void* const* sendbufs,
                                       void* const* recvbufs, size_t len_elements, void* stream);

/* One rank's share on its own.  ibcomm_hip_world_record runs the whole world once (like
 * ibcomm_hip_world_allreduce) while keeping, in device memory, every message `rank` receives and the
 * point of its own schedule at which each became available.  ibcomm_hip_replay_allreduce then runs
 * that rank's complete schedule alone: the peers are ghosts whose messages come from the recording,
 * paced as in the recorded run, and whose receives cost nothing.  Same result in recvbuf as the
 * world run gives that rank (for the same sendbuf contents).  This is how one GPU's part of
 * AllreduceRingCuda / AllreduceRabenseifnerCuda (ibcomm/allreduce_cuda_impl.h:35-301, 326-717) is
 * timed without the other ranks' work on the same device; the reference has no counterpart.
 * Like ibcomm_hip_world_allreduce these two drive a fabric from one host thread: calls on one fabric
 * must not overlap in time (the recording, the graph cache and the completion word belong to the
 * fabric). */
int ibcomm_hip_world_record(ibcomm_hip_comm* const* comms, int world_size, int rank, int algo, int dtype,
                            const void* const* sendbufs, void* const* recvbufs, size_t len_elements);
int ibcomm_hip_replay_allreduce(ibcomm_hip_comm* comm, int algo, int dtype, const void* sendbuf, void* recvbuf,
                                size_t len_elements);

/* ibcomm_hip_world_allreduce records the device work of a call shape (same buffers, length, chunk
 * size and knobs) into a HIP graph on its second use and replays the graph from then on; mode 0
 * turns that off (every call is issued eagerly), mode 1 is the default (IBCOMM_HIP_GRAPH).  No
 * counterpart in the reference, whose host loop re-issues every operation on every call. */
int ibcomm_hip_fabric_set_graph_mode(ibcomm_hip_fabric* fabric, int mode);
int ibcomm_hip_fabric_graph_counters(ibcomm_hip_fabric* fabric, uint64_t* eager_calls, uint64_t* captures,
                                     uint64_t* replays);

/* While a whole world is recorded, the launches the ranks issue for one step of the algorithm --
 * independent of one another, what N devices would run side by side -- are merged into one launch
 * as far as their memory accesses allow, so that a replay pays one kernel boundary per step instead
 * of one per rank and step (8 ranks, ring: 14 launches instead of 112).  Results are unchanged bit
 * for bit.  mode 0 turns that off, mode 1 is the default (IBCOMM_HIP_MERGE_RANKS); the counters say
 * how many launches the ranks handed in during recordings and how many were recorded.  No
 * counterpart in the reference, where every rank is a process with a device of its own. */
int ibcomm_hip_fabric_set_merge_mode(ibcomm_hip_fabric* fabric, int mode);
int ibcomm_hip_fabric_merge_counters(ibcomm_hip_fabric* fabric, uint64_t* launches_collected, uint64_t* launches_recorded);

/* The reduction kernel on its own, asynchronous on `stream` (a hipStream_t, NULL = default
 * stream): dst[i] = a[i] + b[i].  Stands for _reduce_inplace_cuda<T>
 * (ibcomm/allreduce_cuda_impl.h:26-33, launches at :132-133 and :510-512), which is the case
 * dst == a. */
int ibcomm_hip_reduce(int dtype, void* dst, const void* a, const void* b, size_t len_elements, void* stream);
/* Several independent segments in one launch (at most ibcomm_hip_max_segments()). */
int ibcomm_hip_reduce_segments(int dtype, int n_segments, void* const* dst, const void* const* a,
                               const void* const* b, const size_t* len_elements, void* stream);
int ibcomm_hip_max_segments(void);
/* The copy launch of the engine on its own: dst[i] = src[i] over several segments, asynchronous on
 * `stream`.  Stands for the per-chunk cudaMemcpyAsync calls around the reference's kernel
 * (ibcomm/allreduce_cuda_impl.h:129-130 and :528-529 into recvbuf, :503-504 into the working buffer). */
int ibcomm_hip_copy_segments(int dtype, int n_segments, void* const* dst, const void* const* src,
                             const size_t* len_elements, void* stream);
/* How ibcomm_hip_reduce_segments would issue these segments, without launching: *aligned = 1 for the
 * kernel that takes 16-byte aligned pointers (dst: 128-byte aligned) and whole vectors (0: the general kernel), *threads the
 * workgroup size, *die_local = 1 if tiles are ordered in runs per accelerator die, *write_through = 1
 * if the stores carry the agent-scope bit sc1 (0: the non-temporal hint).  Stands for the launch geometry
 * the reference fixes at ibcomm/allreduce_cuda_impl.h:24, 116-117. */
int ibcomm_hip_describe_launch(int dtype, int n_segments, void* const* dst, const void* const* a, const void* const* b,
                               const size_t* len_elements, int* aligned, int* threads, int* die_local, int* write_through);

/* ---- point-to-point messaging over the loopback ------------------------------------------------ */

/* IBVerbsCommunicator::Send / Recv (ibcomm/ibverbs_communicator.cpp:371-384, 486-499), SendPoll /
 * RecvPoll (:416-461, 529-572), SendWait / RecvWait (:463-473, 574-584) and Bcast (:586-606).
 * Buffers may be host or device memory; len is in bytes.  One non-blocking send and one non-blocking
 * receive per peer may be outstanding: posting another before the matching Wait returns 4 with the
 * reference's message.  *completed is 1 once per finished operation, else 0; polls never block.
 * The receiving side moves the data when it polls or waits.  Each rank calls from its own thread. */
int ibcomm_hip_send(ibcomm_hip_comm* comm, int dest_rank, const void* buf, size_t len, int blocking);
int ibcomm_hip_recv(ibcomm_hip_comm* comm, int src_rank, void* buf, size_t len, int blocking);
int ibcomm_hip_send_poll(ibcomm_hip_comm* comm, int dest_rank, int* completed);
int ibcomm_hip_recv_poll(ibcomm_hip_comm* comm, int src_rank, int* completed);
int ibcomm_hip_send_wait(ibcomm_hip_comm* comm, int dest_rank);
int ibcomm_hip_recv_wait(ibcomm_hip_comm* comm, int src_rank);
int ibcomm_hip_bcast(ibcomm_hip_comm* comm, void* buf, size_t len, int root);

/* ---- partitioning and plans (host only, no device needed) ---------------------------------- */

/* IBVerbsCommunicator::SplitBuffer (ibcomm/ibverbs_communicator.cpp:637-683).  env_chunksize is
 * the text IBCOMM_CHUNKSIZE would hold, NULL for "unset".  Writes up to cap ranges
 * [starts[i], ends[i]) and the total count to *n_ranges. */
int ibcomm_hip_split_buffer(size_t len_elements, size_t sizeof_element, int world_size, const char* env_chunksize,
                            size_t* starts, size_t* ends, int cap, int* n_ranges);
/* IBVerbsCommunicator::GetRankToChunk (ibcomm/ibverbs_communicator.cpp:685-707): rank r owns
 * chunks first_chunk[r] .. first_chunk[r] + n_chunks[r] - 1. */
int ibcomm_hip_rank_to_chunk(int n_ranges, int world_size, int* first_chunk, int* n_chunks);
/* util::GetExpOfTwo (ibcomm/util.h:156-175) */
int ibcomm_hip_get_exp_of_two(int n);

/* The ordered messages one rank consumes and emits: the content of the reference's reg_q /
 * first_send_q (ibcomm/allreduce_cuda_impl.h:61-89) and recv_q / send_q / first_send_q
 * (:387-466).  kind: 0 = add to sendbuf's chunk, 1 = add to the running sum, 2 = store. */
int ibcomm_hip_plan_create(int algo, int world_size, int rank, size_t len_elements, size_t sizeof_element,
                           const char* env_chunksize, ibcomm_hip_plan** out);
void ibcomm_hip_plan_destroy(ibcomm_hip_plan* plan);
int ibcomm_hip_plan_counts(const ibcomm_hip_plan* plan, int* n_chunks, int* n_recvs, int* n_sends);
int ibcomm_hip_plan_range(const ibcomm_hip_plan* plan, int chunk, size_t* begin, size_t* end);
int ibcomm_hip_plan_recv(const ibcomm_hip_plan* plan, int k, int* chunk, int* peer, int* kind);
int ibcomm_hip_plan_send(const ibcomm_hip_plan* plan, int k, int* chunk, int* peer, int* dep);

/* ---- knobs and counters --------------------------------------------------------------------- */

/* Chunks reduced per kernel launch at most (1 = one launch per chunk, like the reference).  At its
 * ceiling and default, ibcomm_hip_max_segments(), a launch takes every chunk that is ready, however
 * many, as long as they merge into that many kernel segments. */
int ibcomm_hip_comm_set_max_fuse(ibcomm_hip_comm* comm, int max_chunks_per_launch);
/* How a message reaches the reduction: 0 = hipMemcpyAsync into a pool slot, 1 = one copy-kernel
 * launch for all messages of a pass, 2 = the reduction reads the sender's buffer directly, 3 = as 2,
 * and a partial sum that is only forwarded is produced into a pool slot (send staging) instead of
 * recvbuf, where the next rank's reduction reads it (the default).  IBCOMM_HIP_LANDING = memcpy |
 * kernel | direct | staged sets the initial mode. */
int ibcomm_hip_comm_set_landing(ibcomm_hip_comm* comm, int mode);

/* Host-side pipeline trace in the reference's seven categories and .dat format
 * (IBVerbsCommunicator::SetTimerBase / DumpTrace, ibcomm/ibverbs_communicator.cpp:157-216; TRACE()
 * call sites in ibcomm/allreduce_cuda_impl.h).  The reference compiles it in with -DUSE_TRACE and
 * dumps in the destructor; here it is switched on with IBCOMM_HIP_TRACE=1 or set_trace, dumped by
 * dump_trace and by comm_destroy, to ${IBCOMM_TRACE_FILE:-ibcomm_trace}_<rank>.dat.  Graph replays
 * do no host-side pipeline work and therefore add no events. */
int ibcomm_hip_comm_set_trace(ibcomm_hip_comm* comm, int enabled);
int ibcomm_hip_comm_set_timer_base(ibcomm_hip_comm* comm);
int ibcomm_hip_comm_dump_trace(ibcomm_hip_comm* comm);

typedef struct {
  uint64_t calls;
  uint64_t reduce_launches;
  uint64_t reduce_segments;        /* chunks reduced */
  uint64_t reduce_elements;
  uint64_t landing_copies;
  uint64_t landing_bytes;
  uint64_t gather_copies;
  uint64_t gather_bytes;
  uint64_t messages_sent;
  uint64_t messages_received;
  uint64_t events_recorded;
  uint64_t stream_waits;
  uint64_t streams_created;
  uint64_t slots_high_water;
  uint64_t slot_count;
  uint64_t pool_blocks;
  uint64_t pool_bytes;
  uint64_t progress_passes;
  uint64_t reduce_kernel_segments; /* kernel segments of the reduction launches: chunks that follow one
                                      another in all three operands are merged into one segment */
  uint64_t largest_reduce_elements;        /* the reduction launch with the most elements: its elements */
  uint64_t largest_reduce_kernel_segments; /* ... and its kernel segments */
  uint64_t largest_reduce_launches;        /* how many reduction launches had that many elements */
} ibcomm_hip_stats;

int ibcomm_hip_comm_stats(ibcomm_hip_comm* comm, ibcomm_hip_stats* out);
int ibcomm_hip_comm_reset_stats(ibcomm_hip_comm* comm);

#ifdef __cplusplus
}
#endif
#endif /* IBCOMM_HIP_H_ */
