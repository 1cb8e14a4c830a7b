/*
 * CPU oracle for the PFNProto allreduce hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * algorithms (partitioning, the scalar reduction loop, the four allreduce
 * schedules) run over an in-memory FIFO loopback, one host thread per emulated
 * rank.  It exists so that the HIP path can be compared bit-for-bit against
 * the reference's summation order.  Nothing in the shipped library may link,
 * load or call it; only tests, the smoke check and the benchmark's CPU
 * baseline leg do.
 *
 * Pinning status (what fixes each function independently of this file):
 *   orc_ceil_div, orc_get_exp_of_two   reference KATs tests/unittest.cpp:65-71
 *                                      + the reference's own util.h compiled
 *                                      into oracle/_ref (when available)
 *   orc_split_buffer, orc_rank_to_chunk  invariants by brute force + the cases
 *                                      held by tests/allreduce_test.py:102-225
 *   orc_reduce_inplace                 numpy IEEE-754 binary32/64 and wrapping
 *                                      integer add
 *   orc_allreduce (all four schedules) numpy closed forms (ring: left fold from
 *                                      the chunk's owner rank; Rabenseifner:
 *                                      balanced pairwise tree), the tester's
 *                                      integer known answers
 *                                      (tests/allreduce_test.py:66-67), brute
 *                                      force on tiny inputs
 *   orc_closed_form_ring / _tree       equality with orc_allreduce + numpy
 * No function here is "parity unpinned".
 */
#ifndef IBCOMM_ORACLE_H_
#define IBCOMM_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* util.h:32-42 */
enum {
  ORC_OK = 0,
  ORC_INVALID_ARGUMENT = 1,
  ORC_IBVERBS_ERROR = 2,
  ORC_CUDA_ERROR = 3,
  ORC_NOT_SUPPORTED = 4,
  ORC_INTERNAL = 100 /* oracle's own failure: deadlock watchdog, size mismatch */
};

enum { ORC_F32 = 0, ORC_I32 = 1, ORC_F64 = 2, ORC_I64 = 3 };

enum {
  ORC_RING_CPU = 0,        /* AllreduceRing<T>            allreduce_cpu_impl.h:23-244  */
  ORC_RABEN_CPU = 1,       /* AllreduceRabenseifner<T>    allreduce_cpu_impl.h:246-372 */
  ORC_RING_GPU = 2,        /* AllreduceRingCuda<T>        allreduce_cuda_impl.h:35-301 */
  ORC_RABEN_GPU = 3        /* AllreduceRabenseifnerCuda<T> allreduce_cuda_impl.h:326-717 */
};

size_t orc_dtype_size(int dtype);

/* util.h:151-154 */
int64_t orc_ceil_div(int64_t v1, int64_t v2);
/* util.h:156-175 */
int orc_get_exp_of_two(int n);

/* ibverbs_communicator.cpp:619-634.  env == NULL means "variable unset":
 * *out_bytes = -1 and ORC_OK.  Otherwise atoi(env); <= 0 is
 * ORC_INVALID_ARGUMENT. */
int orc_read_chunk_size(const char* env, int* out_bytes);

/* ibverbs_communicator.cpp:637-683.  Writes at most cap ranges; *n_ranges is
 * the number produced.  Returns ORC_OK, ORC_INVALID_ARGUMENT or
 * ORC_NOT_SUPPORTED exactly where the reference calls IbcommError. */
int orc_split_buffer(size_t len_elements, size_t sizeof_element, int world_size,
                     const char* env_chunksize, size_t* starts, size_t* ends,
                     int cap, int* n_ranges);

/* ibverbs_communicator.cpp:685-707.  Groups are contiguous, so a group is
 * described by its first chunk id and its chunk count. */
void orc_rank_to_chunk(int n_ranges, int world_size, int* first_chunk,
                       int* n_chunks);

/* allreduce_cpu_impl.h:16-21 */
void orc_reduce_inplace(int dtype, void* result, const void* value,
                        size_t len_elements);

typedef struct {
  int pool_slots_high_water; /* GPU schedules: max slots simultaneously held by one rank */
  int pool_blocks;           /* GPU schedules: max blocks allocated by one rank */
  int slots_leaked;          /* GPU schedules: slots not returned at exit (must be 0) */
  long messages;             /* total messages delivered over the loopback */
} orc_stats;

/* Run one allreduce of `algo` on `world_size` emulated ranks (one thread
 * each).  sendbufs[r] / recvbufs[r] are rank r's host buffers of len_elements
 * elements.  env_chunksize is the value IBCOMM_CHUNKSIZE would hold (NULL =
 * unset).  pool_block_bytes is IBCOMM_MEMORY_POOL_PRE_ALLOC (0 = the
 * reference default, 64 MiB); only the GPU schedules use it.
 * Returns the reference's exit code for the call (0 on success). */
int orc_allreduce(int algo, int dtype, int world_size,
                  const void* const* sendbufs, void* const* recvbufs,
                  size_t len_elements, const char* env_chunksize,
                  size_t pool_block_bytes, orc_stats* stats);

/* Wire log of the last orc_allreduce call: the k-th message src -> dst as an
 * element range [offset, offset + n) of the allreduce buffer.  Per ordered
 * pair the order is deterministic (FIFO matching). */
long orc_wire_count(int src, int dst);
int orc_wire_get(int src, int dst, long k, size_t* offset_elements,
                 size_t* n_elements);

/* Closed forms of what the schedules compute, element by element.
 * ring: out[e] = ((x_g + x_{g+1}) + ...) + x_{g-1}, g = rank owning e's chunk
 *       under orc_split_buffer / orc_rank_to_chunk (indices mod world_size).
 * tree: out[e] = balanced pairwise tree over rank index (world_size = 2^k). */
int orc_closed_form_ring(int dtype, int world_size, const void* const* sendbufs,
                         void* out, size_t len_elements,
                         const char* env_chunksize);
int orc_closed_form_tree(int dtype, int world_size, const void* const* sendbufs,
                         void* out, size_t len_elements);

/* Single-core streaming rate of the reference's scalar loop, for the CPU
 * baseline: runs result += value over n fp32 elements `reps` times and
 * returns seconds per pass (minimum over reps). */
double orc_time_reduce_f32(size_t n, int reps);

#ifdef __cplusplus
}
#endif
#endif  /* IBCOMM_ORACLE_H_ */
