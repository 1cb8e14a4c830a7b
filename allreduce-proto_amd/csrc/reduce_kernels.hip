// gfx950 streaming add / copy kernels.  See reduce_kernels.hpp for the contract.
#include "reduce_kernels.hpp"

#include <hip/hip_ext.h>

namespace ibcomm_hip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));

// Cache policy of the streaming accesses.  Loads carry the non-temporal hint: nothing is read
// twice, so neither the L2 nor the memory-side cache should keep the lines.  Stores of the aligned
// kernel carry the sc1 bit instead.  In the memory model of the gfx940 family sc1 alone marks an
// access as agent (device) scope; system scope is sc0 sc1.  The device has eight L2s, one per die, so
// an agent-scope store cannot stay behind in the L2 of the die that issued it; it has to reach
// the level all dies share, which is where the 256 MB cache in front of HBM sits.  That much is
// the model; what is measured on MI355X, against non-temporal stores: a ring step of 32 MiB per
// operand whose results cycle through a 64 MiB staging region is 7 % faster (15.3 against 16.6 us),
// copies of 32 to 64 MiB are 3 to 4 % faster, sc0 sc1 (system scope) performs like sc1, and once a
// launch writes more than about half of that cache nothing is gained and non-temporal stores are 1
// to 2 % ahead; the host picks by the bytes a launch writes.  The explanation offered for the gain
// (the stores are absorbed by the memory-side cache, which writes back in longer runs than the
// kernel's interleaving of two reads and one write gives the DRAM, and a destination written
// again soon is still there) fits the dependence on the size of the destination but has not been
// confirmed with a counter that separates cache hits from DRAM writes.  The builtin offers no such
// store, hence the one instruction of inline assembly; the compiler still schedules everything
// around it.
template <typename V>
__device__ __forceinline__ void StoreWriteThrough(V* p, V v) {
  static_assert(sizeof(V) == 16, "one 16-byte vector");
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}

// What a multi-segment kernel receives: the segments and, for the aligned kernel, how many leading
// tiles are visited in die-local order.
template <int N>
struct KernelSegments {
  Segment seg[N];
  uint32_t die_local_tiles;
  uint32_t write_through;  // stores carry sc1, the agent-scope bit (see StoreWriteThrough), instead of the non-temporal hint
};

template <int N>
KernelSegments<N> MakeKernelSegments(const SegmentBatch& batch, uint32_t die_local_tiles, uint32_t write_through) {
  KernelSegments<N> k;
  for (int i = 0; i < batch.count && i < N; i++) k.seg[i] = batch.seg[i];
  k.die_local_tiles = die_local_tiles;
  k.write_through = write_through;
  return k;
}

// The die-local tile order (see AlignedTile below): within the first die_local_tiles tiles every
// aligned group of 64 workgroup ids is transposed 8 x 8.
__device__ __forceinline__ uint64_t TileOf(uint32_t block, uint32_t die_local_tiles) {
  uint64_t tile = block;
  if (tile < die_local_tiles) tile = (tile & ~63ull) + (tile % 8) * 8 + (tile / 8) % 8;
  return tile;
}

// Any alignment, any length.  T is the element type, V the 16-byte vector of T.  Integer types
// are instantiated unsigned so that += wraps.  ADD selects dst = a + b; otherwise the launch is a
// copy, dst = a.  A segment is peeled: element by element until dst reaches a 128-byte boundary
// (so that a wave's kilobyte of stores covers whole cache lines: starting at the first 16-byte
// boundary instead leaves every wave a partial line at each end and costs 4 % at 8 Mi fp32),
// 16-byte vectors from there, the rest element by element, with the tile order and the store
// policy of the aligned kernel.  Operands that do not share dst's 16-byte phase are loaded as
// 16-byte vectors all the same, from addresses that are only element-aligned (gfx950 takes those
// in its global memory instructions).  Only pointers that are not even element-aligned send a
// segment through the element loop as a whole.
template <typename T, typename V, int THREADS, bool ADD>
__device__ __forceinline__ void PeeledTile(T* dst, const T* a, const T* b, uint64_t n, uint32_t die_local_tiles, uint32_t write_through) {
  typedef V ElementAlignedV __attribute__((aligned(sizeof(T))));
  constexpr uint64_t kPerVec = 16 / sizeof(T);
  constexpr uintptr_t kHeadAlign = 128;
  const uintptr_t pd = reinterpret_cast<uintptr_t>(dst) & 15;
  const uintptr_t all = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(a) | (ADD ? reinterpret_cast<uintptr_t>(b) : 0);
  const bool same_phase = ((reinterpret_cast<uintptr_t>(a) & 15) == pd) && (!ADD || (reinterpret_cast<uintptr_t>(b) & 15) == pd);

  // [0, head) scalar, [head, head + nvec * kPerVec) as 16-byte vectors, rest scalar.
  uint64_t head = n, nvec = 0;
  if (all % sizeof(T) == 0) {
    head = ((kHeadAlign - (reinterpret_cast<uintptr_t>(dst) & (kHeadAlign - 1))) & (kHeadAlign - 1)) / sizeof(T);
    if (head > n) head = n;
    nvec = (n - head) / kPerVec;
  }

  const uint64_t i = TileOf(blockIdx.x, die_local_tiles) * THREADS + threadIdx.x;
  if (i < nvec) {
    V v;
    if (same_phase) {
      v = __builtin_nontemporal_load(reinterpret_cast<const V*>(a + head) + i);
      if (ADD) v = v + __builtin_nontemporal_load(reinterpret_cast<const V*>(b + head) + i);
    } else {
      v = __builtin_nontemporal_load(reinterpret_cast<const ElementAlignedV*>(a + head) + i);
      if (ADD) v = v + __builtin_nontemporal_load(reinterpret_cast<const ElementAlignedV*>(b + head) + i);
    }
    if (write_through) StoreWriteThrough(reinterpret_cast<V*>(dst + head) + i, v);
    else __builtin_nontemporal_store(v, reinterpret_cast<V*>(dst + head) + i);
  }

  // Scalar remainder: less than 128 + 16 bytes, or the whole segment.
  const uint64_t tail_begin = head + nvec * kPerVec;
  const uint64_t scalar_count = head + (n - tail_begin);
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * THREADS;
  for (uint64_t k = static_cast<uint64_t>(blockIdx.x) * THREADS + threadIdx.x; k < scalar_count; k += stride) {
    const uint64_t e = (k < head) ? k : tail_begin + (k - head);
    T v = a[e];
    if (ADD) v = v + b[e];
    dst[e] = v;
  }
}

// One workgroup column (blockIdx.y) per segment; blockIdx.x is the tile of THREADS 16-byte vectors.
// Adds and copies are separate kernels so that a profile tells reductions from landing copies.
template <typename T, typename V, int THREADS, bool ADD>
__global__ __launch_bounds__(THREADS) void SegmentKernel(const KernelSegments<kMaxSegments> batch) {
  const Segment s = batch.seg[blockIdx.y];
  PeeledTile<T, V, THREADS, ADD>(static_cast<T*>(s.dst), static_cast<const T*>(s.a), static_cast<const T*>(s.b), s.n, batch.die_local_tiles,
                                 batch.write_through);
}

// The same for a launch of one segment, operands as plain kernel arguments (see AlignedOneSegmentKernel).
template <typename T, typename V, int THREADS, bool ADD>
__global__ __launch_bounds__(THREADS) void OneSegmentKernel(T* dst, const T* a, const T* b, uint64_t n, uint32_t die_local_tiles,
                                                            uint32_t write_through) {
  PeeledTile<T, V, THREADS, ADD>(dst, a, b, n, die_local_tiles, write_through);
}

// The common case on its own: every pointer of every segment on a 16-byte boundary, every length a
// whole number of vectors, one vector per lane.  Without the peeling logic a workgroup issues its
// loads a few hundred nanoseconds earlier, which a launch of a few tens of megabytes feels
// (thousands of short-lived workgroups over 256 CUs start in several rounds).
//
// Workgroups are dealt to the 8 accelerator dies round-robin by their linear id, so with the plain
// mapping each die walks every eighth 4 KiB tile.  Within the first die_local_tiles tiles (a
// multiple of 64) every aligned group of 64 workgroup ids is permuted so that a die gets 8
// consecutive tiles (32 KiB of each operand) of the group: a few percent faster for launches up to
// some tens of megabytes per operand, slower beyond, so the host sets it by launch size (0 = plain).
template <typename V, int THREADS, bool ADD>
__device__ __forceinline__ void AlignedTile(V* dst, const V* a, const V* b, uint64_t nvec, uint32_t die_local_tiles, uint32_t write_through) {
  const uint64_t i = TileOf(blockIdx.x, die_local_tiles) * THREADS + threadIdx.x;
  if (i >= nvec) return;
  V v = __builtin_nontemporal_load(a + i);
  if (ADD) v = v + __builtin_nontemporal_load(b + i);
  if (write_through) StoreWriteThrough(dst + i, v);
  else __builtin_nontemporal_store(v, dst + i);
}

template <typename V, int PER_VEC, int THREADS, bool ADD>
__global__ __launch_bounds__(THREADS) void AlignedSegmentKernel(const KernelSegments<kMaxSegments> batch) {
  const Segment s = batch.seg[blockIdx.y];
  AlignedTile<V, THREADS, ADD>(static_cast<V*>(s.dst), static_cast<const V*>(s.a), static_cast<const V*>(s.b), s.n / PER_VEC,
                               batch.die_local_tiles, batch.write_through);
}

// A launch of one segment (a ring step whose chunks merged into one) takes its operands as plain
// kernel arguments: 36 bytes in one cache line, which the command processor can hand to a wave in
// registers, where the table form costs every workgroup a scalar load from a 2 KiB argument block
// before it can issue its only loads.
template <typename V, int THREADS, bool ADD>
__global__ __launch_bounds__(THREADS) void AlignedOneSegmentKernel(V* dst, const V* a, const V* b, uint64_t nvec, uint32_t die_local_tiles,
                                                                   uint32_t write_through) {
  AlignedTile<V, THREADS, ADD>(dst, a, b, nvec, die_local_tiles, write_through);
}

namespace {

// With `start` / `stop` set the launch goes through the extended call, which makes the two events
// carry the kernel's own begin and end timestamps (what a profiler reports for the dispatch) instead
// of the times at which markers before and after it were processed.
template <typename... Params, typename... Args>
void Launch(void (*kernel)(Params...), dim3 grid, dim3 block, hipStream_t stream, hipEvent_t start, hipEvent_t stop, Args... args) {
  if (start || stop) hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, start, stop, 0, args...);
  else hipLaunchKernelGGL(kernel, grid, block, 0, stream, args...);
}

template <typename V, int PER_VEC, int THREADS>
hipError_t LaunchAlignedOne(const SegmentBatch& batch, uint64_t max_nvec, bool add, const LaunchShape& shape, hipStream_t stream, hipEvent_t e0,
                            hipEvent_t e1) {
  const uint64_t blocks = (max_nvec + THREADS - 1) / THREADS;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(batch.count));
  const uint32_t die_local_tiles = shape.die_local ? static_cast<uint32_t>(blocks & ~63ull) : 0u;
  const uint32_t write_through = shape.write_through ? 1u : 0u;
  // A copy moves bits: the element types of one width share a copy kernel.
  if (batch.count == 1) {
    const Segment& s = batch.seg[0];
    if (add)
      Launch(AlignedOneSegmentKernel<V, THREADS, true>, grid, dim3(THREADS), stream, e0, e1, static_cast<V*>(s.dst), static_cast<const V*>(s.a),
             static_cast<const V*>(s.b), max_nvec, die_local_tiles, write_through);
    else
      Launch(AlignedOneSegmentKernel<u32x4, THREADS, false>, grid, dim3(THREADS), stream, e0, e1, static_cast<u32x4*>(s.dst),
             static_cast<const u32x4*>(s.a), static_cast<const u32x4*>(nullptr), max_nvec, die_local_tiles, write_through);
  } else {
    const KernelSegments<kMaxSegments> args = MakeKernelSegments<kMaxSegments>(batch, die_local_tiles, write_through);
    if (add) Launch(AlignedSegmentKernel<V, PER_VEC, THREADS, true>, grid, dim3(THREADS), stream, e0, e1, args);
    else Launch(AlignedSegmentKernel<u32x4, PER_VEC, THREADS, false>, grid, dim3(THREADS), stream, e0, e1, args);
  }
  return hipGetLastError();
}

template <typename V, int PER_VEC>
hipError_t LaunchAligned(const SegmentBatch& batch, uint64_t max_nvec, bool add, const LaunchShape& shape, hipStream_t stream, hipEvent_t e0,
                         hipEvent_t e1) {
  return shape.threads == 256 ? LaunchAlignedOne<V, PER_VEC, 256>(batch, max_nvec, add, shape, stream, e0, e1)
                              : LaunchAlignedOne<V, PER_VEC, 128>(batch, max_nvec, add, shape, stream, e0, e1);
}

template <typename T, typename V, int THREADS, bool ADD>
hipError_t LaunchPeeledOne(const SegmentBatch& batch, uint64_t max_n, const LaunchShape& shape, hipStream_t stream, hipEvent_t e0, hipEvent_t e1) {
  uint64_t blocks = (max_n / (16 / sizeof(T)) + THREADS - 1) / THREADS;
  if (blocks == 0) blocks = 1;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(batch.count));
  const uint32_t die_local_tiles = shape.die_local ? static_cast<uint32_t>(blocks & ~63ull) : 0u;
  const uint32_t write_through = shape.write_through ? 1u : 0u;
  if (batch.count == 1) {
    const Segment& s = batch.seg[0];
    Launch(OneSegmentKernel<T, V, THREADS, ADD>, grid, dim3(THREADS), stream, e0, e1, static_cast<T*>(s.dst), static_cast<const T*>(s.a),
           static_cast<const T*>(s.b), static_cast<uint64_t>(s.n), die_local_tiles, write_through);
  } else {
    const KernelSegments<kMaxSegments> args = MakeKernelSegments<kMaxSegments>(batch, die_local_tiles, write_through);
    Launch(SegmentKernel<T, V, THREADS, ADD>, grid, dim3(THREADS), stream, e0, e1, args);
  }
  return hipGetLastError();
}

// A copy moves bits: the element types of one width share a copy kernel (CopyT, CopyV).
template <typename T, typename V, typename CopyT, typename CopyV>
hipError_t LaunchPeeled(const SegmentBatch& batch, uint64_t max_n, bool add, const LaunchShape& shape, hipStream_t stream, hipEvent_t e0, hipEvent_t e1) {
  if (shape.threads == 256)
    return add ? LaunchPeeledOne<T, V, 256, true>(batch, max_n, shape, stream, e0, e1)
               : LaunchPeeledOne<CopyT, CopyV, 256, false>(batch, max_n, shape, stream, e0, e1);
  return add ? LaunchPeeledOne<T, V, 128, true>(batch, max_n, shape, stream, e0, e1)
             : LaunchPeeledOne<CopyT, CopyV, 128, false>(batch, max_n, shape, stream, e0, e1);
}

}  // namespace

namespace {

// Drops empty segments (their pointers may be anything), checks the rest and decides how the launch
// is issued.  *max_n is the length of the longest segment; 0 means there is nothing to launch.
hipError_t Prepare(const SegmentBatch& given, int dtype, SegmentBatch* batch, LaunchShape* shape, uint64_t* max_n) {
  *shape = LaunchShape{false, 256, false, false, 0};
  *max_n = 0;
  batch->count = 0;
  if (given.count <= 0) return hipSuccess;
  if (given.count > kMaxSegments) return hipErrorInvalidValue;
  const size_t es = DTypeSize(dtype);
  if (es == 0) return hipErrorInvalidValue;
  const uint64_t per_vec = 16 / es;
  uintptr_t misfit = 0;  // any low pointer bit that matters, any length remainder
  uint64_t written = 0;  // bytes the launch stores
  for (int i = 0; i < given.count; i++) {
    const Segment& s = given.seg[i];
    if (s.n == 0) continue;
    if (!s.dst || !s.a) return hipErrorInvalidValue;
    if (batch->count && (s.b != nullptr) != (batch->seg[0].b != nullptr)) return hipErrorInvalidValue;  // all adds or all copies
    if (s.n > *max_n) *max_n = s.n;
    written += s.n * es;
    // dst off the 128-byte grid counts as a misfit too: the peeled kernel then starts its vectors at
    // the next whole cache line, which is 3 % faster than the aligned kernel straddling lines.
    misfit |= ((reinterpret_cast<uintptr_t>(s.dst) | reinterpret_cast<uintptr_t>(s.a) | reinterpret_cast<uintptr_t>(s.b)) & 15) |
              (reinterpret_cast<uintptr_t>(s.dst) & 127) | (s.n % per_vec);
    batch->seg[batch->count++] = s;
  }
  shape->segments = batch->count;
  if (*max_n == 0) return hipSuccess;
  // Measured on MI355X with fp32, one segment, non-temporal stores (us per launch: 256 threads plain /
  // 256 die-local / 128 die-local / 128 plain): 1 Mi elements 3.40 / 3.42 / 3.68 / 3.74; 2 Mi 5.5 / 5.5 /
  // 5.5 / 6.4; 4 Mi 9.87 / 9.44 / 9.21 / 10.6; 8 Mi 17.5 / 17.1 / 16.8 / 18.5; 16 Mi 32.7 / 32.3 / 31.7 /
  // 32.4; 32 Mi 63.3 / 63.3 / 61.0 / 63.1; 64 Mi 125 / 129 / 122.2 / 122.1; 128 Mi 250 / 265 / 248 / 244.
  // With written-through stores the two workgroup sizes are closer (256 / 128 threads, die-local: 1 Mi
  // 3.36 / 3.38; 2 Mi 4.94 / 4.87; 4 Mi 8.52 / 8.49; 8 Mi 15.37 / 15.18; 12 Mi 22.10 / 21.86), same order.
  // Hence: 256 threads up to 2 Mi elements, 128 beyond; die-local tile order up to 32 Mi elements.
  // Both limits are in 256-vector tiles (4 KiB) of the largest segment.
  constexpr uint64_t kWg128MinTiles = 2049, kDieLocalMaxTiles = 32768;
  const uint64_t tiles = (*max_n / per_vec + 255) / 256;
  shape->aligned = misfit == 0;
  shape->threads = tiles >= kWg128MinTiles ? 128 : 256;
  shape->die_local = tiles >= 64 && tiles <= kDieLocalMaxTiles;
  // Stores go through the memory-side cache while a launch writes at most half of its 256 MB
  // (config 2's ring step writes 32 MiB, config 5's 64 MiB; config 3's first halving step 192 MiB).
  shape->write_through = written <= kWriteThroughMaxBytes;
  return hipSuccess;
}

}  // namespace

hipError_t DescribeLaunch(const SegmentBatch& given, int dtype, LaunchShape* shape) {
  SegmentBatch batch;
  uint64_t max_n = 0;
  return Prepare(given, dtype, &batch, shape, &max_n);
}

hipError_t LaunchSegments(const SegmentBatch& given, int dtype, hipStream_t stream, hipEvent_t start, hipEvent_t stop) {
  SegmentBatch batch;
  LaunchShape shape;
  uint64_t max_n = 0;
  const hipError_t e = Prepare(given, dtype, &batch, &shape, &max_n);
  if (e != hipSuccess || max_n == 0) return e;
  const bool add = batch.seg[0].b != nullptr;
  const uint64_t per_vec = 16 / DTypeSize(dtype);

  if (shape.aligned) {
    const uint64_t max_nvec = max_n / per_vec;
    switch (dtype) {
      case kF32: return LaunchAligned<f32x4, 4>(batch, max_nvec, add, shape, stream, start, stop);
      case kI32: return LaunchAligned<u32x4, 4>(batch, max_nvec, add, shape, stream, start, stop);
      case kF64: return LaunchAligned<f64x2, 2>(batch, max_nvec, add, shape, stream, start, stop);
      case kI64: return LaunchAligned<u64x2, 2>(batch, max_nvec, add, shape, stream, start, stop);
      default: return hipErrorInvalidValue;
    }
  }

  switch (dtype) {
    case kF32: return LaunchPeeled<float, f32x4, uint32_t, u32x4>(batch, max_n, add, shape, stream, start, stop);
    case kI32: return LaunchPeeled<uint32_t, u32x4, uint32_t, u32x4>(batch, max_n, add, shape, stream, start, stop);
    case kF64: return LaunchPeeled<double, f64x2, uint64_t, u64x2>(batch, max_n, add, shape, stream, start, stop);
    case kI64: return LaunchPeeled<uint64_t, u64x2, uint64_t, u64x2>(batch, max_n, add, shape, stream, start, stop);
    default: return hipErrorInvalidValue;
  }
}

hipError_t LaunchReduce2(void* dst, const void* a, const void* b, size_t n, int dtype, hipStream_t stream) {
  SegmentBatch batch;
  batch.count = 1;
  batch.seg[0] = Segment{dst, a, b, n};
  return LaunchSegments(batch, dtype, stream);
}

hipError_t LaunchCopy(void* dst, const void* a, size_t n, int dtype, hipStream_t stream) {
  SegmentBatch batch;
  batch.count = 1;
  batch.seg[0] = Segment{dst, a, nullptr, n};
  return LaunchSegments(batch, dtype, stream);
}

}  // namespace ibcomm_hip
