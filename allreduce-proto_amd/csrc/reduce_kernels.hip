// gfx950 streaming add / copy kernels.  See reduce_kernels.hpp for the contract.
#include "reduce_kernels.hpp"

#include <stdlib.h>

namespace ibcomm_hip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));

template <bool NT, typename V>
__device__ __forceinline__ V LoadVec(const V* p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}

template <bool NT, typename V>
__device__ __forceinline__ void StoreVec(V* p, V v) {
  if (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// One workgroup column (blockIdx.y) per segment; blockIdx.x strides over tiles
// of THREADS * UNROLL 16-byte vectors.  T is the element type, V the 16-byte
// vector of T.  Integer types are instantiated unsigned so that += wraps.
// ADD selects dst = a + b; otherwise the launch is a copy, dst = a.  The two are
// separate kernels so that a profile tells reductions from landing copies.
// NT is a mask of which accesses carry the non-temporal hint: 1 = loads of a,
// 2 = loads of b, 4 = stores.
template <typename T, typename V, int THREADS, int UNROLL, int NT, bool ADD>
__global__ __launch_bounds__(THREADS) void SegmentKernel(const SegmentBatch batch) {
  const Segment s = batch.seg[blockIdx.y];
  const uint64_t n = s.n;
  if (n == 0) return;

  T* dst = static_cast<T*>(s.dst);
  T* dst2 = static_cast<T*>(s.dst2);
  const T* a = static_cast<const T*>(s.a);
  const T* b = static_cast<const T*>(s.b);
  constexpr bool has_b = ADD;
  const bool has_d2 = (dst2 != nullptr);

  constexpr uint64_t kPerVec = 16 / sizeof(T);
  const uintptr_t pd = reinterpret_cast<uintptr_t>(dst) & 15;
  const bool same_phase = ((reinterpret_cast<uintptr_t>(a) & 15) == pd) &&
                          (!has_b || (reinterpret_cast<uintptr_t>(b) & 15) == pd) &&
                          (!has_d2 || (reinterpret_cast<uintptr_t>(dst2) & 15) == pd) &&
                          (pd % sizeof(T) == 0);

  // [0, head) scalar, [head, head + nvec * kPerVec) as 16-byte vectors, rest scalar.
  uint64_t head = n, nvec = 0;
  if (same_phase) {
    head = ((16 - pd) & 15) / sizeof(T);
    if (head > n) head = n;
    nvec = (n - head) / kPerVec;
  }

  if (nvec) {
    const V* av = reinterpret_cast<const V*>(a + head);
    const V* bv = reinterpret_cast<const V*>(b + head);
    V* dv = reinterpret_cast<V*>(dst + head);
    V* d2v = reinterpret_cast<V*>(dst2 + head);
    constexpr uint64_t kTile = static_cast<uint64_t>(THREADS) * UNROLL;
    for (uint64_t base = static_cast<uint64_t>(blockIdx.x) * kTile; base < nvec;
         base += static_cast<uint64_t>(gridDim.x) * kTile) {
      V ra[UNROLL];
      V rb[UNROLL];
      if (base + kTile <= nvec) {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) ra[u] = LoadVec<(NT & 1) != 0>(av + base + u * THREADS + threadIdx.x);
        if (has_b) {
#pragma unroll
          for (int u = 0; u < UNROLL; u++) rb[u] = LoadVec<(NT & 2) != 0>(bv + base + u * THREADS + threadIdx.x);
#pragma unroll
          for (int u = 0; u < UNROLL; u++) ra[u] = ra[u] + rb[u];
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) StoreVec<(NT & 4) != 0>(dv + base + u * THREADS + threadIdx.x, ra[u]);
        if (has_d2) {
#pragma unroll
          for (int u = 0; u < UNROLL; u++) StoreVec<(NT & 4) != 0>(d2v + base + u * THREADS + threadIdx.x, ra[u]);
        }
      } else {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
          const uint64_t i = base + u * THREADS + threadIdx.x;
          if (i < nvec) {
            V v = LoadVec<(NT & 1) != 0>(av + i);
            if (has_b) v = v + LoadVec<(NT & 2) != 0>(bv + i);
            StoreVec<(NT & 4) != 0>(dv + i, v);
            if (has_d2) StoreVec<(NT & 4) != 0>(d2v + i, v);
          }
        }
      }
    }
  }

  // Scalar remainder: fewer than two vectors' worth when the phases agree,
  // the whole segment when they do not.
  const uint64_t tail_begin = head + nvec * kPerVec;
  const uint64_t scalar_count = head + (n - tail_begin);
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * THREADS;
  for (uint64_t k = static_cast<uint64_t>(blockIdx.x) * THREADS + threadIdx.x; k < scalar_count; k += stride) {
    const uint64_t i = (k < head) ? k : tail_begin + (k - head);
    T v = a[i];
    if (has_b) v = v + b[i];
    dst[i] = v;
    if (has_d2) dst2[i] = v;
  }
}

// The common case on its own: every pointer of every segment on a 16-byte boundary, every length a
// whole number of vectors, one destination, one vector per lane.  Without the peeling logic a
// workgroup issues its loads a few hundred nanoseconds earlier, which a launch of a few tens of
// megabytes feels (8192 short-lived workgroups over 256 CUs start in several rounds).
//
// XCD: workgroups are dealt to the 8 accelerator dies round-robin by their linear id, so with the
// plain mapping each die walks every eighth 4 KiB tile.  With XCD set, every aligned group of 64
// workgroup ids is permuted so that a die gets 8 consecutive tiles (32 KiB of each operand) of
// the group: a few percent faster for launches up to some tens of megabytes per operand, slower
// beyond, so the host sets it by launch size.
template <typename T, typename V, int THREADS, int NT, bool ADD, bool XCD>
__global__ __launch_bounds__(THREADS) void AlignedSegmentKernel(const SegmentBatch batch) {
  const Segment s = batch.seg[blockIdx.y];
  const uint64_t nvec = s.n / (16 / sizeof(T));
  uint64_t tile = blockIdx.x;
  if (XCD && tile < (gridDim.x & ~63u)) tile = (tile & ~63ull) + (tile % 8) * 8 + (tile / 8) % 8;
  const uint64_t i = tile * THREADS + threadIdx.x;
  if (i >= nvec) return;
  V v = LoadVec<(NT & 1) != 0>(static_cast<const V*>(s.a) + i);
  if (ADD) v = v + LoadVec<(NT & 2) != 0>(static_cast<const V*>(s.b) + i);
  StoreVec<(NT & 4) != 0>(static_cast<V*>(s.dst) + i, v);
}

namespace {

int EnvInt(const char* name, int fallback) {
  const char* v = getenv(name);
  return v ? atoi(v) : fallback;
}

// How the aligned kernel is launched, chosen by the size of the largest segment.
struct AlignedShape {
  int threads;     // 256 or 128
  bool die_local;  // the XCD tile order
};

template <typename T, typename V, int NT, int THREADS, bool XCD>
hipError_t LaunchAlignedOne(const SegmentBatch& batch, uint64_t max_nvec, hipStream_t stream) {
  const uint64_t blocks = (max_nvec + THREADS - 1) / THREADS;
  if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
  const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(batch.count));
  if (batch.seg[0].b != nullptr)
    hipLaunchKernelGGL((AlignedSegmentKernel<T, V, THREADS, NT, true, XCD>), grid, dim3(THREADS), 0, stream, batch);
  else
    hipLaunchKernelGGL((AlignedSegmentKernel<T, V, THREADS, NT, false, XCD>), grid, dim3(THREADS), 0, stream, batch);
  return hipGetLastError();
}

template <typename T, typename V, int NT>
hipError_t LaunchAlignedShape(const SegmentBatch& batch, uint64_t max_nvec, AlignedShape shape, hipStream_t stream) {
  if (shape.threads == 256)
    return shape.die_local ? LaunchAlignedOne<T, V, NT, 256, true>(batch, max_nvec, stream)
                           : LaunchAlignedOne<T, V, NT, 256, false>(batch, max_nvec, stream);
  return shape.die_local ? LaunchAlignedOne<T, V, NT, 128, true>(batch, max_nvec, stream)
                         : LaunchAlignedOne<T, V, NT, 128, false>(batch, max_nvec, stream);
}

template <typename T, typename V>
hipError_t LaunchAligned(const SegmentBatch& batch, uint64_t max_nvec, int nt, AlignedShape shape, hipStream_t stream) {
  switch (nt & 7) {
    case 0: return LaunchAlignedShape<T, V, 0>(batch, max_nvec, shape, stream);
    case 1: return LaunchAlignedShape<T, V, 1>(batch, max_nvec, shape, stream);
    case 2: return LaunchAlignedShape<T, V, 2>(batch, max_nvec, shape, stream);
    case 3: return LaunchAlignedShape<T, V, 3>(batch, max_nvec, shape, stream);
    case 4: return LaunchAlignedShape<T, V, 4>(batch, max_nvec, shape, stream);
    case 5: return LaunchAlignedShape<T, V, 5>(batch, max_nvec, shape, stream);
    case 6: return LaunchAlignedShape<T, V, 6>(batch, max_nvec, shape, stream);
    default: return LaunchAlignedShape<T, V, 7>(batch, max_nvec, shape, stream);
  }
}

template <typename T, typename V, int THREADS, int UNROLL, int NT>
hipError_t LaunchOne(const SegmentBatch& batch, dim3 grid, hipStream_t stream) {
  if (batch.seg[0].b != nullptr)
    hipLaunchKernelGGL((SegmentKernel<T, V, THREADS, UNROLL, NT, true>), grid, dim3(THREADS), 0, stream, batch);
  else
    hipLaunchKernelGGL((SegmentKernel<T, V, THREADS, UNROLL, NT, false>), grid, dim3(THREADS), 0, stream, batch);
  return hipGetLastError();
}

template <typename T, typename V, int THREADS, int UNROLL>
hipError_t LaunchNT(const SegmentBatch& batch, dim3 grid, int nt, hipStream_t stream) {
  switch (nt & 7) {
    case 0: return LaunchOne<T, V, THREADS, UNROLL, 0>(batch, grid, stream);
    case 1: return LaunchOne<T, V, THREADS, UNROLL, 1>(batch, grid, stream);
    case 2: return LaunchOne<T, V, THREADS, UNROLL, 2>(batch, grid, stream);
    case 3: return LaunchOne<T, V, THREADS, UNROLL, 3>(batch, grid, stream);
    case 4: return LaunchOne<T, V, THREADS, UNROLL, 4>(batch, grid, stream);
    case 5: return LaunchOne<T, V, THREADS, UNROLL, 5>(batch, grid, stream);
    case 6: return LaunchOne<T, V, THREADS, UNROLL, 6>(batch, grid, stream);
    default: return LaunchOne<T, V, THREADS, UNROLL, 7>(batch, grid, stream);
  }
}

template <typename T, typename V, int THREADS>
hipError_t LaunchUnroll(const SegmentBatch& batch, dim3 grid, int unroll, int nt, hipStream_t stream) {
  switch (unroll) {
    case 1: return LaunchNT<T, V, THREADS, 1>(batch, grid, nt, stream);
    case 2: return LaunchNT<T, V, THREADS, 2>(batch, grid, nt, stream);
    case 4: return LaunchNT<T, V, THREADS, 4>(batch, grid, nt, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename T, typename V>
hipError_t LaunchThreads(const SegmentBatch& batch, dim3 grid, const LaunchTuning& t, hipStream_t stream) {
  switch (t.threads) {
    case 256: return LaunchUnroll<T, V, 256>(batch, grid, t.unroll, t.nontemporal, stream);
    case 1024: return LaunchUnroll<T, V, 1024>(batch, grid, t.unroll, t.nontemporal, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

LaunchTuning DefaultTuning() {
  // Tunables for experiments; the defaults are what the sweep on MI355X picked.
  static const LaunchTuning t = {
      EnvInt("IBCOMM_HIP_THREADS", 256),
      EnvInt("IBCOMM_HIP_UNROLL", 1),
      EnvInt("IBCOMM_HIP_MAX_BLOCKS", 0),
      EnvInt("IBCOMM_HIP_NONTEMPORAL", 7),
  };
  return t;
}

hipError_t LaunchSegments(const SegmentBatch& given, int dtype, const LaunchTuning& tuning, hipStream_t stream) {
  if (given.count <= 0) return hipSuccess;
  if (given.count > kMaxSegments) return hipErrorInvalidValue;
  const size_t es = DTypeSize(dtype);
  if (es == 0) return hipErrorInvalidValue;

  // Empty segments are dropped here (their pointers may be anything); the kernels see the rest.
  SegmentBatch batch;
  batch.count = 0;
  uint64_t max_n = 0;
  const uint64_t per_vec = 16 / es;
  uintptr_t misfit = 0;  // any low pointer bit, any length remainder, any second destination
  for (int i = 0; i < given.count; i++) {
    const Segment& s = given.seg[i];
    if (s.n == 0) continue;
    if (!s.dst || !s.a) return hipErrorInvalidValue;
    if (batch.count && (s.b != nullptr) != (batch.seg[0].b != nullptr)) return hipErrorInvalidValue;  // all adds or all copies
    if (s.n > max_n) max_n = s.n;
    misfit |= ((reinterpret_cast<uintptr_t>(s.dst) | reinterpret_cast<uintptr_t>(s.a) | reinterpret_cast<uintptr_t>(s.b)) & 15) |
              (s.n % per_vec) | reinterpret_cast<uintptr_t>(s.dst2);
    batch.seg[batch.count++] = s;
  }
  if (max_n == 0) return hipSuccess;

  static const bool fast_path_off = EnvInt("IBCOMM_HIP_NO_ALIGNED_KERNEL", 0) != 0;
  if (misfit == 0 && tuning.threads == 256 && tuning.unroll == 1 && tuning.max_blocks_x == 0 && !fast_path_off) {
    // Measured on MI355X with fp32 (µs per launch of one segment, 256 threads plain / 256 die-local /
    // 128 die-local / 128 plain): 1 Mi elements 3.40 / 3.42 / 3.68 / 3.74; 2 Mi 5.5 / 5.5 / 5.5 / 6.4;
    // 4 Mi 9.87 / 9.44 / 9.21 / 10.6; 8 Mi 17.5 / 17.1 / 16.8 / 18.5; 16 Mi 32.7 / 32.3 / 31.7 / 32.4;
    // 32 Mi 63.3 / 63.3 / 61.0 / 63.1; 64 Mi 125 / 129 / 122.2 / 122.1; 128 Mi 250 / 265 / 248 / 244.
    // Hence: 256 threads up to 2 Mi elements, 128 beyond; die-local tile order up to 32 Mi elements.
    // Both limits are in 256-vector tiles (1 Ki fp32) of the largest segment.
    static const uint64_t wg128_min_tiles = static_cast<uint64_t>(EnvInt("IBCOMM_HIP_WG128_MIN_BLOCKS", 2049));
    static const uint64_t xcd_max_tiles = static_cast<uint64_t>(EnvInt("IBCOMM_HIP_XCD_RUN_MAX_BLOCKS", 32768));
    const uint64_t max_nvec = max_n / per_vec;
    const uint64_t tiles = (max_nvec + 255) / 256;
    const AlignedShape shape = {tiles >= wg128_min_tiles ? 128 : 256, tiles >= 64 && tiles <= xcd_max_tiles};
    switch (dtype) {
      case kF32: return LaunchAligned<float, f32x4>(batch, max_nvec, tuning.nontemporal, shape, stream);
      case kI32: return LaunchAligned<uint32_t, u32x4>(batch, max_nvec, tuning.nontemporal, shape, stream);
      case kF64: return LaunchAligned<double, f64x2>(batch, max_nvec, tuning.nontemporal, shape, stream);
      case kI64: return LaunchAligned<uint64_t, u64x2>(batch, max_nvec, tuning.nontemporal, shape, stream);
      default: return hipErrorInvalidValue;
    }
  }

  const uint64_t tile = static_cast<uint64_t>(tuning.threads) * tuning.unroll;
  uint64_t blocks = (max_n / per_vec + tile - 1) / tile;
  if (blocks == 0) blocks = 1;
  if (tuning.max_blocks_x > 0 && blocks > static_cast<uint64_t>(tuning.max_blocks_x)) blocks = tuning.max_blocks_x;
  if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
  const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(batch.count));

  switch (dtype) {
    case kF32: return LaunchThreads<float, f32x4>(batch, grid, tuning, stream);
    case kI32: return LaunchThreads<uint32_t, u32x4>(batch, grid, tuning, stream);
    case kF64: return LaunchThreads<double, f64x2>(batch, grid, tuning, stream);
    case kI64: return LaunchThreads<uint64_t, u64x2>(batch, grid, tuning, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t LaunchReduce2(void* dst, const void* a, const void* b, size_t n, int dtype, hipStream_t stream) {
  SegmentBatch batch;
  batch.count = 1;
  batch.seg[0] = Segment{dst, nullptr, a, b, n};
  return LaunchSegments(batch, dtype, DefaultTuning(), stream);
}

hipError_t LaunchCopy(void* dst, const void* a, size_t n, int dtype, hipStream_t stream) {
  SegmentBatch batch;
  batch.count = 1;
  batch.seg[0] = Segment{dst, nullptr, a, nullptr, n};
  return LaunchSegments(batch, dtype, DefaultTuning(), stream);
}

}  // namespace ibcomm_hip
