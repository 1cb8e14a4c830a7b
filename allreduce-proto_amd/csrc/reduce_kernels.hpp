// Streaming reduction / copy kernels for gfx950 (MI355X, CDNA4, wave64).
//
// These replace the reference's only kernel, _reduce_inplace_cuda
// (ibcomm/allreduce_cuda_impl.h:24-33: result[i] += value[i], scalar 4-byte
// accesses, one launch per chunk) with an out-of-place, multi-segment form:
//
//     dst[i] = a[i] + b[i]
//     dst[i] = a[i]                   (b == nullptr: landing / staging copy)
//
// One launch takes up to kMaxSegments independent segments, so every chunk
// that has landed can be reduced by a single launch, and a chunk whose two
// operands live in different buffers (pool slot + sendbuf) needs no staging
// copy.  The work is pure HBM streaming: 12 bytes per fp32 element for the
// two-source add, 8 for a copy; there is nothing for MFMA or LDS to do.  Each
// lane moves one 16-byte vector per operand (global_load_dwordx4 /
// global_store_dwordx4), loads with the non-temporal hint, stores with the
// agent-scope bit (sc1) while a launch writes little enough for the cache in
// front of HBM to take it, non-temporal beyond.
//
// Two kernels share that contract.  AlignedSegmentKernel takes the launches in which every pointer
// is on a 16-byte boundary (dst on a 128-byte one) and every length a whole number of vectors (in practice all of the
// engine's, since chunk sizes and buffers are aligned): load, add, store, nothing else, because
// with one vector per lane a workgroup lives for one memory round trip and every instruction ahead
// of its loads delays them; for launches of moderate size it also orders its tiles so that each
// of the 8 dies works on runs of consecutive tiles.  SegmentKernel takes everything else (odd
// offsets, ragged tails): a segment is peeled at head and tail so that the body runs in 16-byte
// vectors on dst's grid, with the same workgroup size, tile order and store policy; operands at
// another 16-byte phase are loaded as vectors from element-aligned addresses.
//
// One workgroup per tile and nothing persistent, on purpose: on MI355X the hardware's own
// in-order workgroup dispatch keeps the addresses in flight in one narrow moving window, and
// grid-stride, software-pipelined and several-vectors-per-lane forms of the same kernel all
// measured slower (6 to 10 % at 256 MiB per operand).
//
// One IEEE-754 add per element, no multiply, so nothing can contract into an
// FMA: results are bit-identical to the host's `float` add, provided fp32
// denormals are kept (they are: the kernels are built without
// -fgpu-flush-denormals-to-zero).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "segments.hpp"

namespace ibcomm_hip {

// A launch's stores carry sc1 while it writes at most this many bytes, the non-temporal hint beyond (half of
// the 256 MB cache in front of HBM; see the kernels' source for the measurements).
constexpr uint64_t kWriteThroughMaxBytes = uint64_t(128) << 20;

// How a launch will be issued, for tests and the benchmark's report.
struct LaunchShape {
  bool aligned;    // AlignedSegmentKernel (true) or SegmentKernel (false)
  int threads;     // workgroup size: 256, or 128 for large segments
  bool die_local;  // tiles ordered so that each die gets runs of 8 consecutive tiles
  bool write_through;  // vector stores carry sc1 (agent scope: past the die's L2, into the memory-side cache) instead of the non-temporal hint
  int segments;    // non-empty segments
};

// Enqueue one launch covering batch.seg[0..count).  Empty segments are legal; all segments of a
// launch must be of one kind (every b set: add, every b null: copy).
// Returns the HIP error of the launch.  `start` and `stop`, when given (events created with timing), receive
// the kernel's own begin and end timestamps; the time between them is the kernel's duration.  A launch
// with nothing to do leaves them untouched.
hipError_t LaunchSegments(const SegmentBatch& batch, int dtype, hipStream_t stream, hipEvent_t start = nullptr, hipEvent_t stop = nullptr);
// How LaunchSegments would issue this batch, without launching anything.
hipError_t DescribeLaunch(const SegmentBatch& batch, int dtype, LaunchShape* shape);

// Convenience for a single segment.
hipError_t LaunchReduce2(void* dst, const void* a, const void* b, size_t n, int dtype, hipStream_t stream);
hipError_t LaunchCopy(void* dst, const void* a, size_t n, int dtype, hipStream_t stream);

}  // namespace ibcomm_hip
