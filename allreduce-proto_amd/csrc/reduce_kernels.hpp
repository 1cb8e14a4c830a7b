// Streaming reduction / copy kernels for gfx950 (MI355X, CDNA4, wave64).
//
// These replace the reference's only kernel, _reduce_inplace_cuda
// (ibcomm/allreduce_cuda_impl.h:24-33: result[i] += value[i], scalar 4-byte
// accesses, one launch per chunk) with an out-of-place, multi-segment form:
//
//     dst[i] = a[i] + b[i]            (and optionally dst2[i] = the same value)
//     dst[i] = a[i]                   (b == nullptr: landing / staging copy)
//
// One launch takes up to kMaxSegments independent segments, so every chunk
// that has landed can be reduced by a single launch, and a chunk whose two
// operands live in different buffers (pool slot + sendbuf) needs no staging
// copy.  The work is pure HBM streaming: 12 bytes per fp32 element for the
// two-source add (16 with the second store), 8 for a copy; there is nothing
// for MFMA or LDS to do.  Each lane moves 16-byte vectors (global_load_dwordx4
// / global_store_dwordx4), kUnroll of them per operand in flight, and a
// segment whose three pointers share their 16-byte phase is peeled at head and
// tail so the body stays vectorised even when a chunk starts at an odd element.
//
// Two kernels share that contract.  AlignedSegmentKernel takes the launches in which every pointer
// is on a 16-byte boundary and every length a whole number of vectors (in practice all of the
// engine's, since chunk sizes and buffers are aligned): load, add, store, nothing else, because
// with one vector per lane a workgroup lives for one memory round trip and every instruction ahead
// of its loads delays them; for launches of moderate size it also orders its tiles so that each
// of the 8 dies works on runs of consecutive tiles.  SegmentKernel takes everything else (odd offsets, ragged tails, a
// second destination, the tuning experiments).
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

struct LaunchTuning {
  int threads;        // workgroup size: 256 or 1024
  int unroll;         // 16-byte vectors per lane per operand in flight: 1, 2 or 4
  int max_blocks_x;   // cap on workgroups per segment (grid-stride beyond it); 0 = no cap
  int nontemporal;    // which accesses stream past the caches: 1 = loads of a, 2 = loads of b, 4 = stores
};

LaunchTuning DefaultTuning();

// Enqueue one launch covering batch.seg[0..count).  Empty segments are legal; all segments of a
// launch must be of one kind (every b set: add, every b null: copy).
// Returns the HIP error of the launch.
hipError_t LaunchSegments(const SegmentBatch& batch, int dtype, const LaunchTuning& tuning, hipStream_t stream);

// Convenience for a single segment.
hipError_t LaunchReduce2(void* dst, const void* a, const void* b, size_t n, int dtype, hipStream_t stream);
hipError_t LaunchCopy(void* dst, const void* a, size_t n, int dtype, hipStream_t stream);

}  // namespace ibcomm_hip
