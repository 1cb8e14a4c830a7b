// Plain descriptions of the work one segment-kernel launch does; no device runtime needed.
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace ibcomm_hip {

constexpr int kMaxSegments = 64;  // 64 * 32 B of kernel arguments, under the 4 KiB limit

struct Segment {
  void* dst;        // written
  const void* a;    // first operand (always read)
  const void* b;    // second operand (nullptr = copy)
  uint64_t n;       // elements
};

struct SegmentBatch {
  Segment seg[kMaxSegments];
  int count;
};

enum DType : int { kF32 = 0, kI32 = 1, kF64 = 2, kI64 = 3 };

inline size_t DTypeSize(int dtype) {
  switch (dtype) {
    case kF32: case kI32: return 4;
    case kF64: case kI64: return 8;
    default: return 0;
  }
}

}  // namespace ibcomm_hip
