// The device layer the engine is written against, bound to the HIP runtime.
//
// The engine, the pool and the loopback transport are templates over a
// "backend" that supplies streams, events, device memory, an asynchronous copy
// and the segment kernel.  The shipped library instantiates them with
// HipBackend only; there is no host execution path in it.
#pragma once

#include <hip/hip_runtime.h>

#include "reduce_kernels.hpp"
#include "status.hpp"

namespace ibcomm_hip {

#define IBCOMM_HIP_CHECK(cmd)                                                                  \
  do {                                                                                         \
    hipError_t _e = (cmd);                                                                     \
    if (_e != hipSuccess)                                                                      \
      return ::ibcomm_hip::Fail(::ibcomm_hip::kDeviceError, "%s failed at %s:%d: %s", #cmd, __FILE__, __LINE__, \
                                hipGetErrorString(_e));                                        \
  } while (0)

struct HipBackend {
  using Stream = hipStream_t;
  using Event = hipEvent_t;

  static int Malloc(void** p, size_t bytes) {
    IBCOMM_HIP_CHECK(hipMalloc(p, bytes));
    return kOk;
  }
  static int Free(void* p) {
    IBCOMM_HIP_CHECK(hipFree(p));
    return kOk;
  }
  // Pool streams do not synchronise with the legacy default stream
  // (the reference creates them with cudaStreamNonBlocking, memory_pool.h:96).
  static int StreamCreate(Stream* s) {
    IBCOMM_HIP_CHECK(hipStreamCreateWithFlags(s, hipStreamNonBlocking));
    return kOk;
  }
  static int StreamDestroy(Stream s) {
    IBCOMM_HIP_CHECK(hipStreamDestroy(s));
    return kOk;
  }
  static int StreamSynchronize(Stream s) {
    IBCOMM_HIP_CHECK(hipStreamSynchronize(s));
    return kOk;
  }
  static int EventCreate(Event* e) {
    IBCOMM_HIP_CHECK(hipEventCreateWithFlags(e, hipEventDisableTiming));
    return kOk;
  }
  static int EventDestroy(Event e) {
    IBCOMM_HIP_CHECK(hipEventDestroy(e));
    return kOk;
  }
  static int EventRecord(Event e, Stream s) {
    IBCOMM_HIP_CHECK(hipEventRecord(e, s));
    return kOk;
  }
  static int StreamWaitEvent(Stream s, Event e) {
    IBCOMM_HIP_CHECK(hipStreamWaitEvent(s, e, 0));
    return kOk;
  }
  static int EventSynchronize(Event e) {
    IBCOMM_HIP_CHECK(hipEventSynchronize(e));
    return kOk;
  }
  // Timers: events that keep a device timestamp, for the trace's device durations.
  using Timer = hipEvent_t;
  static constexpr bool kHasTimers = true;
  static int TimerCreate(Timer* t) {
    IBCOMM_HIP_CHECK(hipEventCreate(t));
    return kOk;
  }
  static int TimerDestroy(Timer t) {
    IBCOMM_HIP_CHECK(hipEventDestroy(t));
    return kOk;
  }
  static int TimerRecord(Timer t, Stream s) {
    IBCOMM_HIP_CHECK(hipEventRecord(t, s));
    return kOk;
  }
  static int TimerElapsedMs(Timer from, Timer to, float* ms) {
    IBCOMM_HIP_CHECK(hipEventElapsedTime(ms, from, to));
    return kOk;
  }
  // Blocking copy between any two buffers, host or device (point-to-point Send/Recv).
  static int CopySync(void* dst, const void* src, size_t bytes) {
    IBCOMM_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDefault));
    return kOk;
  }
  static int CopyAsync(void* dst, const void* src, size_t bytes, Stream s) {
    IBCOMM_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s));
    return kOk;
  }
  // `role` says what the launch is for (0 = reduction, 1 = landing copy into a pool slot,
  // 2 = gather into recvbuf); the kernels are the same for all three.  With timers the kernel leaves
  // its own begin and end times in them; a batch without elements launches nothing, and then the
  // timers are recorded on the stream so that they still hold a (zero-length) span.
  static int LaunchSegments(const SegmentBatch& batch, int dtype, Stream s, int /*role*/ = 0, Timer start = nullptr, Timer stop = nullptr) {
    bool empty = true;
    for (int i = 0; i < batch.count; i++) empty = empty && batch.seg[i].n == 0;
    if (empty && start && stop) {
      IBCOMM_HIP_CHECK(hipEventRecord(start, s));
      IBCOMM_HIP_CHECK(hipEventRecord(stop, s));
      return kOk;
    }
    IBCOMM_HIP_CHECK(::ibcomm_hip::LaunchSegments(batch, dtype, s, start, stop));
    return kOk;
  }
};

}  // namespace ibcomm_hip
