// ibcomm_hip_world_allreduce_noalloc: the whole-world allreduce for callers that cannot allocate.
//
// ibcomm_hip_world_allreduce keeps its staging slots in a pool of hipMalloc blocks and creates
// streams and events as it goes.  Code under HIP graph capture, tight serving loops and harnesses
// that forbid allocation cannot call that.  This variant runs the same engine over a backend whose
// "device memory" is a fixed array that lives in the library's code object, whose only stream is the
// caller's, and whose events are nothing at all: every launch of every emulated rank is enqueued on
// the one stream in the dependency-respecting order the single-threaded driver issues them in, and
// an in-order stream then carries every ordering an event would have carried (and launches of
// different ranks that touch no common memory are merged into one, as in a recorded world).  The
// call makes no hipMalloc, hipFree, stream or event creation, and does not wait for the device.
//
// Every call on a GPU uses that GPU's copy of the array and finds the previous call's staging data
// in it.  Nothing has to start at zero: a staging slot is written in full by the launch that
// produces it before any launch reads it.  Two calls that overlap in time on one GPU (different
// streams, different threads) would hand out the same slots and race; callers serialise them.
#include "ibcomm_hip.h"

#include <memory>
#include <mutex>
#include <vector>

#include "backend_hip.hpp"
#include "engine.hpp"
#include "reduce_kernels.hpp"
#include "world.hpp"

using namespace ibcomm_hip;

namespace {

// Staging memory of the no-allocation entry point: 64 MiB per GPU from the moment the library's
// code object is loaded there until the process ends.
constexpr size_t kScratchBytes = size_t(64) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// `scratch` is a host-side stand-in in host code, not an address a kernel can use.  The device
// address is looked up once per device, with that device current, and kept here.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

int ScratchFor(int device, char** out) {
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (device < 0 || device >= kMaxDevices) return Fail(kInvalidArgument, "device %d outside [0, %d)", device, kMaxDevices);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return Fail(kDeviceError, "hipGetSymbolAddress(scratch) failed on device %d: %s", device, hipGetErrorString(e));
    g_scratch_ptr[device] = p;
  }
  *out = static_cast<char*>(g_scratch_ptr[device]);
  return kOk;
}

// What a call may use: its GPU's scratch array, handed out front to back, and the caller's stream.
struct Arena {
  char* base = nullptr;
  size_t size = 0;
  size_t used = 0;
  hipStream_t stream = nullptr;
};
thread_local Arena* t_arena = nullptr;

// The engine's device layer without allocation: memory comes out of the arena, the stream is the
// caller's, events do nothing (one in-order stream), copies are copy-kernel launches.
struct StaticBackend {
  using Stream = hipStream_t;
  using Event = int;

  static int Malloc(void** p, size_t bytes) {
    Arena* a = t_arena;
    const size_t rounded = (bytes + 255) & ~size_t(255);
    if (!a || rounded > a->size - a->used)
      return Fail(kInvalidArgument, "the no-allocation allreduce ran out of its %zu bytes of built-in staging memory", kScratchBytes);
    *p = a->base + a->used;
    a->used += rounded;
    return kOk;
  }
  static int Free(void*) { return kOk; }
  static int StreamCreate(Stream* s) {
    *s = t_arena ? t_arena->stream : nullptr;
    return kOk;
  }
  static int StreamDestroy(Stream) { return kOk; }
  static int StreamSynchronize(Stream) { return kOk; }  // the caller synchronises its stream
  static int EventCreate(Event* e) {
    *e = 0;
    return kOk;
  }
  static int EventDestroy(Event) { return kOk; }
  static int EventRecord(Event, Stream) { return kOk; }
  static int StreamWaitEvent(Stream, Event) { return kOk; }
  static int EventSynchronize(Event) { return kOk; }
  using Timer = int;
  static constexpr bool kHasTimers = false;
  static int TimerCreate(Timer*) { return kOk; }
  static int TimerDestroy(Timer) { return kOk; }
  static int TimerRecord(Timer, Stream) { return kOk; }
  static int TimerElapsedMs(Timer, Timer, float* ms) {
    *ms = 0;
    return kOk;
  }
  static int CopySync(void*, const void*, size_t) { return Fail(kNotSupported, "no point-to-point messaging on this backend"); }
  static int CopyAsync(void* dst, const void* src, size_t bytes, Stream s) {
    if (bytes % 4) return Fail(kInvalidArgument, "copy of %zu bytes is not a whole number of elements", bytes);
    IBCOMM_HIP_CHECK(LaunchCopy(dst, src, bytes / 4, kI32, s));
    return kOk;
  }
  static int LaunchSegments(const SegmentBatch& batch, int dtype, Stream s, int /*role*/ = 0, Timer = 0, Timer = 0) {
    IBCOMM_HIP_CHECK(::ibcomm_hip::LaunchSegments(batch, dtype, s));
    return kOk;
  }
};

}  // namespace

extern "C" int ibcomm_hip_world_allreduce_noalloc(int world_size, int algo, int dtype, const void* const* sendbufs,
                                                  void* const* recvbufs, size_t len_elements, void* stream) {
  if (!sendbufs || !recvbufs) return Fail(kInvalidArgument, "null argument");
  if (world_size < 1 || world_size > 4096) return Fail(kInvalidArgument, "world_size %d out of range", world_size);
  if (algo != kRing && algo != kRabenseifner) return Fail(kInvalidArgument, "unknown algorithm %d", algo);
  const size_t es = DTypeSize(dtype);
  if (es == 0) return Fail(kInvalidArgument, "unsupported element type %d", dtype);

  // Staging the call can use at most: every rank holding two slots per chunk of the buffer (the
  // sums it has produced for the next rank and those it is producing).  Each rank's pool gets one
  // block of exactly that size out of the array below, before anything is enqueued, and the engine
  // never asks a pool that holds a slot for another block; so a call is either refused here, with
  // the stream untouched, or runs to its end.
  size_t block_bytes = 0;
  if (world_size > 1) {
    std::vector<Range> ranges;
    IBCOMM_RETURN_IF_ERROR(SplitBuffer(len_elements, es, world_size, getenv("IBCOMM_CHUNKSIZE"), &ranges));
    const size_t stride = (ranges[0].size() * es + 16 + 255) & ~size_t(255);
    block_bytes = 2 * ranges.size() * stride;
    if (block_bytes > kScratchBytes / static_cast<size_t>(world_size))
      return Fail(kInvalidArgument,
                  "ibcomm_hip_world_allreduce_noalloc: %d ranks x %zu elements need %zu bytes of staging, the built-in "
                  "scratch holds %zu; use ibcomm_hip_world_allreduce for this size",
                  world_size, len_elements, block_bytes * world_size, kScratchBytes);
  } else {
    block_bytes = 256;
  }

  int device = 0;
  IBCOMM_HIP_CHECK(hipGetDevice(&device));
  Arena arena;
  IBCOMM_RETURN_IF_ERROR(ScratchFor(device, &arena.base));
  arena.size = kScratchBytes;
  arena.stream = static_cast<hipStream_t>(stream);
  t_arena = &arena;

  // Host-side objects only from here on; the ranks' pools take their one block each from the arena.
  int rc = kOk;
  {
    Fabric<StaticBackend> fabric(world_size);
    std::vector<std::unique_ptr<Communicator<StaticBackend>>> comms;
    std::vector<Communicator<StaticBackend>*> cs;
    for (int r = 0; r < world_size && rc == kOk; r++) {
      comms.emplace_back(new Communicator<StaticBackend>(&fabric, world_size));
      rc = comms.back()->Init(block_bytes);
      comms.back()->RegisterMyself(r);
      comms.back()->set_landing(kLandStaged);
      comms.back()->trace().Enable(false);
      cs.push_back(comms.back().get());
    }
    // one in-order stream for all ranks: their launches of one step merge as in a recorded world (merge.hpp)
    LaunchCollector<StaticBackend> collector;
    collector.set_write_limit(kWriteThroughMaxBytes);
    if (rc == kOk) rc = RunWorld<StaticBackend>(cs.data(), world_size, algo, dtype, sendbufs, recvbufs, len_elements, false, &collector);
  }
  t_arena = nullptr;
  return rc;
}
