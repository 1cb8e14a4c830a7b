// MEASUREMENT ONLY: libibcomm_hip_bench.so, loaded by bench.py's --sweep, --ceiling and --overlap
// legs and by nothing else.  The shipped library (libibcomm_hip.so) contains none of this.
//
// Two things live here:
//
//  1. Alternative forms of the streaming kernel dst = a + b (or dst = a) on fp32, one segment, all
//     pointers 16-byte aligned: other workgroup sizes, several vectors per lane, persistent
//     grid-stride loops with and without software pipelining, contiguous spans per workgroup, and
//     every cache-policy bit combination the gfx950 vector memory instructions take.  The sweep
//     times each at the launch shapes the allreduce schedules use, next to the shipped kernel,
//     which is how the shipped geometry was chosen and how far it is from the best any of these
//     forms reaches ("the ceiling") is tracked.
//
//  2. Probes of what it costs to run a schedule of dependent launches in other ways than one
//     in-order chain: parallel chains of kernel nodes in a HIP graph, several streams, launches
//     without the implicit barrier (hipExtAnyOrderLaunch), per-chunk ready counters polled and
//     signalled by the kernels themselves, and the ways a blocking call can wait for its last
//     kernel.  These decided how the engine issues a collective.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <chrono>
#include <functional>
#include <string>
#include <vector>

typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

thread_local char g_error[256] = "";
#define IBV_CHECK(cmd)                                                                                         \
  do {                                                                                                         \
    hipError_t e_ = (cmd);                                                                                     \
    if (e_ != hipSuccess) {                                                                                    \
      snprintf(g_error, sizeof g_error, "%s failed at line %d: %s", #cmd, __LINE__, hipGetErrorString(e_));     \
      return 3;                                                                                                \
    }                                                                                                          \
  } while (0)

// The shipped kernel's die-local tile order: every aligned group of 64 tiles is transposed 8 x 8.
__device__ __forceinline__ uint64_t DieLocal(uint64_t t, uint64_t ntiles) {
  if (t < (ntiles & ~63ull)) return (t & ~63ull) + (t % 8) * 8 + (t / 8) % 8;
  return t;
}

// ---- one workgroup per tile of T * U vectors ------------------------------------------------------
template <int T, int U, bool XCD, bool ADD>
__global__ __launch_bounds__(T) void OneShot(f32x4* __restrict__ d, const f32x4* __restrict__ a, const f32x4* __restrict__ b, uint64_t ntiles) {
  const uint64_t blk = XCD ? DieLocal(blockIdx.x, ntiles) : blockIdx.x;
  const uint64_t base = blk * (uint64_t)(T * U) + threadIdx.x;
  f32x4 x[U];
#pragma unroll
  for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(a + base + u * T);
  if (ADD) {
    f32x4 y[U];
#pragma unroll
    for (int u = 0; u < U; u++) y[u] = __builtin_nontemporal_load(b + base + u * T);
#pragma unroll
    for (int u = 0; u < U; u++) x[u] = x[u] + y[u];
  }
#pragma unroll
  for (int u = 0; u < U; u++) __builtin_nontemporal_store(x[u], d + base + u * T);
}

// ---- persistent grid-stride loop; PIPE issues the next tile's loads before this tile's stores -------
template <int T, int U, bool PIPE, bool ADD>
__global__ __launch_bounds__(T) void Persistent(f32x4* __restrict__ d, const f32x4* __restrict__ a, const f32x4* __restrict__ b, uint64_t ntiles) {
  const uint64_t G = gridDim.x;
  uint64_t tile = blockIdx.x;
  if (tile >= ntiles) return;
  f32x4 x[U], y[U];
  uint64_t base = tile * (uint64_t)(T * U) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(a + base + u * T);
  if (ADD) {
#pragma unroll
    for (int u = 0; u < U; u++) y[u] = __builtin_nontemporal_load(b + base + u * T);
  }
  for (;;) {
    const uint64_t next = tile + G;
    f32x4 r[U];
#pragma unroll
    for (int u = 0; u < U; u++) r[u] = ADD ? x[u] + y[u] : x[u];
    const uint64_t nbase = next * (uint64_t)(T * U) + threadIdx.x;
    if (PIPE && next < ntiles) {
#pragma unroll
      for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(a + nbase + u * T);
      if (ADD) {
#pragma unroll
        for (int u = 0; u < U; u++) y[u] = __builtin_nontemporal_load(b + nbase + u * T);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) __builtin_nontemporal_store(r[u], d + base + u * T);
    if (next >= ntiles) break;
    if (!PIPE) {
#pragma unroll
      for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(a + nbase + u * T);
      if (ADD) {
#pragma unroll
        for (int u = 0; u < U; u++) y[u] = __builtin_nontemporal_load(b + nbase + u * T);
      }
    }
    tile = next;
    base = nbase;
  }
}

// ---- persistent, each workgroup streams through one contiguous span, software pipelined -------------
template <int T, int U, bool ADD>
__global__ __launch_bounds__(T) void Span(f32x4* __restrict__ d, const f32x4* __restrict__ a, const f32x4* __restrict__ b, uint64_t ntiles) {
  const uint64_t G = gridDim.x;
  const uint64_t per = (ntiles + G - 1) / G;
  const uint64_t t0 = blockIdx.x * per;
  uint64_t t1 = t0 + per;
  if (t1 > ntiles) t1 = ntiles;
  if (t0 >= t1) return;
  f32x4 x[U], y[U];
  uint64_t base = t0 * (uint64_t)(T * U) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(a + base + u * T);
  if (ADD) {
#pragma unroll
    for (int u = 0; u < U; u++) y[u] = __builtin_nontemporal_load(b + base + u * T);
  }
  for (uint64_t t = t0;;) {
    f32x4 r[U];
#pragma unroll
    for (int u = 0; u < U; u++) r[u] = ADD ? x[u] + y[u] : x[u];
    const uint64_t nbase = base + (uint64_t)(T * U);
    if (t + 1 < t1) {
#pragma unroll
      for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(a + nbase + u * T);
      if (ADD) {
#pragma unroll
        for (int u = 0; u < U; u++) y[u] = __builtin_nontemporal_load(b + nbase + u * T);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) __builtin_nontemporal_store(r[u], d + base + u * T);
    if (++t >= t1) break;
    base = nbase;
  }
}

// ---- cache-policy bits of the loads and the stores (die-local tile order, one vector per lane) -----
// 0 none, 1 nt, 2 sc1, 3 sc0 sc1, 4 sc1 nt, 5 sc0 sc1 nt, 6 sc0, 7 sc0 nt
#define IBV_LOAD(mods) asm volatile("global_load_dwordx4 %0, %1, off " mods : "=v"(v) : "v"(p) : "memory")
#define IBV_STORE(mods) asm volatile("global_store_dwordx4 %0, %1, off " mods : : "v"(p), "v"(v) : "memory")
template <int H>
__device__ __forceinline__ f32x4 LoadHint(const f32x4* p) {
  f32x4 v;
  if (H == 0) IBV_LOAD("");
  if (H == 1) IBV_LOAD("nt");
  if (H == 2) IBV_LOAD("sc1");
  if (H == 3) IBV_LOAD("sc0 sc1");
  if (H == 4) IBV_LOAD("sc1 nt");
  if (H == 5) IBV_LOAD("sc0 sc1 nt");
  if (H == 6) IBV_LOAD("sc0");
  if (H == 7) IBV_LOAD("sc0 nt");
  return v;
}
template <int H>
__device__ __forceinline__ void StoreHint(f32x4* p, f32x4 v) {
  if (H == 0) IBV_STORE("");
  if (H == 1) IBV_STORE("nt");
  if (H == 2) IBV_STORE("sc1");
  if (H == 3) IBV_STORE("sc0 sc1");
  if (H == 4) IBV_STORE("sc1 nt");
  if (H == 5) IBV_STORE("sc0 sc1 nt");
  if (H == 6) IBV_STORE("sc0");
  if (H == 7) IBV_STORE("sc0 nt");
}
template <int T, int LH, int SH, bool ADD>
__global__ __launch_bounds__(T) void Hinted(f32x4* __restrict__ d, const f32x4* __restrict__ a, const f32x4* __restrict__ b, uint64_t ntiles) {
  const uint64_t i = DieLocal(blockIdx.x, ntiles) * (uint64_t)T + threadIdx.x;
  f32x4 x = LoadHint<LH>(a + i);
  if (ADD) {
    f32x4 y = LoadHint<LH>(b + i);
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(x), "+v"(y));
    x = x + y;
  } else {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(x));
  }
  StoreHint<SH>(d + i, x);
}

struct Variant {
  std::string name;
  int tile_vectors;  // n / 4 must be a multiple of this
  std::function<void(f32x4*, const f32x4*, const f32x4*, uint64_t nvec, hipStream_t)> launch;
};

int CuCount() {
  static int cus = 0;
  if (!cus) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, 0) == hipSuccess) cus = p.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

std::vector<Variant>& Variants() {
  static std::vector<Variant> v;
  if (!v.empty()) return v;
#define ONE(T, U, X)                                                                                                          \
  v.push_back({"one workgroup per tile, " #T " threads x " #U " vectors, " + std::string(X ? "die-local" : "plain") + " tile order", T * U, \
               [](f32x4* d, const f32x4* a, const f32x4* b, uint64_t nvec, hipStream_t s) {                                     \
                 const uint64_t nt = nvec / (T * U);                                                                            \
                 if (b) hipLaunchKernelGGL((OneShot<T, U, X, true>), dim3((unsigned)nt), dim3(T), 0, s, d, a, b, nt);            \
                 else hipLaunchKernelGGL((OneShot<T, U, X, false>), dim3((unsigned)nt), dim3(T), 0, s, d, a, b, nt);             \
               }})
  ONE(256, 1, true); ONE(256, 1, false); ONE(128, 1, true); ONE(128, 1, false); ONE(64, 1, true); ONE(512, 1, true); ONE(1024, 1, true);
  ONE(64, 2, true); ONE(128, 2, true); ONE(256, 2, true); ONE(512, 2, true);
  ONE(64, 4, true); ONE(128, 4, true); ONE(256, 4, true); ONE(256, 4, false); ONE(256, 8, false);
#define PER(T, U, P, K)                                                                                                        \
  v.push_back({"persistent grid-stride, " #T " threads x " #U " vectors, " #K " workgroups per CU, " +                            \
                   std::string(P ? "next loads before stores" : "loads after stores"), T * U,                                    \
               [](f32x4* d, const f32x4* a, const f32x4* b, uint64_t nvec, hipStream_t s) {                                     \
                 const uint64_t nt = nvec / (T * U);                                                                            \
                 const unsigned g = (unsigned)(CuCount() * K);                                                                   \
                 if (b) hipLaunchKernelGGL((Persistent<T, U, P, true>), dim3(g), dim3(T), 0, s, d, a, b, nt);                    \
                 else hipLaunchKernelGGL((Persistent<T, U, P, false>), dim3(g), dim3(T), 0, s, d, a, b, nt);                     \
               }})
  PER(256, 1, true, 8); PER(256, 1, false, 8); PER(256, 1, true, 4); PER(256, 2, true, 8); PER(256, 2, true, 4); PER(256, 2, false, 8);
  PER(256, 4, true, 4); PER(256, 4, true, 2); PER(128, 2, true, 16); PER(128, 4, true, 8); PER(64, 4, true, 16); PER(64, 4, true, 32);
  PER(512, 1, true, 4); PER(512, 2, true, 4); PER(1024, 1, true, 2); PER(1024, 2, true, 2);
#define SPAN(T, U, K)                                                                                                          \
  v.push_back({"persistent contiguous spans, " #T " threads x " #U " vectors, " #K " workgroups per CU", T * U,                  \
               [](f32x4* d, const f32x4* a, const f32x4* b, uint64_t nvec, hipStream_t s) {                                     \
                 const uint64_t nt = nvec / (T * U);                                                                            \
                 const unsigned g = (unsigned)(CuCount() * K);                                                                   \
                 if (b) hipLaunchKernelGGL((Span<T, U, true>), dim3(g), dim3(T), 0, s, d, a, b, nt);                             \
                 else hipLaunchKernelGGL((Span<T, U, false>), dim3(g), dim3(T), 0, s, d, a, b, nt);                              \
               }})
  SPAN(256, 1, 8); SPAN(256, 2, 8); SPAN(256, 4, 4); SPAN(64, 4, 16);
  static const char* hint_names[8] = {"cached", "nt", "sc1", "sc0 sc1", "sc1 nt", "sc0 sc1 nt", "sc0", "sc0 nt"};
#define HINT(T, LH, SH)                                                                                                        \
  v.push_back({std::string("cache policy: loads ") + hint_names[LH] + ", stores " + hint_names[SH] + ", " #T " threads, die-local", T, \
               [](f32x4* d, const f32x4* a, const f32x4* b, uint64_t nvec, hipStream_t s) {                                     \
                 const uint64_t nt = nvec / T;                                                                                  \
                 if (b) hipLaunchKernelGGL((Hinted<T, LH, SH, true>), dim3((unsigned)nt), dim3(T), 0, s, d, a, b, nt);           \
                 else hipLaunchKernelGGL((Hinted<T, LH, SH, false>), dim3((unsigned)nt), dim3(T), 0, s, d, a, b, nt);            \
               }})
  HINT(128, 0, 0); HINT(128, 1, 1); HINT(128, 1, 0); HINT(128, 0, 1); HINT(128, 2, 2); HINT(128, 3, 3); HINT(128, 4, 4); HINT(128, 5, 5);
  HINT(128, 6, 6); HINT(128, 7, 7); HINT(128, 1, 2); HINT(128, 1, 3); HINT(128, 1, 4); HINT(128, 1, 5); HINT(128, 4, 1); HINT(128, 5, 1);
  HINT(128, 2, 1); HINT(128, 3, 1); HINT(256, 1, 1); HINT(256, 4, 4); HINT(256, 1, 2);
  return v;
}

// ---- probes ------------------------------------------------------------------------------------------

// The shipped kernel's geometry (one vector per lane, die-local, 256 threads up to 2 Mi elements, 128 beyond).
void LaunchLikeShipped(f32x4* d, const f32x4* a, const f32x4* b, uint64_t nvec, hipStream_t s, unsigned flags) {
  if (nvec / 256 >= 2049) {
    const uint64_t nt = nvec / 128;
    hipExtLaunchKernelGGL((OneShot<128, 1, true, true>), dim3((unsigned)nt), dim3(128), 0, s, nullptr, nullptr, flags, d, a, b, nt);
  } else {
    const uint64_t nt = nvec / 256;
    hipExtLaunchKernelGGL((OneShot<256, 1, true, true>), dim3((unsigned)nt), dim3(256), 0, s, nullptr, nullptr, flags, d, a, b, nt);
  }
}

// Ready counters: every wave adds 1 to its chunk's counter once its stores are done (SIGNAL); every
// workgroup first waits until the previous step's counter of its chunk has reached `target` (WAIT).
// The wait is bounded: a workgroup that gives up raises *err and goes on, so every wave exits.
template <int T, bool SIGNAL, bool WAIT>
__global__ __launch_bounds__(T) void Flagged(f32x4* __restrict__ d, const f32x4* __restrict__ a, const f32x4* __restrict__ b, uint64_t ntiles,
                                             const uint32_t* prev, uint32_t* mine, uint32_t tiles_per_chunk, uint32_t target, uint32_t* err) {
  const uint64_t blk = DieLocal(blockIdx.x, ntiles);
  const uint32_t chunk = (uint32_t)(blk / tiles_per_chunk);
  const uint64_t i = blk * (uint64_t)T + threadIdx.x;
  f32x4 y = LoadHint<4>(b + i);
  if (WAIT && prev) {
    uint32_t v = __hip_atomic_load(prev + chunk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    int spins = 0;
    while (v < target) {
      if (++spins > (1 << 12) || *(volatile uint32_t*)err) {
        *err = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(4);
      v = __hip_atomic_load(prev + chunk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  f32x4 x = LoadHint<4>(a + i);
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(x), "+v"(y));
  StoreHint<4>(d + i, x + y);
  if (SIGNAL) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(mine + chunk, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

__global__ void SetFlag(volatile uint32_t* flag, uint32_t v) { *flag = v; }
__global__ void Null() {}
__global__ void StoreClock(uint64_t* host_word) {
  __hip_atomic_store(host_word, static_cast<uint64_t>(wall_clock64()), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

struct Region {
  char *a, *b, *d;
  size_t bytes;
};

// microseconds per call of `call`, timed with events on `s` (device pace, calls back to back)
int DevicePace(hipStream_t s, int warm, int iters, const std::function<int(int)>& call, double* us) {
  hipEvent_t e0, e1;
  IBV_CHECK(hipEventCreate(&e0));
  IBV_CHECK(hipEventCreate(&e1));
  for (int i = 0; i < warm; i++)
    if (int rc = call(i)) return rc;
  IBV_CHECK(hipStreamSynchronize(s));
  IBV_CHECK(hipEventRecord(e0, s));
  for (int i = 0; i < iters; i++)
    if (int rc = call(warm + i)) return rc;
  IBV_CHECK(hipEventRecord(e1, s));
  IBV_CHECK(hipEventSynchronize(e1));
  IBV_CHECK(hipGetLastError());
  float ms = 0;
  IBV_CHECK(hipEventElapsedTime(&ms, e0, e1));
  IBV_CHECK(hipEventDestroy(e0));
  IBV_CHECK(hipEventDestroy(e1));
  *us = ms * 1e3 / iters;
  return 0;
}

// microseconds per call of `call` on the host clock; each call is expected to block until its work is done
int WallClock(int warm, int iters, const std::function<int(int)>& call, double* us) {
  for (int i = 0; i < warm; i++)
    if (int rc = call(i)) return rc;
  IBV_CHECK(hipDeviceSynchronize());
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < iters; i++)
    if (int rc = call(warm + i)) return rc;
  IBV_CHECK(hipDeviceSynchronize());
  *us = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() * 1e6 / iters;
  return 0;
}

}  // namespace

extern "C" {

const char* ibv_last_error(void) { return g_error; }

int ibv_variant_count(void) { return static_cast<int>(Variants().size()); }
const char* ibv_variant_name(int v) { return (v >= 0 && v < ibv_variant_count()) ? Variants()[v].name.c_str() : ""; }
// Whether variant v can take n fp32 elements (n / 4 vectors must be whole tiles of the variant).
int ibv_variant_accepts(int v, size_t n) {
  if (v < 0 || v >= ibv_variant_count() || n % 4) return 0;
  return (n / 4) % static_cast<size_t>(Variants()[v].tile_vectors) == 0 && n / 4 / Variants()[v].tile_vectors < 0x7fffffffull;
}
// dst = a + b (b == NULL: dst = a) over n fp32 elements, asynchronous on `stream`.
int ibv_variant_launch(int v, void* dst, const void* a, const void* b, size_t n, void* stream) {
  if (!ibv_variant_accepts(v, n)) {
    snprintf(g_error, sizeof g_error, "variant %d does not take %zu elements", v, n);
    return 1;
  }
  Variants()[v].launch(static_cast<f32x4*>(dst), static_cast<const f32x4*>(a), static_cast<const f32x4*>(b), n / 4, static_cast<hipStream_t>(stream));
  IBV_CHECK(hipGetLastError());
  return 0;
}

// One "schedule" = `steps` dependent steps of n fp32 elements each (dst = a + b), operands walking
// through three regions of region_bytes.  How the steps are issued:
//   mode 0  one stream, ordinary in-order launches (what the engine's chain of launches is)
//   mode 1  one stream, launches without the implicit barrier between them (hipExtAnyOrderLaunch)
//   mode 2  an explicit HIP graph of kernel nodes: `chains` parallel chains, each taking 1/chains of every step
//   mode 3  `chains` streams, issued eagerly, each taking 1/chains of every step
//   mode 4  one stream, only every `chains`-th launch keeps the implicit barrier
// Result: microseconds per schedule at device pace (schedules issued back to back, no host wait between).
int ibv_probe_chains(int mode, void* ra, void* rb, void* rd, size_t region_bytes, size_t n, int steps, int chains, int iters, double* us) {
  const Region m = {static_cast<char*>(ra), static_cast<char*>(rb), static_cast<char*>(rd), region_bytes};
  const size_t bytes = n * 4, positions = m.bytes / bytes;
  if (positions == 0 || chains < 1 || n % (static_cast<size_t>(mode == 4 ? 1 : chains) * 4 * 1024)) {
    snprintf(g_error, sizeof g_error, "bad shape");
    return 1;
  }
  hipStream_t s;
  IBV_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  const uint64_t sub = n / chains, subvec = sub / 4;
  int rc = 0;
  if (mode == 0 || mode == 1 || mode == 4) {
    // mode 4: every `chains`-th launch keeps the barrier, the others go without it
    rc = DevicePace(s, 2, iters, [&](int) {
      for (int r = 0; r < steps; r++) {
        const size_t pos = r % positions;
        const unsigned flags = mode == 4 ? (r % chains == 0 ? 0u : 1u) : static_cast<unsigned>(mode);
        LaunchLikeShipped((f32x4*)(m.d + pos * bytes), (const f32x4*)(m.a + pos * bytes), (const f32x4*)(m.b + pos * bytes), n / 4, s, flags);
      }
      return 0;
    }, us);
  } else if (mode == 2) {
    hipGraph_t g;
    IBV_CHECK(hipGraphCreate(&g, 0));
    struct Args {
      f32x4* d;
      const f32x4* a;
      const f32x4* b;
      uint64_t nt;
    };
    std::vector<Args> args(static_cast<size_t>(chains) * steps);
    std::vector<void*> ptrs(args.size() * 4);
    std::vector<hipGraphNode_t> last(chains, nullptr);
    const bool small = subvec / 256 < 2049;
    for (int r = 0; r < steps; r++) {
      const size_t pos = r % positions;
      for (int c = 0; c < chains; c++) {
        Args& A = args[static_cast<size_t>(r) * chains + c];
        A = Args{(f32x4*)(m.d + pos * bytes + c * sub * 4), (const f32x4*)(m.a + pos * bytes + c * sub * 4),
                 (const f32x4*)(m.b + pos * bytes + c * sub * 4), subvec / (small ? 256 : 128)};
        void** kp = &ptrs[(static_cast<size_t>(r) * chains + c) * 4];
        kp[0] = &A.d; kp[1] = &A.a; kp[2] = &A.b; kp[3] = &A.nt;
        hipKernelNodeParams p;
        memset(&p, 0, sizeof p);
        p.func = small ? (void*)OneShot<256, 1, true, true> : (void*)OneShot<128, 1, true, true>;
        p.gridDim = dim3((unsigned)A.nt);
        p.blockDim = dim3(small ? 256 : 128);
        p.kernelParams = kp;
        hipGraphNode_t node;
        IBV_CHECK(hipGraphAddKernelNode(&node, g, last[c] ? &last[c] : nullptr, last[c] ? 1 : 0, &p));
        last[c] = node;
      }
    }
    hipGraphExec_t ex;
    IBV_CHECK(hipGraphInstantiate(&ex, g, nullptr, nullptr, 0));
    rc = DevicePace(s, 2, iters, [&](int) { IBV_CHECK(hipGraphLaunch(ex, s)); return 0; }, us);
    (void)hipGraphExecDestroy(ex);
    (void)hipGraphDestroy(g);
  } else if (mode == 3) {
    std::vector<hipStream_t> st(chains);
    std::vector<hipEvent_t> ev(chains);
    hipEvent_t go;
    IBV_CHECK(hipEventCreateWithFlags(&go, hipEventDisableTiming));
    for (int i = 0; i < chains; i++) {
      IBV_CHECK(hipStreamCreateWithFlags(&st[i], hipStreamNonBlocking));
      IBV_CHECK(hipEventCreateWithFlags(&ev[i], hipEventDisableTiming));
    }
    rc = DevicePace(s, 2, iters, [&](int) {
      IBV_CHECK(hipEventRecord(go, s));
      for (int c = 0; c < chains; c++) IBV_CHECK(hipStreamWaitEvent(st[c], go, 0));
      for (int r = 0; r < steps; r++) {
        const size_t pos = r % positions;
        for (int c = 0; c < chains; c++)
          LaunchLikeShipped((f32x4*)(m.d + pos * bytes + c * sub * 4), (const f32x4*)(m.a + pos * bytes + c * sub * 4),
                            (const f32x4*)(m.b + pos * bytes + c * sub * 4), subvec, st[c], 0);
      }
      for (int c = 0; c < chains; c++) {
        IBV_CHECK(hipEventRecord(ev[c], st[c]));
        IBV_CHECK(hipStreamWaitEvent(s, ev[c], 0));
      }
      return 0;
    }, us);
    for (int i = 0; i < chains; i++) {
      (void)hipStreamSynchronize(st[i]);
      (void)hipStreamDestroy(st[i]);
      (void)hipEventDestroy(ev[i]);
    }
    (void)hipEventDestroy(go);
  } else {
    snprintf(g_error, sizeof g_error, "unknown mode %d", mode);
    rc = 1;
  }
  (void)hipStreamSynchronize(s);
  (void)hipStreamDestroy(s);
  return rc;
}

// The same schedule with per-chunk ready counters in the kernels (4 chunks per step):
//   flags 1 = every wave signals its chunk's counter, 3 = and every workgroup waits for the previous step's.
// any_order as in mode 1 above.  *gave_up is set if some workgroup's bounded wait ran out.
int ibv_probe_flags(int flags, int any_order, void* ra, void* rb, void* rd, size_t region_bytes, size_t n, int steps, int iters, double* us,
                    int* gave_up) {
  const Region m = {static_cast<char*>(ra), static_cast<char*>(rb), static_cast<char*>(rd), region_bytes};
  const size_t bytes = n * 4, positions = m.bytes / bytes;
  if (positions == 0 || n % (4 * 4 * 1024) || steps > 60) {
    snprintf(g_error, sizeof g_error, "bad shape");
    return 1;
  }
  hipStream_t s;
  IBV_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  uint32_t* ctr;
  IBV_CHECK(hipMalloc(&ctr, 64 * 64 * 4));
  IBV_CHECK(hipMemset(ctr, 0, 64 * 64 * 4));
  uint32_t* err = ctr + 63 * 64;
  constexpr int T = 128;
  const uint64_t nt = n / 4 / T;
  const uint32_t tiles_per_chunk = (uint32_t)(nt / 4), waves_per_chunk = tiles_per_chunk * (T / 64);
  uint32_t epoch = 0;
  const int rc = DevicePace(s, 2, iters, [&](int) {
    epoch++;
    for (int r = 0; r < steps; r++) {
      const size_t pos = r % positions;
      f32x4* d = (f32x4*)(m.d + pos * bytes);
      const f32x4* a = (const f32x4*)(m.a + pos * bytes);
      const f32x4* b = (const f32x4*)(m.b + pos * bytes);
      const uint32_t* prev = r ? ctr + (r - 1) * 64 : nullptr;
      uint32_t* mine = ctr + r * 64;
      const uint32_t target = epoch * waves_per_chunk;
      if (flags == 3)
        hipExtLaunchKernelGGL((Flagged<T, true, true>), dim3((unsigned)nt), dim3(T), 0, s, nullptr, nullptr, any_order, d, a, b, nt, prev, mine,
                              tiles_per_chunk, target, err);
      else if (flags == 1)
        hipExtLaunchKernelGGL((Flagged<T, true, false>), dim3((unsigned)nt), dim3(T), 0, s, nullptr, nullptr, any_order, d, a, b, nt, prev, mine,
                              tiles_per_chunk, target, err);
      else
        hipExtLaunchKernelGGL((Flagged<T, false, false>), dim3((unsigned)nt), dim3(T), 0, s, nullptr, nullptr, any_order, d, a, b, nt, prev, mine,
                              tiles_per_chunk, target, err);
    }
    return 0;
  }, us);
  uint32_t e = 0;
  if (rc == 0) IBV_CHECK(hipMemcpy(&e, err, 4, hipMemcpyDeviceToHost));
  *gave_up = static_cast<int>(e);
  (void)hipFree(ctr);
  (void)hipStreamDestroy(s);
  return rc;
}

// Host cost of ONE BLOCKING CALL that issues `steps` dependent launches of n elements and returns when
// they are done; *us is wall time per call, to be compared with mode 0 of ibv_probe_chains.
//   method 0  eager launches + hipStreamSynchronize
//   method 1  eager launches + spin on hipStreamQuery
//   method 2  eager launches + a one-thread kernel that writes a flag in pinned host memory; the host spins on the flag
//   method 3  graph (one chain) + hipStreamSynchronize
//   method 4  graph + the flag kernel (launched eagerly behind it) + host spins on the flag
//   method 7  graph + hipStreamWriteValue64 of a flag in pinned host memory (a command-processor write, no kernel) + host spins
//   method 9  graph whose last node stores the device clock to pinned host memory; host spins until the word changes (what the library does)
//   method 5  `steps` empty kernels + hipStreamSynchronize (n ignored)
//   method 6  `steps` empty kernels, calls back to back without waiting (the device's cost of a kernel boundary)
int ibv_probe_blocking_call(int method, void* ra, void* rb, void* rd, size_t region_bytes, size_t n, int steps, int iters, double* us) {
  const Region m = {static_cast<char*>(ra), static_cast<char*>(rb), static_cast<char*>(rd), region_bytes};
  const size_t bytes = n * 4, positions = m.bytes / bytes;
  if (positions == 0 || n % (4 * 1024)) {
    snprintf(g_error, sizeof g_error, "bad shape");
    return 1;
  }
  hipStream_t s;
  IBV_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  uint32_t* hflag = nullptr;
  IBV_CHECK(hipHostMalloc((void**)&hflag, 64, hipHostMallocMapped));
  hflag[0] = hflag[1] = 0;
  uint32_t* dflag = nullptr;
  IBV_CHECK(hipHostGetDevicePointer((void**)&dflag, hflag, 0));
  auto issue = [&]() {
    for (int r = 0; r < steps; r++) {
      const size_t pos = r % positions;
      LaunchLikeShipped((f32x4*)(m.d + pos * bytes), (const f32x4*)(m.a + pos * bytes), (const f32x4*)(m.b + pos * bytes), n / 4, s, 0);
    }
  };
  hipGraph_t g = nullptr;
  hipGraphExec_t ex = nullptr;
  struct Args {
    f32x4* d;
    const f32x4* a;
    const f32x4* b;
    uint64_t nt;
  };
  std::vector<Args> args(steps);
  std::vector<void*> ptrs(static_cast<size_t>(steps) * 4);
  uint64_t* dclock = reinterpret_cast<uint64_t*>(dflag);
  void* clock_args[1] = {&dclock};
  if (method == 3 || method == 4 || method >= 7) {
    IBV_CHECK(hipGraphCreate(&g, 0));
    hipGraphNode_t last = nullptr;
    const bool small = n / 4 / 256 < 2049;
    for (int r = 0; r < steps; r++) {
      const size_t pos = r % positions;
      args[r] = Args{(f32x4*)(m.d + pos * bytes), (const f32x4*)(m.a + pos * bytes), (const f32x4*)(m.b + pos * bytes), n / 4 / (small ? 256 : 128)};
      void** kp = &ptrs[static_cast<size_t>(r) * 4];
      kp[0] = &args[r].d; kp[1] = &args[r].a; kp[2] = &args[r].b; kp[3] = &args[r].nt;
      hipKernelNodeParams p;
      memset(&p, 0, sizeof p);
      p.func = small ? (void*)OneShot<256, 1, true, true> : (void*)OneShot<128, 1, true, true>;
      p.gridDim = dim3((unsigned)args[r].nt);
      p.blockDim = dim3(small ? 256 : 128);
      p.kernelParams = kp;
      hipGraphNode_t node;
      IBV_CHECK(hipGraphAddKernelNode(&node, g, last ? &last : nullptr, last ? 1 : 0, &p));
      last = node;
    }
    if (method == 9) {
      hipKernelNodeParams p;
      memset(&p, 0, sizeof p);
      p.func = (void*)StoreClock;
      p.gridDim = dim3(1);
      p.blockDim = dim3(1);
      p.kernelParams = clock_args;
      hipGraphNode_t node;
      IBV_CHECK(hipGraphAddKernelNode(&node, g, last ? &last : nullptr, last ? 1 : 0, &p));
    }
    IBV_CHECK(hipGraphInstantiate(&ex, g, nullptr, nullptr, 0));
  }
  const volatile uint64_t* hclock = reinterpret_cast<volatile uint64_t*>(hflag);
  uint32_t tick = 0;
  int rc = 0;
  switch (method) {
    case 0: rc = WallClock(3, iters, [&](int) { issue(); IBV_CHECK(hipStreamSynchronize(s)); return 0; }, us); break;
    case 1: rc = WallClock(3, iters, [&](int) { issue(); while (hipStreamQuery(s) == hipErrorNotReady) {} return 0; }, us); break;
    case 2: rc = WallClock(3, iters, [&](int) {
        issue();
        tick++;
        hipLaunchKernelGGL(SetFlag, dim3(1), dim3(1), 0, s, (volatile uint32_t*)dflag, tick);
        while (*(volatile uint32_t*)hflag != tick) {}
        return 0;
      }, us); break;
    case 3: rc = WallClock(3, iters, [&](int) { IBV_CHECK(hipGraphLaunch(ex, s)); IBV_CHECK(hipStreamSynchronize(s)); return 0; }, us); break;
    case 4: rc = WallClock(3, iters, [&](int) {
        IBV_CHECK(hipGraphLaunch(ex, s));
        tick++;
        hipLaunchKernelGGL(SetFlag, dim3(1), dim3(1), 0, s, (volatile uint32_t*)dflag, tick);
        while (*(volatile uint32_t*)hflag != tick) {}
        return 0;
      }, us); break;
    case 7: rc = WallClock(3, iters, [&](int) {
        IBV_CHECK(hipGraphLaunch(ex, s));
        tick++;
        IBV_CHECK(hipStreamWriteValue64(s, dflag, tick, 0));
        while (*(volatile uint64_t*)hflag != tick) {}
        return 0;
      }, us); break;
    case 9: rc = WallClock(3, iters, [&](int) {
        const uint64_t before = *hclock;
        IBV_CHECK(hipGraphLaunch(ex, s));
        while (*hclock == before) {}
        return 0;
      }, us); break;
    case 5: rc = WallClock(3, iters, [&](int) {
        for (int r = 0; r < steps; r++) hipLaunchKernelGGL(Null, dim3(1), dim3(64), 0, s);
        IBV_CHECK(hipStreamSynchronize(s));
        return 0;
      }, us); break;
    case 6: rc = DevicePace(s, 3, iters, [&](int) {
        for (int r = 0; r < steps; r++) hipLaunchKernelGGL(Null, dim3(1), dim3(64), 0, s);
        return 0;
      }, us); break;
    default:
      snprintf(g_error, sizeof g_error, "unknown method %d", method);
      rc = 1;
  }
  (void)hipStreamSynchronize(s);
  if (ex) (void)hipGraphExecDestroy(ex);
  if (g) (void)hipGraphDestroy(g);
  (void)hipHostFree(hflag);
  (void)hipStreamDestroy(s);
  return rc;
}

}  // extern "C"
