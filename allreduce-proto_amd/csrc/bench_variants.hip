// MEASUREMENT ONLY: libibcomm_hip_bench.so, loaded by bench.py's --sweep and --ceiling legs (and for
// `roofline.ceiling` of the default run) and by nothing else.  The shipped library (libibcomm_hip.so)
// contains none of this.
//
// Alternative forms of the streaming kernel dst = a + b (or dst = a) on fp32, one segment, all
// pointers 16-byte aligned: other workgroup sizes, several vectors per lane, persistent grid-stride
// loops with and without software pipelining, contiguous spans per workgroup, and every cache-policy
// bit combination the gfx950 vector memory instructions take.  The sweep times each at the launch
// shapes the allreduce schedules use, next to the shipped kernel, which is how the shipped geometry
// was chosen and how far it is from the best any of these forms reaches ("the ceiling") is tracked.
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

}  // extern "C"
