// Plain streaming kernels of known traffic for bench.py: what the memory system gives the simplest possible
// kernel of the codecs' shape (16 KiB per workgroup, 128-bit accesses, launch order = address order).  Not part
// of the product library; built into bench_probe.so beside bench.py.
//   kind 0  read `bytes` of a            (non-temporal loads)
//   kind 1  write `bytes` of a           (non-temporal stores)
//   kind 2  write `bytes` of a           (plain stores)
//   kind 3  a = a + b over `bytes` each  (read, read, write in place; non-temporal)
// a and b are device pointers, 16-byte aligned; bytes is rounded down to a multiple of 16 KiB.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <vector>

namespace {
constexpr int kWave = 64;
constexpr int kThreads = 256;
constexpr int kIters = 4;  // 16 KiB per workgroup

__device__ __forceinline__ float4 ld4_stream(const float* p) {
  return make_float4(__builtin_nontemporal_load(p), __builtin_nontemporal_load(p + 1), __builtin_nontemporal_load(p + 2),
                     __builtin_nontemporal_load(p + 3));
}
__device__ __forceinline__ void st4_stream(float* p, float4 v) {
  __builtin_nontemporal_store(v.x, p);
  __builtin_nontemporal_store(v.y, p + 1);
  __builtin_nontemporal_store(v.z, p + 2);
  __builtin_nontemporal_store(v.w, p + 3);
}

template <int KIND>
__global__ __launch_bounds__(kThreads) void probe_stream_kernel(float* __restrict__ a, const float* __restrict__ b) {
  const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const size_t g0 = size_t(blockIdx.x) * (kThreads * kIters) + wave * (kWave * kIters) + lane;  // float4 units
  if (KIND == 0) {
    float4 v[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++) v[k] = ld4_stream(a + (g0 + k * kWave) * 4);
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < kIters; k++) s += v[k].x + v[k].y + v[k].z + v[k].w;
    if (s == 1.2345e38f) a[0] = s;  // keeps the loads; never true for finite data of ordinary size
  } else if (KIND == 1 || KIND == 2) {
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const float4 v = make_float4(1.f, 2.f, 3.f, float(k));
      if (KIND == 1) st4_stream(a + (g0 + k * kWave) * 4, v); else *reinterpret_cast<float4*>(a + (g0 + k * kWave) * 4) = v;
    }
  } else {
    float4 x[kIters], y[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      x[k] = ld4_stream(a + (g0 + k * kWave) * 4);
      y[k] = ld4_stream(b + (g0 + k * kWave) * 4);
    }
#pragma unroll
    for (int k = 0; k < kIters; k++)
      st4_stream(a + (g0 + k * kWave) * 4, make_float4(x[k].x + y[k].x, x[k].y + y[k].y, x[k].z + y[k].z, x[k].w + y[k].w));
  }
}
}  // namespace

namespace {
// Event pairs for timed launches: a launch carries its pair, which takes the kernel's own begin and end times
// (the way the library's hpx_profile_* measures its kernels), not the hand-over between launches.
std::vector<hipEvent_t> g_events;
bool event_pair(int slot, hipEvent_t* e0, hipEvent_t* e1) {
  while (g_events.size() < size_t(2 * slot + 2)) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return false;
    g_events.push_back(e);
  }
  *e0 = g_events[2 * slot];
  *e1 = g_events[2 * slot + 1];
  return true;
}
}  // namespace

// 0 on success, -3 for a bad argument, -2 for a HIP error.  slot < 0: an ordinary launch; slot >= 0: the launch
// carries event pair `slot`, read back with bench_probe_elapsed_us once the stream has drained.
extern "C" __attribute__((visibility("default"))) int bench_probe_stream_timed(int kind, void* a, const void* b,
                                                                              int64_t bytes, void* stream, int slot) {
  if (kind < 0 || kind > 3 || !a || (kind == 3 && !b) || slot > 4095) return -3;
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) return -3;
  constexpr int64_t kTile = int64_t(kThreads) * kIters * 16;
  const int64_t tiles = bytes / kTile;
  if (tiles <= 0 || tiles > INT32_MAX) return -3;
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* fa = static_cast<float*>(a);
  const float* fb = static_cast<const float*>(b);
  const dim3 grid(static_cast<uint32_t>(tiles)), block(kThreads);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (slot >= 0 && !event_pair(slot, &e0, &e1)) return -2;
#define PROBE_LAUNCH(K)                                                                              \
  if (slot >= 0) hipExtLaunchKernelGGL(probe_stream_kernel<K>, grid, block, 0, st, e0, e1, 0, fa, fb); \
  else hipLaunchKernelGGL(probe_stream_kernel<K>, grid, block, 0, st, fa, fb)
  switch (kind) {
    case 0: PROBE_LAUNCH(0); break;
    case 1: PROBE_LAUNCH(1); break;
    case 2: PROBE_LAUNCH(2); break;
    default: PROBE_LAUNCH(3); break;
  }
#undef PROBE_LAUNCH
  return hipGetLastError() == hipSuccess ? 0 : -2;
}

extern "C" __attribute__((visibility("default"))) int bench_probe_stream(int kind, void* a, const void* b, int64_t bytes,
                                                                        void* stream) {
  return bench_probe_stream_timed(kind, a, b, bytes, stream, -1);
}

// Duration of the launch that carried event pair `slot`, in microseconds; negative on failure.
extern "C" __attribute__((visibility("default"))) double bench_probe_elapsed_us(int slot) {
  if (slot < 0 || size_t(2 * slot + 1) >= g_events.size()) return -1.0;
  float ms = 0.f;
  if (hipEventSynchronize(g_events[2 * slot + 1]) != hipSuccess) return -1.0;
  if (hipEventElapsedTime(&ms, g_events[2 * slot], g_events[2 * slot + 1]) != hipSuccess) return -1.0;
  return double(ms) * 1e3;
}
