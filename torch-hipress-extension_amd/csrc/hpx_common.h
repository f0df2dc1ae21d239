// Shared host/device helpers of the hpx kernel library (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "hpx.h"

#define HPX_API extern "C" __attribute__((visibility("default")))

namespace hpx {

// ---- error reporting -------------------------------------------------------
void set_error(const char* fmt, ...);
void clear_error();

#define HPX_HIP(call)                                                              \
  do {                                                                             \
    hipError_t e__ = (call);                                                       \
    if (e__ != hipSuccess) {                                                       \
      hpx::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__, __LINE__); \
      return HPX_ERR_HIP;                                                          \
    }                                                                              \
  } while (0)

#define HPX_ARG(cond, ...)        \
  do {                            \
    if (!(cond)) {                \
      hpx::set_error(__VA_ARGS__); \
      return HPX_ERR_ARG;         \
    }                             \
  } while (0)

// ---- per-kernel timing (measurement aid, off by default) ---------------------
extern bool g_prof_on;
void prof_begin(const char* name, hipStream_t st);
void prof_end(hipStream_t st);

// Every kernel goes out through this macro so that hpx_profile_* can bracket it
// with HIP events on the stream it is launched on.
#define HPX_LAUNCH(NAME, KERNEL, GRID, BLOCK, STREAM, ...)            \
  do {                                                                \
    if (hpx::g_prof_on) hpx::prof_begin(NAME, STREAM);                \
    hipLaunchKernelGGL(KERNEL, GRID, BLOCK, 0, STREAM, __VA_ARGS__);  \
    if (hpx::g_prof_on) hpx::prof_end(STREAM);                        \
  } while (0)

// ---- per-(device, stream) workspace ----------------------------------------
// `dev` is grow-only scratch whose contents are meaningless between calls.
// `state` is a small block that is zero when the library creates it and that
// every kernel leaves zero again (arrival counters), except the sticky status
// words at its end.  `pinned` is host memory for small read-backs.
struct Workspace {
  std::mutex mu;  // held while a call enqueues on this stream
  int device = -1;
  hipStream_t stream = nullptr;
  uint8_t* dev = nullptr;
  size_t dev_bytes = 0;
  uint32_t* state = nullptr;
  uint8_t* pinned = nullptr;
};
constexpr size_t kStateWords = 4096;       // 16 KiB
constexpr size_t kStatusWord = kStateWords - 16;  // sticky flags live here
constexpr size_t kPinnedBytes = 1 << 16;

// The record for the calling thread's current device and `stream` (created on
// first use).  Lock its `mu`, then call ensure_workspace for the scratch size
// the call needs (may wait for the stream when the block has to grow).
Workspace* workspace_record(hipStream_t stream);
int ensure_workspace(Workspace* ws, size_t dev_bytes);

uint64_t clock_seed();

// ---- device helpers --------------------------------------------------------
constexpr int kWave = 64;

// 16-byte vector of floats that is only assumed 4-byte aligned: tensors handed
// over by the caller may start at any element.  gfx950 global memory accepts
// unaligned 128-bit accesses.
struct __attribute__((packed, aligned(4))) f32x4u {
  float x, y, z, w;
};

__device__ __forceinline__ float4 ld4(const float* p) {
  f32x4u v = *reinterpret_cast<const f32x4u*>(p);
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st4(float* p, float4 v) {
  f32x4u u;
  u.x = v.x; u.y = v.y; u.z = v.z; u.w = v.w;
  *reinterpret_cast<f32x4u*>(p) = u;
}

// Index of the segment owning `tile`: largest s with start[s] <= tile, where
// start[0] = 0 < ... is the exclusive prefix of tiles per segment.  `tile` is
// wave-uniform, so this runs on the scalar unit.
template <int MAXSEG>
__device__ __forceinline__ int find_segment(const int32_t (&start)[MAXSEG + 1], int nseg, int tile) {
  int lo = 0, hi = nseg - 1;
  while (lo < hi) {
    int mid = (lo + hi + 1) >> 1;
    if (start[mid] <= tile) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// The reference's 32-bit LCG (naive_random.hpp:15-33): x <- a*x + c.
constexpr uint32_t kLcgA = 1103515245u;
constexpr uint32_t kLcgC = 12345u;
// k-step jump x_k = A_k * x_0 + C_k, evaluated at compile time.
constexpr uint32_t lcg_mul(int k) { uint32_t a = 1; for (int i = 0; i < k; i++) a *= kLcgA; return a; }
constexpr uint32_t lcg_add(int k) { uint32_t c = 0; for (int i = 0; i < k; i++) c = c * kLcgA + kLcgC; return c; }

}  // namespace hpx
