// Shared host/device helpers of the hpx kernel library (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <mutex>
#include <vector>

#include "hpx.h"
#include "hpx_completion_log.h"

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
// A new record under `name` and its two events, not yet recorded.
void prof_events(const char* name, hipEvent_t* start, hipEvent_t* stop);

// Every kernel goes out through these macros.  With hpx_profile_enable(1) a launch carries two HIP events that
// take the kernel's own begin and end times (hipExtLaunchKernelGGL), so hpx_profile_query reports the durations a
// kernel trace shows; events recorded on the stream around a launch would add the hand-over between launches
// (1-2 us) to every kernel.
#define HPX_LAUNCH_LDS(NAME, PROF, KERNEL, GRID, BLOCK, LDS, STREAM, ...)                        \
  do {                                                                                           \
    if (PROF) {                                                                                  \
      hipEvent_t hpx_e0_ = nullptr, hpx_e1_ = nullptr;                                           \
      hpx::prof_events(NAME, &hpx_e0_, &hpx_e1_);                                                \
      hipExtLaunchKernelGGL(KERNEL, GRID, BLOCK, LDS, STREAM, hpx_e0_, hpx_e1_, 0, __VA_ARGS__); \
    } else {                                                                                     \
      hipLaunchKernelGGL(KERNEL, GRID, BLOCK, LDS, STREAM, __VA_ARGS__);                         \
    }                                                                                            \
  } while (0)
#define HPX_LAUNCH(NAME, KERNEL, GRID, BLOCK, STREAM, ...) \
  HPX_LAUNCH_LDS(NAME, hpx::g_prof_on, KERNEL, GRID, BLOCK, 0, STREAM, __VA_ARGS__)

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
  uint8_t* aux = nullptr;  // second grow-only block, for the rare call whose needs are only known half-way through
  size_t aux_bytes = 0;
  uint32_t* state = nullptr;
  uint8_t* pinned = nullptr;
  // Epoch-tagged 64-bit reduction slots (see ensure_slots): memory that only ever
  // holds (epoch << 32 | key) words, so a call with a newer epoch needs no reset.
  uint64_t* slots = nullptr;
  size_t slot_words = 0;
  uint32_t epoch = 0;
  // Exchange memory of the grid-wide barrier (see ensure_barrier): it only ever
  // holds generation-tagged words; bar_gen is the generation of the last launch.
  uint32_t* bar = nullptr;
  uint32_t bar_gen = 0;
  int num_cus = 0;
  bool barrier_broken = false;  // a barrier wait expired on this stream: barrier kernels stay off
  // Tensors that barrier kernels have encoded on this stream since the stream was last known to be
  // good: if one of those kernels gave up at its barrier, its messages are encoded again from
  // these records by the kernels that need no barrier (hpx_terngrad_encode_status).
  struct ResidentRec {
    const float* x;
    uint8_t* out;
    int32_t n, out_size;
    uint64_t seed;
    uint8_t bits, random;
  };
  // Every workgroup of a barrier launch that gets through its barrier stores the launch's generation into its
  // word of `done` (pinned host memory); a launch is marked in the log by its generation and grid, and the next
  // call drops the records of every launch whose workgroups have all reported while the expiry flag is down, so
  // the log only ever names buffers of launches that may still have to be repeated (hpx_completion_log.h).  No
  // event, nothing extra on the stream.
  struct ResidentMark {
    uint32_t gen;
    int32_t grid;
  };
  CompletionLog<ResidentRec, ResidentMark> resident_log;
  uint32_t* done = nullptr;  // kBarMaxWorkgroups words, see ensure_barrier
  uint64_t repaired = 0;  // tensors encoded again after an expired barrier, ever
  uint64_t gd_fallbacks = 0;  // sparsifier tensors whose provisional threshold was not below the exact one, ever
};
constexpr size_t kStateWords = 4096;       // 16 KiB
constexpr size_t kStatusWord = kStateWords - 16;  // sticky flags live here
constexpr size_t kPinnedBytes = 1 << 16;
constexpr size_t kBarWords = 524288;                      // 2 MiB of exchange memory for grid-wide barriers
constexpr size_t kPinnedFlagOffset = kPinnedBytes - 64;   // host word raised by a kernel whose barrier wait expired

// The record for the calling thread's current device and `stream` (created on
// first use).  Lock its `mu`, then call ensure_workspace for the scratch size
// the call needs (may wait for the stream when the block has to grow).
Workspace* workspace_record(hipStream_t stream);
int ensure_workspace(Workspace* ws, size_t dev_bytes);
// The same for the second block (ws->aux); waits for the stream when it has to grow.
int ensure_aux(Workspace* ws, size_t bytes);
// At least `words` zero-initialised-at-allocation 64-bit slots, never used for anything else.
int ensure_slots(Workspace* ws, size_t words);
// Zeroed barrier exchange memory and the CU count of the device (both created once).
int ensure_barrier(Workspace* ws);
// Kernels that wait at a grid-wide barrier need every CU for themselves: two of them
// running at once on different streams could each hold CUs the other is waiting
// for.  So only one stream per device may launch them: the first that asks.
// Returns whether `ws` is (now) that stream's workspace.
bool claim_barrier_kernels(Workspace* ws);
// Whether a barrier kernel on this stream has raised the pinned expiry flag (ws->mu held, workspace ensured).
bool barrier_expired(const Workspace* ws);
// Frees the workspace of (current device, `stream`) and hands back its claim on the barrier kernels.
int release_stream_workspace(hipStream_t stream);

uint64_t clock_seed();

// HPX_ERR_ARG (text names `who`) when `stream` is being captured into a graph: for entry points that wait for
// the stream or put per-call tags into their kernel arguments, neither of which a replayed graph could repeat.
int reject_capture(hipStream_t stream, const char* who);

// Copies `count` byte ranges in as few launches as their number allows (one kernel, a table of ranges in
// its arguments).  Either side may be device memory or pinned host memory: the scheduler moves all
// messages of a batch between the device buffers and the host buffers with it instead of one
// hipMemcpyAsync per message (200 of those cost the host more than the copies take).
int copy_ranges(int count, uint8_t* const* dst, const uint8_t* const* src, const int64_t* bytes, hipStream_t st);

// How the outputs of a decode call relate: 0 = pairwise disjoint, 1 = some are
// named more than once but every overlap is an exact duplicate (same pointer,
// same size: several messages accumulate into one tensor), 2 = partial overlaps.
int classify_outputs(int count, float* const* outs, const int32_t* sizes);

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

// Streaming variants: data that is touched once (or for the last time) is
// loaded and stored with the non-temporal hint so it does not displace lines in
// L2 / Infinity Cache; on MI355X this lifts a read-read-write stream from about
// 5.5 to 6.4 TB/s.
__device__ __forceinline__ float4 ld4_stream(const float* p) {
  const f32x4u* q = reinterpret_cast<const f32x4u*>(p);
  return make_float4(__builtin_nontemporal_load(&q->x), __builtin_nontemporal_load(&q->y),
                     __builtin_nontemporal_load(&q->z), __builtin_nontemporal_load(&q->w));
}
__device__ __forceinline__ void st4_stream(float* p, float4 v) {
  f32x4u* q = reinterpret_cast<f32x4u*>(p);
  __builtin_nontemporal_store(v.x, &q->x);
  __builtin_nontemporal_store(v.y, &q->y);
  __builtin_nontemporal_store(v.z, &q->z);
  __builtin_nontemporal_store(v.w, &q->w);
}

// Output policy of the write-only decoders: streaming (non-temporal) stores whatever the size of the output.  A
// pure write stream that fits the 256 MB Infinity Cache would otherwise finish with its lines dirty in the cache
// and leave the write-back to whichever kernel runs next; a larger one is simply written faster (110 M elements:
// 73 us against 91 with plain stores in the TernGrad decode, 73 against 85 in TBQ's).  The option stays for
// callers whose next kernel reads the decoded tensor straight back.
constexpr size_t kStreamStoreMaxBytes = size_t(1) << 62;
// A write stream of streaming stores runs faster with few workgroups per CU (their stores then reach memory as a
// compact front): launches of the write-mode decoders ask for this much LDS they never touch, which holds a CU to
// three (52 KiB) or four (40 KiB) workgroups of 256 lanes.  TBQ decode of 110 M elements: 73 -> 62 us at three
// (66 at four, 80 at two); TernGrad decode: 73 -> 65 us at four (72 at three).  Kernels that also read what they
// write (the add-mode decoders, the encoders' in-place residual update, GradDrop's stream pass) gain nothing.
constexpr int kWriteStreamPadLds2 = 64 * 1024;  // two per CU: the PowerSGD decode (one read, three writes: 792 -> 755 us)
constexpr int kWriteStreamPadLds3 = 52 * 1024;
constexpr int kWriteStreamPadLds4 = 40 * 1024;
// The limit in force: option "stream_store_max_bytes".
size_t stream_store_max_bytes();

// Tuning options (hpx_set_option / hpx_get_option).  Each starts from the
// environment variable HPX_<NAME IN CAPITALS> when that is set, else from its default.
enum Option {
  kOptStreamStoreMaxBytes = 0,  // "stream_store_max_bytes", default kStreamStoreMaxBytes
  kOptTerngradResidentMin,      // "terngrad_resident_min": smallest tensor (elements) that takes the
                                // single-launch resident encode; negative = never.  Default 5 * 2^20:
                                // below about 4 M elements the two-launch encode is faster (2 M: 7.3 against 10.9 us;
                                // 4 M: 11.0 against 11.3; 6 M: 13.7 against 12.1).
  kOptTerngradBarrierMs,        // "terngrad_barrier_ms": bound on the resident kernel's barrier wait.  Default 2000.
  kOptTerngradResidentBucket,   // "terngrad_resident_bucket": 1 = a call with several tensors that fit the chip together
                                // and add up to terngrad_resident_min elements takes ONE resident launch.  Default 1.
  kOptTerngradResidentWorkgroups,  // "terngrad_resident_workgroups": workgroups of a resident launch; 0 (default) = one per CU.
                                   // For a process that may only use some of the CUs (a CU mask), which the device's CU
                                   // count does not show: a resident launch needs all its workgroups running at once.
  kOptTerngradResidentStreamed,  // "terngrad_resident_streamed": 1 (default) = a tensor larger than the chip holds also
                                 // takes the single launch, which keeps the tensor's head on chip and streams the
                                 // rest twice; 0 = such tensors take the two-launch encode.
  kOptGdProvisionalMinSamples,  // "gd_provisional_min_samples": a sparsifier call whose tensors' samples add up to this many
                                // takes the path that starts its pass from a provisional threshold (hpx_gd.hip); negative
                                // (the default): never.  Measured on the 138 M-element configuration it does not pay:
                                // 355-363 us against 346 for the gather path (the gather's lines warm the cache for the
                                // pass, which runs 25 us longer without them, and the single-workgroup selections and the
                                // recount cost what the gather saved).
  kOptGdProvisionalMargin,      // "gd_provisional_margin": how many times the expected number of entries that threshold lets
                                // through.  Default 3; 0 puts it at the top of its samples, which all but forces the
                                // fall-back to the gather path (for tests of that fall-back).
  kOptClockSeed,                // "clock_seed": what an encoder called with seeds == NULL uses in place of the wall clock
                                // (terngrad_body.h:247-251, gd_body.h:138-140); negative (default) = read the clock.
                                // Makes the C++ drivers, which cannot pass seeds, reproducible.
  kOptCount
};
int64_t option(Option o);

// Index of the segment owning `tile`: the largest s < nseg with start[s] <= tile,
// where start[] is the strictly increasing exclusive prefix of tiles per
// segment.  `tile` is wave-uniform and every lane of the wave must be active.
// Each round of dependent loads from the argument table, cold at the start of
// a launch, delays the first data load of every workgroup of the first wave
// of workgroups by about a microsecond, so the search is ONE round: tables of
// up to 16 entries are read whole on the scalar unit; larger ones are read by
// the lanes (entry k by lane k % 64), and the answer is the number of entries
// that do not exceed `tile`, counted with ballots.
template <int CAP>
__device__ __forceinline__ int find_segment(const int32_t (&start)[CAP + 1], int nseg, int tile) {
  if constexpr (CAP <= 16) {
    int s = 0;
#pragma unroll
    for (int k = 1; k < CAP; k++) s += (k < nseg && start[k] <= tile) ? 1 : 0;
    return s;
  } else {
    const int lane = threadIdx.x & (kWave - 1);
    int s = 0;
#pragma unroll
    for (int j = 0; j < CAP; j += kWave) {
      const int k = j + lane;
      const int v = start[k < CAP ? k : CAP];
      s += __popcll(__ballot(k >= 1 && k < nseg && v <= tile));
    }
    return s;
  }
}

// A pointer that has been kept in LDS, or put together from integers, has lost its address space, and a load
// through it becomes a FLAT instruction.  The compiler must assume that FLAT loads finish out of order with all
// other memory operations, so with one of them in flight every wait becomes a wait for everything
// (s_waitcnt vmcnt(0) lgkmcnt(0)) and nothing overlaps.  as_global says what the pointer points to; the load has
// to go through the returned pointer itself (a cast back to an ordinary pointer undoes it).
template <typename T>
using global_ptr = const __attribute__((address_space(1))) T*;
template <typename T>
__device__ __forceinline__ global_ptr<T> as_global(const T* p) {
  return (global_ptr<T>)p;
}

// ---- grid-wide exchange / barrier --------------------------------------------
// For kernels launched with at most kBarMaxWorkgroups workgroups that are all
// resident at once (the host guarantees it: grid <= CUs, one workgroup fits a CU,
// and only one stream per device launches such kernels).
constexpr int kBarMaxWorkgroups = 256;
constexpr int kBarWaves = 4;            // waves of a workgroup that take part: each looks after a quarter of the grid
constexpr int kBarQuarter = kBarMaxWorkgroups / kBarWaves;  // = the lanes of a wave
constexpr int kBarRecWords = 4;         // 64-bit words per record (three used)
// Exchange memory, in 64-bit words: one area per workgroup, holding one record per source workgroup.
constexpr size_t kBarAreaWords = size_t(kBarMaxWorkgroups) * kBarRecWords;  // 8 KiB
constexpr size_t kBarTotalWords = size_t(kBarMaxWorkgroups) * kBarAreaWords;
static_assert(kBarTotalWords * 8 <= kBarWords * 4, "barrier memory too small");
static_assert(kBarQuarter == kWave, "a wave's quarter is one source per lane-quad times four rounds");

// Grid-wide exchange of (max key, min key, first-zero key) and barrier in one.
// All lanes of the first kBarWaves waves of every workgroup call it once per launch
// with the workgroup's three keys (the same in every caller of a workgroup) and the
// caller's wave index.  On success k0, k1, k2 hold, the same in every lane, the maximum of
// each key over the quarter of the grid this wave looks after (workgroups
// 64 * wave ... 64 * wave + 63); the caller folds the quarters.
//
// The protocol is ONE hand-over and uses only stores and polling loads, no
// read-modify-write and no fence: a workgroup writes its record (three
// self-validating 64-bit words, generation in the high half) into the area of
// EVERY workgroup, the three words from neighbouring lanes so that they leave as
// one request; every workgroup polls its own area until all records carry this
// generation.  A polled line has one reader and four writers; nothing is ever
// reset (generations only grow).  With four waves at it, a wave keeps just four
// loads in flight per round.  (Two hand-overs through group leaders - each member
// reports to its leader, the leader to everyone - took 2.4 us from the last
// arrival, this takes 1.4; a counter-based barrier - fence, two dependent atomics, a release flag,
// then reading the reduction slots - took 7 us; polling one shared word from all
// 256 workgroups took 10.)
__device__ __forceinline__ bool grid_exchange(uint64_t* bar, uint32_t gen, uint64_t spin_limit, uint32_t wave, uint32_t& k0, uint32_t& k1, uint32_t& k2) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t nwg = gridDim.x, me = blockIdx.x;
  const uint32_t rec = lane / kBarRecWords, word = lane % kBarRecWords;
  const uint32_t q0 = wave * uint32_t(kBarQuarter);  // first workgroup of this wave's quarter
  if (q0 >= nwg) {
    k0 = k1 = k2 = 0u;
    return true;
  }
  const uint64_t tag = uint64_t(gen) << 32;
  const uint64_t t0 = wall_clock64();
  unsigned long long* base = reinterpret_cast<unsigned long long*>(bar);

  // (written with masks: as a chain of selects the compiler turns it into a table in private memory)
  const uint32_t mine_key = (k0 & (0u - uint32_t(word == 0))) | (k1 & (0u - uint32_t(word == 1))) | (k2 & (0u - uint32_t(word == 2)));
  if (word < 3) {
#pragma unroll
    for (uint32_t j = 0; j < uint32_t(kWave / (kWave / kBarRecWords)); j++) {
      const uint32_t d = q0 + j * (kWave / kBarRecWords) + rec;
      if (d < nwg)
        __hip_atomic_store(&base[(size_t(d) * kBarMaxWorkgroups + me) * kBarRecWords + word], tag | mine_key, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
  }

  const unsigned long long* area = base + size_t(me) * kBarAreaWords + size_t(q0) * kBarRecWords;
  uint32_t k = 0;
  for (;;) {
    unsigned long long v[kBarRecWords];
#pragma unroll
    for (int j = 0; j < kBarRecWords; j++) v[j] = __hip_atomic_load(&area[j * kWave + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool all = true;
    k = 0;
#pragma unroll
    for (int j = 0; j < kBarRecWords; j++) {
      const uint32_t src = q0 + uint32_t(j) * (kWave / kBarRecWords) + rec;
      const bool idle = word == 3 || src >= nwg;
      all = all && (idle || uint32_t(v[j] >> 32) == gen);
      const uint32_t kk = idle ? 0u : uint32_t(v[j]);
      k = kk > k ? kk : k;
    }
    if (__ballot(all) == ~0ull) break;
    if (wall_clock64() - t0 > spin_limit) return false;
    __builtin_amdgcn_s_sleep(1);
  }
#pragma unroll
  for (int o = kBarRecWords; o < kWave; o <<= 1) { const uint32_t t = __shfl_xor(k, o, 64); k = t > k ? t : k; }
  k0 = __builtin_amdgcn_readlane(k, 0);
  k1 = __builtin_amdgcn_readlane(k, 1);
  k2 = __builtin_amdgcn_readlane(k, 2);
  return true;
}


// The reference's 32-bit LCG (naive_random.hpp:15-33): x <- a*x + c.
constexpr uint32_t kLcgA = 1103515245u;
constexpr uint32_t kLcgC = 12345u;
// k-step jump x_k = A_k * x_0 + C_k, evaluated at compile time.
constexpr uint32_t lcg_mul(int k) { uint32_t a = 1; for (int i = 0; i < k; i++) a *= kLcgA; return a; }
constexpr uint32_t lcg_add(int k) { uint32_t c = 0; for (int i = 0; i < k; i++) c = c * kLcgA + kLcgC; return c; }

}  // namespace hpx
