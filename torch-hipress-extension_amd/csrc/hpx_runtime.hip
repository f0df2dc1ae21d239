// Library state that is not a kernel: error text, workspaces, seeds.
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <map>
#include <memory>
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <utility>
#include <vector>

#include "hpx_common.h"

namespace hpx {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
void clear_error() { g_err[0] = 0; }

static std::mutex g_ws_mu;
static std::map<std::pair<int, hipStream_t>, std::unique_ptr<Workspace>> g_ws;
static std::map<int, Workspace*> g_barrier_owner;  // guarded by g_ws_mu

Workspace* workspace_record(hipStream_t stream) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    set_error("hipGetDevice failed");
    return nullptr;
  }
  std::lock_guard<std::mutex> g(g_ws_mu);
  auto& slot = g_ws[{device, stream}];
  if (!slot) {
    slot.reset(new Workspace());
    slot->device = device;
    slot->stream = stream;
  }
  return slot.get();
}

int ensure_workspace(Workspace* ws, size_t dev_bytes) {
  if (!ws->state) {
    HPX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->state), kStateWords * sizeof(uint32_t)));
    HPX_HIP(hipMemset(ws->state, 0, kStateWords * sizeof(uint32_t)));
    // coherent: words a kernel stores with system scope can be read by the host while the kernel is still running
    HPX_HIP(hipHostMalloc(reinterpret_cast<void**>(&ws->pinned), kPinnedBytes, hipHostMallocCoherent));
    std::memset(ws->pinned, 0, kPinnedBytes);
  }
  if (dev_bytes > ws->dev_bytes) {
    // Work already queued on this stream may still use the old block.
    HPX_HIP(hipStreamSynchronize(ws->stream));
    if (ws->dev) HPX_HIP(hipFree(ws->dev));
    ws->dev = nullptr;
    ws->dev_bytes = 0;
    size_t want = dev_bytes + dev_bytes / 8 + (1 << 20);
    want = (want + 255) & ~size_t(255);
    HPX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->dev), want));
    ws->dev_bytes = want;
  }
  return HPX_OK;
}

int ensure_aux(Workspace* ws, size_t bytes) {
  if (bytes <= ws->aux_bytes) return HPX_OK;
  HPX_HIP(hipStreamSynchronize(ws->stream));
  if (ws->aux) HPX_HIP(hipFree(ws->aux));
  ws->aux = nullptr;
  ws->aux_bytes = 0;
  const size_t want = (bytes + bytes / 8 + 255) & ~size_t(255);
  HPX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->aux), want));
  ws->aux_bytes = want;
  return HPX_OK;
}

// ---- per-kernel timing --------------------------------------------------------
bool g_prof_on = false;
namespace {
struct ProfRec {
  const char* name;
  hipEvent_t start, stop;
};
std::mutex g_prof_mu;
std::vector<ProfRec> g_prof_recs;
std::vector<hipEvent_t> g_prof_pool;
hipEvent_t prof_event() {
  if (!g_prof_pool.empty()) {
    hipEvent_t e = g_prof_pool.back();
    g_prof_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
}  // namespace

void prof_events(const char* name, hipEvent_t* start, hipEvent_t* stop) {
  std::lock_guard<std::mutex> g(g_prof_mu);
  ProfRec r{name, prof_event(), prof_event()};
  g_prof_recs.push_back(r);
  *start = r.start;
  *stop = r.stop;
}

int ensure_slots(Workspace* ws, size_t words) {
  if (words <= ws->slot_words) return HPX_OK;
  HPX_HIP(hipStreamSynchronize(ws->stream));
  if (ws->slots) HPX_HIP(hipFree(ws->slots));
  ws->slots = nullptr;
  ws->slot_words = 0;
  const size_t want = words < 4096 ? 4096 : words * 2;
  HPX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->slots), want * sizeof(uint64_t)));
  HPX_HIP(hipMemset(ws->slots, 0, want * sizeof(uint64_t)));  // epoch 0 is never used by a call
  ws->slot_words = want;
  return HPX_OK;
}

bool claim_barrier_kernels(Workspace* ws) {
  std::lock_guard<std::mutex> g(g_ws_mu);
  auto it = g_barrier_owner.find(ws->device);
  if (it == g_barrier_owner.end()) {
    g_barrier_owner[ws->device] = ws;
    return true;
  }
  return it->second == ws;
}

bool barrier_expired(const Workspace* ws) {
  return ws->pinned && *reinterpret_cast<volatile const uint32_t*>(ws->pinned + kPinnedFlagOffset) != 0;
}

namespace {
int free_workspace(Workspace* ws) {
  int rc = HPX_OK;
  if (ws->dev && hipFree(ws->dev) != hipSuccess) rc = HPX_ERR_HIP;
  if (ws->aux && hipFree(ws->aux) != hipSuccess) rc = HPX_ERR_HIP;
  if (ws->state && hipFree(ws->state) != hipSuccess) rc = HPX_ERR_HIP;
  if (ws->slots && hipFree(ws->slots) != hipSuccess) rc = HPX_ERR_HIP;
  if (ws->bar && hipFree(ws->bar) != hipSuccess) rc = HPX_ERR_HIP;
  if (ws->pinned && hipHostFree(ws->pinned) != hipSuccess) rc = HPX_ERR_HIP;
  if (ws->done && hipHostFree(ws->done) != hipSuccess) rc = HPX_ERR_HIP;
  ws->done = nullptr;
  ws->resident_log.clear([](Workspace::ResidentMark) {});
  ws->dev = nullptr; ws->aux = nullptr; ws->state = nullptr; ws->slots = nullptr; ws->bar = nullptr; ws->pinned = nullptr;
  return rc;
}
}  // namespace

int release_stream_workspace(hipStream_t stream) {
  int device = 0;
  HPX_HIP(hipGetDevice(&device));
  std::unique_ptr<Workspace> ws;
  {
    std::lock_guard<std::mutex> g(g_ws_mu);
    auto it = g_ws.find({device, stream});
    if (it == g_ws.end()) return HPX_OK;
    ws = std::move(it->second);
    g_ws.erase(it);
    auto own = g_barrier_owner.find(device);
    if (own != g_barrier_owner.end() && own->second == ws.get()) g_barrier_owner.erase(own);
  }
  // Nothing can find the record any more; a call that had found it before holds its mutex until it has queued its work.
  { std::lock_guard<std::mutex> g(ws->mu); }
  HPX_HIP(hipStreamSynchronize(stream));
  return free_workspace(ws.get());
}

int ensure_barrier(Workspace* ws) {
  if (ws->bar) return HPX_OK;
  HPX_HIP(hipDeviceGetAttribute(&ws->num_cus, hipDeviceAttributeMultiprocessorCount, ws->device));
  HPX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->bar), kBarWords * sizeof(uint32_t)));
  HPX_HIP(hipMemset(ws->bar, 0, kBarWords * sizeof(uint32_t)));
  ws->bar_gen = 0;
  // one word per workgroup of a barrier launch, written by the GPU with system scope, read by the host at any time
  HPX_HIP(hipHostMalloc(reinterpret_cast<void**>(&ws->done), kBarMaxWorkgroups * sizeof(uint32_t), hipHostMallocCoherent));
  std::memset(ws->done, 0, kBarMaxWorkgroups * sizeof(uint32_t));
  return HPX_OK;
}

namespace {
struct OptionDef {
  const char* name;
  const char* env;
  int64_t def;
};
const OptionDef kOptions[kOptCount] = {
    {"stream_store_max_bytes", "HPX_STREAM_STORE_MAX_BYTES", int64_t(kStreamStoreMaxBytes)},
    {"terngrad_resident_min", "HPX_TERNGRAD_RESIDENT_MIN", int64_t(5) << 20},
    {"terngrad_barrier_ms", "HPX_TERNGRAD_BARRIER_MS", 2000},
    {"terngrad_resident_bucket", "HPX_TERNGRAD_RESIDENT_BUCKET", 1},
    {"terngrad_resident_workgroups", "HPX_TERNGRAD_RESIDENT_WORKGROUPS", 0},
    {"terngrad_resident_streamed", "HPX_TERNGRAD_RESIDENT_STREAMED", 1},
    {"gd_provisional_min_samples", "HPX_GD_PROVISIONAL_MIN_SAMPLES", -1},
    {"gd_provisional_margin", "HPX_GD_PROVISIONAL_MARGIN", 3},
    {"clock_seed", "HPX_CLOCK_SEED", -1},
};
std::atomic<int64_t> g_opt[kOptCount];
std::once_flag g_opt_once;
void options_init() {
  std::call_once(g_opt_once, [] {
    for (int i = 0; i < kOptCount; i++) {
      const char* e = std::getenv(kOptions[i].env);
      g_opt[i].store(e ? std::strtoll(e, nullptr, 10) : kOptions[i].def);
    }
  });
}
int option_index(const char* name) {
  for (int i = 0; i < kOptCount; i++)
    if (std::strcmp(name, kOptions[i].name) == 0) return i;
  return -1;
}
}  // namespace

int64_t option(Option o) {
  options_init();
  return g_opt[o].load(std::memory_order_relaxed);
}

size_t stream_store_max_bytes() {
  const int64_t v = option(kOptStreamStoreMaxBytes);
  return v < 0 ? 0 : size_t(v);
}

int classify_outputs(int count, float* const* outs, const int32_t* sizes) {
  struct Span { uintptr_t b, e; };
  std::vector<Span> v;
  v.reserve(count);
  for (int i = 0; i < count; i++)
    if (sizes[i] > 0 && outs[i]) v.push_back({reinterpret_cast<uintptr_t>(outs[i]), reinterpret_cast<uintptr_t>(outs[i]) + size_t(sizes[i]) * 4});
  std::sort(v.begin(), v.end(), [](const Span& x, const Span& y) { return x.b < y.b || (x.b == y.b && x.e < y.e); });
  int cls = 0;
  uintptr_t cur_b = 0, cur_e = 0;
  for (const Span& s : v) {
    if (s.b < cur_e) {
      if (s.b == cur_b && s.e == cur_e) { cls = cls < 1 ? 1 : cls; continue; }
      return 2;
    }
    cur_b = s.b;
    cur_e = s.e;
  }
  return cls;
}

// ---- range copies ---------------------------------------------------------------
namespace {
constexpr int kCopyThreads = 256;
constexpr int kCopySegs = 224;
constexpr uint32_t kCopyTileBytes = kCopyThreads * 4 * 16;  // 16 KiB per workgroup
struct CopySeg {
  uint8_t* dst;
  const uint8_t* src;
  uint32_t bytes;
  uint32_t pad;
};
struct CopyArgs {
  int32_t nseg;
  int32_t tile_start[kCopySegs + 1];
  CopySeg seg[kCopySegs];
};
static_assert(sizeof(CopyArgs) <= 9600, "kernel-argument budget");

struct __attribute__((packed, aligned(1))) u32x4u {
  uint32_t x, y, z, w;
};

__global__ __launch_bounds__(kCopyThreads) void copy_ranges_kernel(const CopyArgs a) {
  const int tile = blockIdx.x;
  const int s = find_segment<kCopySegs>(a.tile_start, a.nseg, tile);
  const uint8_t* __restrict__ src = a.seg[s].src;
  uint8_t* __restrict__ dst = a.seg[s].dst;
  const uint32_t bytes = a.seg[s].bytes;
  const uint32_t b0 = uint32_t(tile - a.tile_start[s]) * kCopyTileBytes;
  const uint32_t b1 = bytes - b0 < kCopyTileBytes ? bytes : b0 + kCopyTileBytes;
  // 16-byte pieces (no alignment assumed: gfx950 global memory takes unaligned 128-bit accesses)
  u32x4u v[4];
  uint32_t at[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    at[k] = b0 + (k * kCopyThreads + threadIdx.x) * 16u;
    if (at[k] + 16u <= b1) v[k] = *reinterpret_cast<const u32x4u*>(src + at[k]);
  }
#pragma unroll
  for (int k = 0; k < 4; k++)
    if (at[k] + 16u <= b1) *reinterpret_cast<u32x4u*>(dst + at[k]) = v[k];
  // the last, partial piece of the range
  const uint32_t whole = b0 + ((b1 - b0) & ~15u);
  if (threadIdx.x < (b1 - whole)) dst[whole + threadIdx.x] = src[whole + threadIdx.x];
}
}  // namespace

int copy_ranges(int count, uint8_t* const* dst, const uint8_t* const* src, const int64_t* bytes, hipStream_t st) {
  CopyArgs a;
  int i = 0;
  while (i < count) {
    a.nseg = 0;
    a.tile_start[0] = 0;
    while (i < count && a.nseg < kCopySegs) {
      if (bytes[i] <= 0) { i++; continue; }
      if (bytes[i] > int64_t(0xFFFFFFFFu) - kCopyTileBytes || !dst[i] || !src[i]) {
        set_error("copy_ranges: range %d has %lld bytes or a null pointer", i, static_cast<long long>(bytes[i]));
        return HPX_ERR_ARG;
      }
      const int64_t tiles = (bytes[i] + kCopyTileBytes - 1) / kCopyTileBytes;
      if (int64_t(a.tile_start[a.nseg]) + tiles > INT32_MAX) break;
      a.seg[a.nseg] = CopySeg{dst[i], src[i], static_cast<uint32_t>(bytes[i]), 0};
      a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + static_cast<int32_t>(tiles);
      a.nseg++;
      i++;
    }
    if (a.nseg == 0) continue;
    HPX_LAUNCH("copy_ranges_kernel", copy_ranges_kernel, dim3(a.tile_start[a.nseg]), dim3(kCopyThreads), st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

int reject_capture(hipStream_t stream, const char* who) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();  // the query itself is refused for some streams while another one captures: not this call's business
    return HPX_OK;
  }
  if (status == hipStreamCaptureStatusNone) return HPX_OK;
  set_error("%s: the stream is being captured into a graph; this entry point cannot be recorded "
            "(it waits for the stream or tags its kernels per call)", who);
  return HPX_ERR_ARG;
}

uint64_t clock_seed() {
  const int64_t fixed = option(kOptClockSeed);
  if (fixed >= 0) return static_cast<uint64_t>(fixed);
  return static_cast<uint64_t>(
      std::chrono::high_resolution_clock::now().time_since_epoch().count());
}

}  // namespace hpx

HPX_API int hpx_version(void) { return 100; }

HPX_API const char* hpx_last_error(void) { return hpx::g_err; }

HPX_API int hpx_release_workspaces(void) {
  std::lock_guard<std::mutex> g(hpx::g_ws_mu);
  int rc = HPX_OK;
  int cur = 0;
  if (hipGetDevice(&cur) != hipSuccess) cur = -1;
  for (auto& kv : hpx::g_ws) {
    hpx::Workspace* ws = kv.second.get();
    std::lock_guard<std::mutex> g2(ws->mu);
    if (hipSetDevice(ws->device) != hipSuccess) { rc = HPX_ERR_HIP; continue; }
    if (hpx::free_workspace(ws) != HPX_OK) rc = HPX_ERR_HIP;
  }
  hpx::g_ws.clear();
  hpx::g_barrier_owner.clear();
  if (cur >= 0) (void)hipSetDevice(cur);
  return rc;
}

HPX_API int hpx_release_stream(hpx_stream_t stream) {
  hpx::clear_error();
  return hpx::release_stream_workspace(static_cast<hipStream_t>(stream));
}

HPX_API int hpx_set_option(const char* name, int64_t value) {
  hpx::clear_error();
  HPX_ARG(name, "hpx_set_option: null name");
  hpx::options_init();
  const int i = hpx::option_index(name);
  HPX_ARG(i >= 0, "hpx_set_option: unknown option '%s'", name);
  hpx::g_opt[i].store(value);
  return HPX_OK;
}

HPX_API int hpx_get_option(const char* name, int64_t* value) {
  hpx::clear_error();
  HPX_ARG(name && value, "hpx_get_option: null argument");
  hpx::options_init();
  const int i = hpx::option_index(name);
  HPX_ARG(i >= 0, "hpx_get_option: unknown option '%s'", name);
  *value = hpx::g_opt[i].load();
  return HPX_OK;
}

HPX_API int hpx_profile_enable(int on) {
  std::lock_guard<std::mutex> g(hpx::g_prof_mu);
  hpx::g_prof_on = on != 0;
  return HPX_OK;
}

HPX_API int hpx_profile_reset(void) {
  std::lock_guard<std::mutex> g(hpx::g_prof_mu);
  for (auto& r : hpx::g_prof_recs) {
    (void)hipEventSynchronize(r.stop);
    hpx::g_prof_pool.push_back(r.start);
    hpx::g_prof_pool.push_back(r.stop);
  }
  hpx::g_prof_recs.clear();
  return HPX_OK;
}

HPX_API int hpx_profile_query(const char* kernel, double* total_ms, int64_t* launches) {
  hpx::clear_error();
  HPX_ARG(kernel && total_ms && launches, "hpx_profile_query: null argument");
  std::lock_guard<std::mutex> g(hpx::g_prof_mu);
  double sum = 0;
  int64_t n = 0;
  for (auto& r : hpx::g_prof_recs) {
    if (std::strcmp(r.name, kernel) != 0) continue;
    HPX_HIP(hipEventSynchronize(r.stop));
    float ms = 0;
    HPX_HIP(hipEventElapsedTime(&ms, r.start, r.stop));
    sum += ms;
    n++;
  }
  *total_ms = sum;
  *launches = n;
  return HPX_OK;
}
