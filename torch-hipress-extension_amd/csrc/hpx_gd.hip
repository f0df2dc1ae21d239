// GradDrop ("DGC") sparsifier: residual accumulation, sampled threshold,
// order-preserving compaction, optional cut to the k largest, scatter decode.
//
// Semantics follow gd_body.h:102-232 (encode) and :283-353 (decode).  The
// reference makes a pass for R += G, a gather for the sample, a full sort of
// the sample, a two-pass copy_if and waits for the stream three times.  Here:
//
//   sample      |G[i]+R[i]| at the reference's LCG index stream, gathered
//               BEFORE the update (the same fp32 sum the update will store)
//   select      exact k-th largest of the sample by three radix-histogram
//               passes over the fp32 bit pattern (11+11+10 bits); no sort
//   stream      ONE pass over the tensor: r = g + r, store r, compare with the
//               threshold, wave64 ballot -> one 64-bit word per 64 elements
//               (bit i = element i) and a popcount per workgroup
//   scan        two-level exclusive prefix of the per-workgroup counts
//   expand      bit words -> ascending indices at the scanned offsets, values
//               out, residual entries zeroed, header written
//
// The stream pass moves 12 bytes per element (g, r in; r out) plus 1/8 byte of
// mask; everything else touches O(sample + selected) data.  The host waits for
// the stream once, after the common case (no cut) has been queued in full, to
// learn whether the cut to `expected` entries is needed; that path orders the
// candidates by |r| with a stable LSD radix sort (ties keep ascending index).
#include <cmath>

#include "hpx_common.h"

namespace {
using namespace hpx;

constexpr int kThreads = 256;
constexpr int kPerLane = 16;
constexpr int kTile = kThreads * kPerLane;       // 4096 elements per workgroup
constexpr int kWaveTile = kWave * kPerLane;      // 1024 elements per wave
constexpr int kSelThreads = 1024;
constexpr int kSelBlocksMax = 128;               // few blocks: their bins meet in global atomics
constexpr int kBins1 = 2048, kBins2 = 2048, kBins3 = 1024;  // key = d1:11 | d2:11 | d3:10

struct GdState {
  uint32_t total;     // candidates found by the stream pass
  uint32_t thr_bits;  // threshold as fp32 bits
  uint32_t arrive;    // arrival counter of the scan kernel's workgroups
  uint32_t pad[61];
};
constexpr int kScanChunk = 4096;   // per-tile counts scanned by one workgroup
constexpr int kMaxChunks = 128;    // 2^31 elements / kTile / kScanChunk

struct SelArgs {
  const float* g;
  const float* r;
  uint32_t n;
  uint32_t sample_cnt;
  uint32_t seed;        // low 32 bits of the 64-bit seed
  uint32_t thr_index;   // rank (descending, 0-based) of the threshold in the sample
  uint32_t* samples;    // |g+r| bit patterns
  uint32_t* hist;       // kBins1 + kBins2 + kBins3 counters, zero on entry
  GdState* st;
};

// Rank search in a descending cumulative histogram: returns the bin holding
// rank `rank_in` (0-based from the top) and the rank left inside that bin.
template <int BINS>
__device__ __forceinline__ void find_digit(const uint32_t* __restrict__ hist, uint32_t rank_in,
                                           uint32_t& digit, uint32_t& rank_out) {
  constexpr int PER = BINS / kSelThreads;
  static_assert(PER >= 1, "one bin per thread at least");
  __shared__ uint32_t s_scan[kSelThreads];
  __shared__ uint32_t s_res[2];
  const int t = threadIdx.x;
  uint32_t h[PER], sum = 0;
#pragma unroll
  for (int j = 0; j < PER; j++) {
    h[j] = hist[BINS - 1 - (t * PER + j)];
    sum += h[j];
  }
  if (t == 0) { s_res[0] = 0; s_res[1] = 0; }
  s_scan[t] = sum;
  __syncthreads();
  for (int off = 1; off < kSelThreads; off <<= 1) {
    const uint32_t v = t >= off ? s_scan[t - off] : 0u;
    __syncthreads();
    s_scan[t] += v;
    __syncthreads();
  }
  const uint32_t excl = s_scan[t] - sum;
  if (rank_in >= excl && rank_in - excl < sum) {
    uint32_t c = excl;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      if (rank_in >= c && rank_in - c < h[j]) {
        s_res[0] = uint32_t(BINS - 1 - (t * PER + j));
        s_res[1] = rank_in - c;
      }
      c += h[j];
    }
  }
  __syncthreads();
  digit = s_res[0];
  rank_out = s_res[1];
  __syncthreads();
}

// generate_sample_G, gd_body.h:36-41: naive_int_random<uint32_t>(0, N-1) seeded
// with (uint32)(t + x), one discarded draw, then rand() % N.
__device__ __forceinline__ uint32_t sample_index(uint32_t seed, uint32_t x, uint32_t n) {
  return (lcg_mul(2) * (seed + x) + lcg_add(2)) % n;
}

// One sample per lane: all the random gathers of the sample are in flight at
// once.  The same launch clears the histograms and the counters of this call.
__global__ __launch_bounds__(kThreads) void gd_sample_kernel(const SelArgs a) {
  const uint32_t x = blockIdx.x * kThreads + threadIdx.x;
  if (x < uint32_t(kBins1 + kBins2 + kBins3)) a.hist[x] = 0;
  if (x == 0) {
    a.st->total = 0;
    a.st->arrive = 0;
  }
  if (x < a.sample_cnt) {
    const uint32_t i = sample_index(a.seed, x, a.n);
    a.samples[x] = __float_as_uint(__builtin_fabsf(a.g[i] + a.r[i]));
  }
}

template <int PASS>
__device__ __forceinline__ void hist_accumulate(const SelArgs& a, uint32_t* s_hist, uint32_t prefix) {
  // PASS 1: all keys, digit = key >> 21.  PASS 2: keys with key>>21 == prefix,
  // digit = (key >> 10) & 2047.  PASS 3: keys with key>>10 == prefix, digit = key & 1023.
  const uint32_t stride = gridDim.x * kSelThreads;
  for (uint32_t x = blockIdx.x * kSelThreads + threadIdx.x; x < a.sample_cnt; x += stride) {
    const uint32_t key = a.samples[x];
    if (PASS == 1) {
      atomicAdd(&s_hist[key >> 21], 1u);
    } else if (PASS == 2) {
      if ((key >> 21) == prefix) atomicAdd(&s_hist[(key >> 10) & 2047u], 1u);
    } else {
      if ((key >> 10) == prefix) atomicAdd(&s_hist[key & 1023u], 1u);
    }
  }
}

template <int PASS>
__global__ __launch_bounds__(kSelThreads) void gd_select_kernel(const SelArgs a) {
  constexpr int BINS = PASS == 1 ? kBins1 : PASS == 2 ? kBins2 : kBins3;
  __shared__ uint32_t s_hist[BINS];
  for (int i = threadIdx.x; i < BINS; i += kSelThreads) s_hist[i] = 0;
  uint32_t prefix = 0;
  if (PASS >= 2) {
    uint32_t d1, rank;
    find_digit<kBins1>(a.hist, a.thr_index, d1, rank);
    prefix = d1;
    if (PASS == 3) {
      uint32_t d2;
      find_digit<kBins2>(a.hist + kBins1, rank, d2, rank);
      prefix = (d1 << 11) | d2;
    }
  }
  __syncthreads();
  hist_accumulate<PASS>(a, s_hist, prefix);
  __syncthreads();
  uint32_t* gh = a.hist + (PASS == 1 ? 0 : PASS == 2 ? kBins1 : kBins1 + kBins2);
  for (int i = threadIdx.x; i < BINS; i += kSelThreads) {
    const uint32_t c = s_hist[i];
    if (c) atomicAdd(&gh[i], c);
  }
}

__global__ __launch_bounds__(kSelThreads) void gd_threshold_kernel(const SelArgs a) {
  uint32_t d1, d2, d3, rank;
  find_digit<kBins1>(a.hist, a.thr_index, d1, rank);
  find_digit<kBins2>(a.hist + kBins1, rank, d2, rank);
  find_digit<kBins3>(a.hist + kBins1 + kBins2, rank, d3, rank);
  if (threadIdx.x == 0) a.st->thr_bits = (d1 << 21) | (d2 << 10) | d3;
}

// The one pass over the tensor.  Lane l of wave w handles elements
// base + w*1024 + c*64 + l for c = 0..15, so ballot number c is the mask word of
// 64 consecutive elements in natural bit order.
__global__ __launch_bounds__(kThreads) void gd_stream_kernel(const float* __restrict__ g, float* __restrict__ r,
                                                             uint32_t n, const GdState* __restrict__ st,
                                                             uint64_t* __restrict__ masks,
                                                             uint32_t* __restrict__ blk_counts) {
  const float thr = __uint_as_float(st->thr_bits);
  const float nthr = -thr;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t base = blockIdx.x * uint32_t(kTile);
  const uint32_t wbase = base + wave * uint32_t(kWaveTile);
  uint32_t lo = 0, hi = 0, cnt = 0;
  if (n - base >= uint32_t(kTile)) {
    float gv[kPerLane], rv[kPerLane];
#pragma unroll
    for (int c = 0; c < kPerLane; c++) {
      gv[c] = __builtin_nontemporal_load(g + size_t(wbase) + c * kWave + lane);
      rv[c] = __builtin_nontemporal_load(r + size_t(wbase) + c * kWave + lane);
    }
#pragma unroll
    for (int c = 0; c < kPerLane; c++) {
      const float x = gv[c] + rv[c];  // thrust::plus<float>()(G, R), gd_body.h:121-128
      __builtin_nontemporal_store(x, r + size_t(wbase) + c * kWave + lane);
      const uint64_t m = __ballot((x > thr) || (x < nthr));  // gd_body.h:59-67
      cnt += __popcll(m);
      lo = lane == uint32_t(c) ? uint32_t(m) : lo;  // lane c keeps mask word c
      hi = lane == uint32_t(c) ? uint32_t(m >> 32) : hi;
    }
  } else {
#pragma unroll
    for (int c = 0; c < kPerLane; c++) {
      const uint32_t e = wbase + c * kWave + lane;
      bool p = false;
      if (e < n) {
        const float x = g[e] + r[e];
        r[e] = x;
        p = (x > thr) || (x < nthr);
      }
      const uint64_t m = __ballot(p);
      cnt += __popcll(m);
      lo = lane == uint32_t(c) ? uint32_t(m) : lo;  // lane c keeps mask word c
      hi = lane == uint32_t(c) ? uint32_t(m >> 32) : hi;
    }
  }
  if (lane < kPerLane) masks[(size_t(wbase) >> 6) + lane] = (uint64_t(hi) << 32) | lo;
  __shared__ uint32_t s_cnt[kThreads / kWave];
  if (lane == 0) s_cnt[wave] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) blk_counts[blockIdx.x] = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
}

// Exclusive prefix of the per-tile counts, two levels.  Workgroup c scans counts
// [c*4096, (c+1)*4096) into `off` (relative to its chunk) and publishes the chunk
// total; the last workgroup to arrive (at most 128 of them, so the shared
// counter costs microseconds at worst) turns the totals into chunk offsets and
// the grand total.
__global__ __launch_bounds__(kSelThreads) void gd_scan_kernel(const uint32_t* __restrict__ cnt, uint32_t* __restrict__ off,
                                                              uint32_t n, uint32_t* __restrict__ chunk_tot,
                                                              uint32_t* __restrict__ chunk_off, GdState* __restrict__ st,
                                                              uint32_t* __restrict__ host_total) {
  __shared__ uint32_t s_wave[kSelThreads / kWave];
  __shared__ uint32_t s_last;
  const uint32_t t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  const uint32_t i0 = blockIdx.x * uint32_t(kScanChunk) + t * 4;
  uint32_t c[4];
#pragma unroll
  for (int j = 0; j < 4; j++) c[j] = (i0 + j < n) ? cnt[i0 + j] : 0u;
  const uint32_t sum = c[0] + c[1] + c[2] + c[3];
  uint32_t incl = sum;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t v = __shfl_up(incl, o, kWave);
    if (lane >= uint32_t(o)) incl += v;
  }
  if (lane == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (uint32_t w = 0; w < kSelThreads / kWave; w++) {
    const uint32_t v = s_wave[w];
    if (w < wave) before += v;
    all += v;
  }
  uint32_t run = before + incl - sum;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if (i0 + j < n) off[i0 + j] = run;
    run += c[j];
  }
  if (t == 0) {
    chunk_tot[blockIdx.x] = all;
    __threadfence();
    s_last = (atomicAdd(&st->arrive, 1u) == gridDim.x - 1);
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  if (t < kWave) {
    // up to 128 chunk totals: two per lane
    const uint32_t a0 = (2 * t < gridDim.x) ? __hip_atomic_load(&chunk_tot[2 * t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    const uint32_t a1 = (2 * t + 1 < gridDim.x) ? __hip_atomic_load(&chunk_tot[2 * t + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    uint32_t inc2 = a0 + a1;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const uint32_t v = __shfl_up(inc2, o, kWave);
      if (t >= uint32_t(o)) inc2 += v;
    }
    const uint32_t ex = inc2 - a0 - a1;
    if (2 * t < gridDim.x) chunk_off[2 * t] = ex;
    if (2 * t + 1 < gridDim.x) chunk_off[2 * t + 1] = ex + a0;
    if (t == kWave - 1) {
      st->total = inc2;
      // pinned host word: the host reads it after its one wait on the stream, no copy command needed
      __hip_atomic_store(host_total, inc2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

// One wave per stream tile: 64 mask words -> ascending indices at the scanned
// offsets.  With `out` set this is the common-case finish (gd_body.h:193-229):
// nothing happens if the stream pass found more than `limit` candidates,
// otherwise indices, values and header are written and the residual entries are
// cleared.  With `out` null the indices go to `dst` (the candidate list of the
// cut path) and nothing else is touched.
__global__ __launch_bounds__(kThreads) void gd_expand_kernel(const uint64_t* __restrict__ masks,
                                                             const uint32_t* __restrict__ tile_off,
                                                             const uint32_t* __restrict__ chunk_off, uint32_t ntiles,
                                                             const GdState* __restrict__ st, int32_t* __restrict__ dst,
                                                             uint32_t limit, uint8_t* __restrict__ out,
                                                             float* __restrict__ r) {
  const uint32_t total = st->total;
  if (out && total > limit) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t tile = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (out && tile == 0 && lane == 0) *reinterpret_cast<int32_t*>(out) = int32_t(4 + total * 8);
  if (tile >= ntiles) return;
  uint64_t m = masks[size_t(tile) * kWave + lane];
  const uint32_t c = __popcll(m);
  uint32_t incl = c;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t v = __shfl_up(incl, o, kWave);
    if (lane >= uint32_t(o)) incl += v;
  }
  uint32_t pos = chunk_off[tile / kScanChunk] + tile_off[tile] + incl - c;
  const uint32_t e0 = tile * uint32_t(kTile) + lane * kWave;
  int32_t* idx = out ? reinterpret_cast<int32_t*>(out + 4) : dst;
  float* val = out ? reinterpret_cast<float*>(out + 4 + size_t(total) * 4) : nullptr;
  while (m) {
    const uint32_t e = e0 + uint32_t(__builtin_ctzll(m));
    m &= m - 1;
    if (pos < limit) {
      idx[pos] = int32_t(e);
      if (out) {
        val[pos] = r[e];
        r[e] = 0.0f;
      }
    }
    pos++;
  }
}

// generate_S_value, gd_body.h:80-99, plus the header (gd_body.h:193-201), for a
// list of k indices already in place (the cut path).
__global__ __launch_bounds__(kThreads) void gd_gather_kernel(uint8_t* __restrict__ out, float* __restrict__ r, uint32_t k) {
  const int32_t* idx = reinterpret_cast<const int32_t*>(out + 4);
  float* val = reinterpret_cast<float*>(out + 4 + size_t(k) * 4);
  const uint32_t x = blockIdx.x * kThreads + threadIdx.x;
  if (x == 0) *reinterpret_cast<int32_t*>(out) = int32_t(4 + k * 8);
  if (x < k) {
    const int32_t i = idx[x];
    val[x] = r[i];
    r[i] = 0.0f;
  }
}

// ---- cut to the `expected` largest |r| (gd_body.h:176-187) ------------------
constexpr int kSortPer = 8;
constexpr int kSortTile = kThreads * kSortPer;  // 2048 pairs per workgroup

__global__ __launch_bounds__(kThreads) void gd_keys_kernel(const int32_t* __restrict__ cand, const float* __restrict__ r,
                                                           uint32_t n, uint32_t* __restrict__ keys) {
  const uint32_t x = blockIdx.x * kThreads + threadIdx.x;
  if (x < n) keys[x] = __float_as_uint(__builtin_fabsf(r[cand[x]]));
}

// Descending order: bin = 255 - byte.  counts is bin-major: counts[bin * nblk + blk].
__global__ __launch_bounds__(kThreads) void gd_sort_count_kernel(const uint32_t* __restrict__ keys, uint32_t n, int shift,
                                                                 uint32_t* __restrict__ counts, uint32_t nblk) {
  __shared__ uint32_t s_hist[256];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const uint32_t b0 = blockIdx.x * uint32_t(kSortTile);
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const uint32_t x = b0 + j * kThreads + threadIdx.x;
    if (x < n) atomicAdd(&s_hist[255u - ((keys[x] >> shift) & 255u)], 1u);
  }
  __syncthreads();
  counts[size_t(threadIdx.x) * nblk + blockIdx.x] = s_hist[threadIdx.x];
}

// Stable scatter of one 8-bit digit.  Elements are taken round by round
// (round j holds x = b0 + j*256 + t), waves in order inside a round, lanes in
// order inside a wave, so equal digits keep their input order.
__global__ __launch_bounds__(kThreads) void gd_sort_scatter_kernel(const uint32_t* __restrict__ keys_in,
                                                                   const int32_t* __restrict__ idx_in, uint32_t n,
                                                                   int shift, const uint32_t* __restrict__ counts,
                                                                   uint32_t nblk, uint32_t* __restrict__ keys_out,
                                                                   int32_t* __restrict__ idx_out) {
  __shared__ uint32_t s_run[256];   // next output slot per bin for this workgroup
  __shared__ uint32_t s_scan[256];
  const uint32_t t = threadIdx.x;
  {
    // bin t: total over all workgroups and the part that precedes this one
    uint32_t total = 0, before = 0;
    const uint32_t* row = counts + size_t(t) * nblk;
    for (uint32_t b = 0; b < nblk; b++) {
      const uint32_t c = row[b];
      total += c;
      if (b < blockIdx.x) before += c;
    }
    s_scan[t] = total;
    __syncthreads();
    for (int o = 1; o < 256; o <<= 1) {
      const uint32_t v = t >= uint32_t(o) ? s_scan[t - o] : 0u;
      __syncthreads();
      s_scan[t] += v;
      __syncthreads();
    }
    s_run[t] = s_scan[t] - total + before;
    __syncthreads();
  }
  const uint32_t lane = t & (kWave - 1), wave = t / kWave;
  const uint32_t b0 = blockIdx.x * uint32_t(kSortTile);
  for (int j = 0; j < kSortPer; j++) {
    const uint32_t x = b0 + j * kThreads + t;
    const bool live = x < n;
    uint32_t key = 0, bin = 0;
    int32_t id = 0;
    if (live) {
      key = keys_in[x];
      id = idx_in[x];
      bin = 255u - ((key >> shift) & 255u);
    }
    // lanes of this wave holding the same bin
    uint64_t same = __ballot(live);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const uint64_t m = __ballot((bin >> b) & 1u);
      same &= ((bin >> b) & 1u) ? m : ~m;
    }
    const uint32_t rank = __popcll(same & ((uint64_t(1) << lane) - 1));
    const uint32_t cnt = __popcll(same);
    uint32_t slot = 0;
    for (uint32_t w = 0; w < kThreads / kWave; w++) {
      if (wave == w && live && rank == 0) {
        slot = s_run[bin];
        s_run[bin] = slot + cnt;
      }
      __syncthreads();
    }
    // the first lane of each group read the base; hand it to the others
    const int leader = live ? __builtin_ctzll(same) : int(lane);
    slot = __shfl(slot, leader, kWave);
    if (live) {
      keys_out[slot + rank] = key;
      idx_out[slot + rank] = id;
    }
  }
}

__global__ __launch_bounds__(kThreads) void gd_copy_idx_kernel(const int32_t* __restrict__ src, int32_t* __restrict__ dst,
                                                               uint32_t n) {
  const uint32_t x = blockIdx.x * kThreads + threadIdx.x;
  if (x < n) dst[x] = src[x];
}

// ---- decode -----------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void gd_zero_kernel(float* __restrict__ out, uint32_t n) {
  const uint32_t stride = gridDim.x * kThreads * 4;
  for (uint32_t e = (blockIdx.x * kThreads + threadIdx.x) * 4; e < n; e += stride) {
    if (n - e >= 4) {
      st4(out + e, make_float4(0.f, 0.f, 0.f, 0.f));
    } else {
      for (uint32_t i = e; i < n; i++) out[i] = 0.f;
    }
  }
}

template <bool ADD>
__global__ __launch_bounds__(kThreads) void gd_scatter_kernel(const int32_t* __restrict__ idx, const float* __restrict__ val,
                                                              uint32_t k, float* __restrict__ out) {
  const uint32_t x = blockIdx.x * kThreads + threadIdx.x;
  if (x < k) {
    const int32_t i = idx[x];
    if (ADD) out[i] += val[x]; else out[i] = val[x];  // gd_body.h:250, :280
  }
}

inline uint32_t cdiv(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }
inline size_t align256(size_t x) { return (x + 255) & ~size_t(255); }

// Sorts (keys, idx) by key descending, stable, `n` pairs; result left in
// (keys_a, idx_a).  counts holds 256 * nblk words.
int sort_pairs_desc(uint32_t* keys_a, int32_t* idx_a, uint32_t* keys_b, int32_t* idx_b, uint32_t* counts, uint32_t n,
                    hipStream_t st) {
  const uint32_t nblk = cdiv(n, kSortTile);
  for (int pass = 0; pass < 4; pass++) {
    const int shift = pass * 8;
    HPX_LAUNCH("gd_sort_count_kernel", gd_sort_count_kernel, dim3(nblk), dim3(kThreads), st, keys_a, n, shift, counts, nblk);
    HPX_LAUNCH("gd_sort_scatter_kernel", gd_sort_scatter_kernel, dim3(nblk), dim3(kThreads), st, keys_a, idx_a, n, shift, counts, nblk,
                       keys_b, idx_b);
    HPX_HIP(hipGetLastError());
    std::swap(keys_a, keys_b);
    std::swap(idx_a, idx_b);
  }
  return HPX_OK;  // four passes: data is back in the caller's (keys_a, idx_a)
}

int gd_encode_one(const float* g, int32_t N, float* r, uint8_t* out, double sample_rate, double drop_ratio,
                  uint64_t seed, hpx::Workspace* ws, hipStream_t st) {
  // size arithmetic of gd_body.h:112-115, :153
  const double s_percent = 1 - drop_ratio;
  const int32_t sample_cnt = static_cast<int32_t>(std::ceil(N * sample_rate));
  const int32_t expected = static_cast<int32_t>(std::ceil(N * s_percent));
  const int32_t thr_index = static_cast<int32_t>(sample_cnt * s_percent);
  HPX_ARG(sample_cnt > 0 && thr_index >= 0 && thr_index < sample_cnt && expected >= 0,
          "hpx_gd_encode: N=%d sample_rate=%g drop_ratio=%g give sample_cnt=%d threshold index=%d", N, sample_rate,
          drop_ratio, sample_cnt, thr_index);

  const uint32_t n = static_cast<uint32_t>(N);
  const uint32_t ntiles = cdiv(n, kTile);
  // workspace layout
  size_t off = 0;
  const size_t o_state = off; off += align256(sizeof(GdState));
  const size_t o_hist = off;  off += align256(sizeof(uint32_t) * (kBins1 + kBins2 + kBins3));
  const size_t o_samples = off; off += align256(sizeof(uint32_t) * size_t(sample_cnt));
  const size_t o_masks = off; off += align256(sizeof(uint64_t) * size_t(ntiles) * kWave);
  const size_t o_cnt = off; off += align256(sizeof(uint32_t) * size_t(ntiles));
  const size_t o_off = off; off += align256(sizeof(uint32_t) * size_t(ntiles));
  const size_t o_ctot = off; off += align256(sizeof(uint32_t) * kMaxChunks);
  const size_t o_coff = off; off += align256(sizeof(uint32_t) * kMaxChunks);
  // Room for the cut path (sorted copies of the candidates) is reserved for a
  // typical overshoot so that path normally needs no reallocation.
  uint64_t cap = uint64_t(expected) * 2 > uint64_t(expected) + 65536 ? uint64_t(expected) * 2 : uint64_t(expected) + 65536;
  if (cap > n) cap = n;
  auto cut_bytes = [](uint64_t total) {
    return 4 * align256(sizeof(uint32_t) * size_t(total)) + align256(sizeof(uint32_t) * 256 * size_t(cdiv(total, kSortTile)));
  };
  int rc = hpx::ensure_workspace(ws, off + cut_bytes(cap));
  if (rc != HPX_OK) return rc;
  uint8_t* base = ws->dev;
  GdState* state = reinterpret_cast<GdState*>(base + o_state);
  uint32_t* hist = reinterpret_cast<uint32_t*>(base + o_hist);
  uint32_t* samples = reinterpret_cast<uint32_t*>(base + o_samples);
  uint64_t* masks = reinterpret_cast<uint64_t*>(base + o_masks);
  uint32_t* blk_cnt = reinterpret_cast<uint32_t*>(base + o_cnt);
  uint32_t* blk_off = reinterpret_cast<uint32_t*>(base + o_off);
  uint32_t* chunk_tot = reinterpret_cast<uint32_t*>(base + o_ctot);
  uint32_t* chunk_off = reinterpret_cast<uint32_t*>(base + o_coff);
  const uint32_t nchunks = cdiv(ntiles, kScanChunk);

  SelArgs sa{g, r, n, static_cast<uint32_t>(sample_cnt), static_cast<uint32_t>(seed), static_cast<uint32_t>(thr_index),
             samples, hist, state};
  uint32_t sel_blocks = cdiv(sample_cnt, kSelThreads * 8);
  if (sel_blocks > kSelBlocksMax) sel_blocks = kSelBlocksMax;
  const uint32_t zero_words = kBins1 + kBins2 + kBins3;
  HPX_LAUNCH("gd_sample_kernel", gd_sample_kernel,
             dim3(cdiv(uint32_t(sample_cnt) > zero_words ? uint32_t(sample_cnt) : zero_words, kThreads)), dim3(kThreads), st, sa);
  HPX_LAUNCH("gd_select_kernel", gd_select_kernel<1>, dim3(sel_blocks), dim3(kSelThreads), st, sa);
  HPX_LAUNCH("gd_select_kernel", gd_select_kernel<2>, dim3(sel_blocks), dim3(kSelThreads), st, sa);
  HPX_LAUNCH("gd_select_kernel", gd_select_kernel<3>, dim3(sel_blocks), dim3(kSelThreads), st, sa);
  HPX_LAUNCH("gd_threshold_kernel", gd_threshold_kernel, dim3(1), dim3(kSelThreads), st, sa);
  HPX_LAUNCH("gd_stream_kernel", gd_stream_kernel, dim3(ntiles), dim3(kThreads), st, g, r, n, state, masks, blk_cnt);
  uint32_t* h_total = reinterpret_cast<uint32_t*>(ws->pinned);
  HPX_LAUNCH("gd_scan_kernel", gd_scan_kernel, dim3(nchunks), dim3(kSelThreads), st, blk_cnt, blk_off, ntiles, chunk_tot,
             chunk_off, state, h_total);
  HPX_HIP(hipGetLastError());
  // Common case (nothing to cut) queued before the host knows the count.
  int32_t* out_idx = reinterpret_cast<int32_t*>(out + 4);
  const uint32_t lim = static_cast<uint32_t>(expected);
  HPX_LAUNCH("gd_expand_kernel", gd_expand_kernel, dim3(cdiv(ntiles, kThreads / kWave)), dim3(kThreads), st, masks, blk_off,
             chunk_off, ntiles, state, out_idx, lim, out, r);
  HPX_HIP(hipGetLastError());
  HPX_HIP(hipStreamSynchronize(st));
  const uint32_t total = *reinterpret_cast<volatile uint32_t*>(h_total);
  if (total <= lim) return HPX_OK;

  // More candidates than `expected`: order them by |r| descending and keep the first `expected`.
  const uint32_t sblk = cdiv(total, kSortTile);
  size_t off2 = off;
  const size_t o_ka = off2; off2 += align256(sizeof(uint32_t) * size_t(total));
  const size_t o_kb = off2; off2 += align256(sizeof(uint32_t) * size_t(total));
  const size_t o_ia = off2; off2 += align256(sizeof(int32_t) * size_t(total));
  const size_t o_ib = off2; off2 += align256(sizeof(int32_t) * size_t(total));
  const size_t o_sc = off2; off2 += align256(sizeof(uint32_t) * 256 * size_t(sblk));
  if (off2 > ws->dev_bytes) {
    // Far more candidates than reserved for.  Growing would discard the masks;
    // build the larger block and carry them over.
    uint8_t* old = ws->dev;
    const size_t old_bytes = ws->dev_bytes;
    ws->dev = nullptr;
    ws->dev_bytes = 0;
    rc = hpx::ensure_workspace(ws, off2);
    if (rc != HPX_OK) { (void)hipFree(old); return rc; }
    HPX_HIP(hipMemcpyAsync(ws->dev, old, off < old_bytes ? off : old_bytes, hipMemcpyDeviceToDevice, st));
    HPX_HIP(hipStreamSynchronize(st));
    HPX_HIP(hipFree(old));
    base = ws->dev;
    state = reinterpret_cast<GdState*>(base + o_state);
    masks = reinterpret_cast<uint64_t*>(base + o_masks);
    blk_off = reinterpret_cast<uint32_t*>(base + o_off);
    chunk_off = reinterpret_cast<uint32_t*>(base + o_coff);
  }
  uint32_t* ka = reinterpret_cast<uint32_t*>(base + o_ka);
  uint32_t* kb = reinterpret_cast<uint32_t*>(base + o_kb);
  int32_t* ia = reinterpret_cast<int32_t*>(base + o_ia);
  int32_t* ib = reinterpret_cast<int32_t*>(base + o_ib);
  uint32_t* sc = reinterpret_cast<uint32_t*>(base + o_sc);
  HPX_LAUNCH("gd_expand_kernel", gd_expand_kernel, dim3(cdiv(ntiles, kThreads / kWave)), dim3(kThreads), st, masks, blk_off,
             chunk_off, ntiles, state, ia, total, static_cast<uint8_t*>(nullptr), static_cast<float*>(nullptr));
  HPX_LAUNCH("gd_keys_kernel", gd_keys_kernel, dim3(cdiv(total, kThreads)), dim3(kThreads), st, ia, r, total, ka);
  HPX_HIP(hipGetLastError());
  rc = sort_pairs_desc(ka, ia, kb, ib, sc, total, st);
  if (rc != HPX_OK) return rc;
  if (lim > 0) HPX_LAUNCH("gd_copy_idx_kernel", gd_copy_idx_kernel, dim3(cdiv(lim, kThreads)), dim3(kThreads), st, ia, out_idx, lim);
  HPX_LAUNCH("gd_gather_kernel", gd_gather_kernel, dim3(cdiv(lim > 0 ? lim : 1, kThreads)), dim3(kThreads), st, out, r, lim);
  HPX_HIP(hipGetLastError());
  return HPX_OK;
}

}  // namespace

HPX_API int hpx_gd_encode(int count, const float* const* grads, const int32_t* Ns, float* const* residuals,
                          uint8_t* const* outs, const double* sample_rates, const double* drop_ratios,
                          const uint64_t* seeds, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_gd_encode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(grads && Ns && residuals && outs && sample_rates && drop_ratios, "hpx_gd_encode: null argument array");
  for (int i = 0; i < count; i++) {
    HPX_ARG(Ns[i] > 0, "hpx_gd_encode: tensor %d has size %d (must be positive)", i, Ns[i]);
    HPX_ARG(grads[i] && residuals[i] && outs[i], "hpx_gd_encode: tensor %d has a null pointer", i);
    HPX_ARG((reinterpret_cast<uintptr_t>(outs[i]) & 3) == 0, "hpx_gd_encode: output %d is not 4-byte aligned", i);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int worst = HPX_OK;
  for (int i = 0; i < count; i++) {
    const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
    const int rc = gd_encode_one(grads[i], Ns[i], residuals[i], outs[i], sample_rates[i], drop_ratios[i], seed, ws, st);
    if (rc != HPX_OK && worst == HPX_OK) worst = rc;  // like the reference driver: report, go on
  }
  return worst;
}

HPX_API int hpx_gd_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes, float* const* outs,
                          const int32_t* out_sizes, const int32_t* is_add_tos, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_gd_decode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(ins && in_sizes && outs && out_sizes && is_add_tos, "hpx_gd_decode: null argument array");
  HPX_ARG(size_t(count) * sizeof(int32_t) <= hpx::kPinnedBytes, "hpx_gd_decode: more than %zu messages in one call",
          hpx::kPinnedBytes / sizeof(int32_t));
  for (int i = 0; i < count; i++) {
    HPX_ARG(ins[i] && outs[i] && out_sizes[i] >= 0, "hpx_gd_decode: message %d has a null pointer or negative size", i);
    HPX_ARG((reinterpret_cast<uintptr_t>(ins[i]) & 3) == 0, "hpx_gd_decode: message %d is not 4-byte aligned", i);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int rc = hpx::ensure_workspace(ws, 0);
  if (rc != HPX_OK) return rc;
  // headers first, one wait (gd_body.h:301-309)
  int32_t* Ms = reinterpret_cast<int32_t*>(ws->pinned);
  for (int i = 0; i < count; i++) HPX_HIP(hipMemcpyAsync(&Ms[i], ins[i], sizeof(int32_t), hipMemcpyDeviceToHost, st));
  HPX_HIP(hipStreamSynchronize(st));
  for (int i = 0; i < count; i++) {
    if (in_sizes[i] < Ms[i]) {  // gd_body.h:317-325
      hpx::set_error("input space provided is not enough! in_uint8_t_size=%d\tM=%d (message %d, is_add_to %d)", in_sizes[i],
                     Ms[i], i, is_add_tos[i]);
      return HPX_ERR_BODY;
    }
    HPX_ARG(Ms[i] >= 4, "hpx_gd_decode: message %d has header %d", i, Ms[i]);
  }
  for (int i = 0; i < count; i++) {
    const uint32_t k = static_cast<uint32_t>((Ms[i] - 4) / 8);
    const int32_t* idx = reinterpret_cast<const int32_t*>(ins[i] + 4);
    const float* val = reinterpret_cast<const float*>(ins[i] + 4 + size_t(k) * 4);
    if (!is_add_tos[i]) {
      const uint32_t n = static_cast<uint32_t>(out_sizes[i]);
      if (n) {
        uint32_t blocks = cdiv(n, kThreads * 4);
        HPX_LAUNCH("gd_zero_kernel", gd_zero_kernel, dim3(blocks), dim3(kThreads), st, outs[i], n);
      }
      if (k) HPX_LAUNCH("gd_scatter_kernel", gd_scatter_kernel<false>, dim3(cdiv(k, kThreads)), dim3(kThreads), st, idx, val, k, outs[i]);
    } else if (k) {
      HPX_LAUNCH("gd_scatter_kernel", gd_scatter_kernel<true>, dim3(cdiv(k, kThreads)), dim3(kThreads), st, idx, val, k, outs[i]);
    }
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}
