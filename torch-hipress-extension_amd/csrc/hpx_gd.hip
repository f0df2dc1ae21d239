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
// learn whether the cut to `expected` entries is needed.  The expand launch has
// by then left the candidates, their keys and the first digit's counts where
// the cut path wants them, so that path is four more launches: a stable LSD radix
// sort by |r| (ties keep ascending index) whose last pass writes the message.
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
    // with a residual: |G[i] + R[i]|, the value the update is about to store; without (dgc_body.h:18-30): |G[i]|
    a.samples[x] = __float_as_uint(__builtin_fabsf(a.r ? a.g[i] + a.r[i] : a.g[i]));
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
// RESIDUAL = false is the sparsifier without residual (dgc_body.h:110-117): the
// values are G itself, nothing is added and nothing is stored (4 bytes per element).
template <bool RESIDUAL>
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
      rv[c] = RESIDUAL ? __builtin_nontemporal_load(r + size_t(wbase) + c * kWave + lane) : 0.0f;
    }
#pragma unroll
    for (int c = 0; c < kPerLane; c++) {
      const float x = RESIDUAL ? gv[c] + rv[c] : gv[c];  // thrust::plus<float>()(G, R), gd_body.h:121-128
      if (RESIDUAL) __builtin_nontemporal_store(x, r + size_t(wbase) + c * kWave + lane);
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
        const float x = RESIDUAL ? g[e] + r[e] : g[e];
        if (RESIDUAL) r[e] = x;
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

// Shape of the cut path's radix sort (further down): tiles of 8192 pairs.
constexpr int kSortThreads = 1024;
constexpr int kSortPer = 8;
constexpr int kSortTile = kSortThreads * kSortPer;
constexpr int kSortWaves = kSortThreads / kWave;

// Turns the per-tile bit masks into the ascending index list, one wave per tile,
// at the offsets the scan produced.  If the stream pass found at most `limit`
// candidates this is the finish (gd_body.h:193-229): indices, values and header
// are written and the residual entries cleared.  If it found more, the candidates
// and their keys (bits of |r|) go to `cand` / `keys` for the cut path instead and
// nothing else is touched; more than `cap` candidates do not fit those buffers
// and the kernel does nothing (the host then calls it again with larger ones and
// limit = 0).
__global__ __launch_bounds__(kThreads) void gd_expand_kernel(const uint64_t* __restrict__ masks,
                                                             const uint32_t* __restrict__ tile_off,
                                                             const uint32_t* __restrict__ chunk_off, uint32_t ntiles,
                                                             const GdState* __restrict__ st, uint32_t limit,
                                                             uint8_t* __restrict__ out, float* __restrict__ r,
                                                             int32_t* __restrict__ cand, uint32_t* __restrict__ keys,
                                                             uint32_t cap) {
  const uint32_t total = st->total;
  const bool cut = total > limit;
  if (cut && total > cap) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t tile = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave;
  if (!cut && tile == 0 && lane == 0) *reinterpret_cast<int32_t*>(out) = int32_t(4 + total * 8);
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
  if (cut) {
    const uint32_t thr_bits = st->thr_bits;
    while (m) {
      const uint32_t e = e0 + uint32_t(__builtin_ctzll(m));
      m &= m - 1;
      cand[pos] = int32_t(e);
      // Sort key: distance of |r| above the threshold in fp32 bit patterns (same order as |r|;
      // the high digits of such keys are mostly zero, which lets the sort skip its last pass).
      keys[pos] = __float_as_uint(__builtin_fabsf(r[e])) - thr_bits;
      pos++;
    }
    return;
  }
  int32_t* idx = reinterpret_cast<int32_t*>(out + 4);
  float* val = reinterpret_cast<float*>(out + 4 + size_t(total) * 4);
  while (m) {
    const uint32_t e = e0 + uint32_t(__builtin_ctzll(m));
    m &= m - 1;
    idx[pos] = int32_t(e);
    val[pos] = r[e];
    r[e] = 0.0f;
    pos++;
  }
}

// generate_S_value, gd_body.h:80-99, plus the header (gd_body.h:193-201), for a
// message whose k indices are already in place (the cut path).  A launch of its
// own with one lane per entry: done by the few workgroups of the last sort pass
// these random accesses to r took three times as long.
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
// Stable LSD radix sort of (key, index) pairs, 8 bits per pass, descending
// (bin = 255 - digit).  A pass is a count launch and a scatter launch over tiles
// of 8192 pairs (1024 lanes x 8), counts[tile * 256 + bin]; the last pass writes
// the message's index block instead of a sorted list.  (All passes in one launch
// with grid-wide barriers was tried and lost: data handed between workgroups
// inside a launch needs device-scope accesses or whole-L2 fences, either of
// which costs more than the launches saved.)  (Counting a pass's digits where its
// input is written, with global atomics, saves the count launches but was five
// times slower: some 10^5 scattered atomics cost more than the launches.)
struct SortArgs {
  const uint32_t* keys_in;
  const int32_t* idx_in;
  uint32_t n;
  int shift;
  const uint32_t* counts;   // this pass, complete
  uint32_t nblk;
  uint32_t* keys_out;       // not used by the last pass
  int32_t* idx_out;
  uint8_t* msg;             // last pass only: the message, whose index block gets the first `keep` indices
  uint32_t keep;
};

// Lanes of the wave whose `bin` equals this lane's, among the lanes in `live`.
__device__ __forceinline__ uint64_t match_bin(uint32_t bin, bool live) {
  uint64_t same = __ballot(live);
#pragma unroll
  for (int b = 0; b < 8; b++) {
    const uint64_t m = __ballot((bin >> b) & 1u);
    same &= ((bin >> b) & 1u) ? m : ~m;
  }
  return same;
}

// One LDS atomic per distinct bin of a wave's 64 keys, not one per key: the top
// digit of keys that are all just above one threshold is the same for nearly all
// of them, and 8192 atomics on one LDS word took longer than the rest of the pass.
__global__ __launch_bounds__(kSortThreads) void gd_sort_count_kernel(const uint32_t* __restrict__ keys, uint32_t n,
                                                                     int shift, uint32_t* __restrict__ counts) {
  __shared__ uint32_t s_hist[256];
  const uint32_t t = threadIdx.x;
  const uint32_t lane = t & (kWave - 1);
  if (t < 256) s_hist[t] = 0;
  const uint32_t b0 = blockIdx.x * uint32_t(kSortTile);
  uint32_t key[kSortPer];
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const uint32_t x = b0 + j * kSortThreads + t;
    key[j] = x < n ? keys[x] : 0u;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const bool live = b0 + j * kSortThreads + t < n;
    const uint32_t bin = 255u - ((key[j] >> shift) & 255u);
    const uint64_t same = match_bin(bin, live);
    if (live && (same & ((uint64_t(1) << lane) - 1)) == 0) atomicAdd(&s_hist[bin], uint32_t(__popcll(same)));
  }
  __syncthreads();
  if (t < 256) counts[size_t(blockIdx.x) * 256 + t] = s_hist[t];
}

// A wave owns 512 consecutive pairs of the tile and takes them 64 at a time, so
// the order wave, round, lane is the input order and equal digits keep it.  Per
// round the lanes of a wave that share a bin are found with ballots; the wave
// keeps its own running count per bin in its row of s_cnt (no workgroup barrier
// inside the loop).  One pass over the 16 rows gives every wave its first place
// per bin within the tile; the pairs are then put in that order in LDS, so that
// consecutive lanes write consecutive slots of a bin's run (scattering straight
// from registers costs one address per lane and made the pass twice as long).
__global__ __launch_bounds__(kSortThreads) void gd_sort_pass_kernel(const SortArgs a) {
  extern __shared__ uint32_t s_stage[];          // [kSortTile] keys, then [kSortTile] indices
  __shared__ uint32_t s_cnt[kSortWaves][256];    // per wave: pairs per bin, then the wave's first place per bin
  __shared__ uint32_t s_first[256];              // first place of the bin within the tile
  __shared__ uint32_t s_slot[256];               // first global slot of the bin's pairs of this tile
  __shared__ uint32_t s_part[8];
  uint32_t* s_key = s_stage;
  uint32_t* s_id = s_stage + kSortTile;
  const uint32_t t = threadIdx.x;
  const uint32_t lane = t & (kWave - 1), wave = t / kWave;
  const uint32_t n = a.n;
  const uint32_t b0 = blockIdx.x * uint32_t(kSortTile);
  const uint32_t x0 = b0 + wave * uint32_t(kSortPer * kWave) + lane;
  uint32_t key[kSortPer];
  int32_t id[kSortPer];
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const uint32_t x = x0 + j * kWave;
    key[j] = x < n ? a.keys_in[x] : 0u;
    id[j] = x < n ? a.idx_in[x] : 0;
  }
  // bin t (first 256 lanes): pairs in all tiles, in the tiles before this one, in this one.
  // The first 32 tiles are read with independent loads.
  uint32_t total = 0, before = 0, mine = 0;
  if (t < 256) {
    constexpr uint32_t kFlat = 32;
    uint32_t c[kFlat];
#pragma unroll
    for (uint32_t q = 0; q < kFlat; q++) c[q] = q < a.nblk ? a.counts[size_t(q) * 256 + t] : 0u;
#pragma unroll
    for (uint32_t q = 0; q < kFlat; q++) {
      total += c[q];
      before += q < blockIdx.x ? c[q] : 0u;
      mine += q == blockIdx.x ? c[q] : 0u;
    }
    for (uint32_t q = kFlat; q < a.nblk; q++) {
      const uint32_t v = a.counts[size_t(q) * 256 + t];
      total += v;
      before += q < blockIdx.x ? v : 0u;
      mine += q == blockIdx.x ? v : 0u;
    }
  }
  if (a.msg) {
    // Last pass: if every key has the same digit the input is already in order.
    if (__syncthreads_or(t < 256 && total == n)) {
#pragma unroll
      for (int j = 0; j < kSortPer; j++) {
        const uint32_t x = x0 + j * kWave;
        if (x < n && x < a.keep) reinterpret_cast<int32_t*>(a.msg + 4)[x] = id[j];
      }
      return;
    }
  }
#pragma unroll
  for (int q = 0; q < 256 / kWave; q++) s_cnt[wave][q * kWave + lane] = 0;  // own row: no barrier needed before use

  uint32_t place[kSortPer], bin[kSortPer];
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const bool live = x0 + j * kWave < n;
    bin[j] = 255u - ((key[j] >> a.shift) & 255u);
    const uint64_t same = match_bin(bin[j], live);
    const uint32_t rank = __popcll(same & ((uint64_t(1) << lane) - 1));
    uint32_t base = 0;
    if (live && rank == 0) {
      base = s_cnt[wave][bin[j]];
      s_cnt[wave][bin[j]] = base + uint32_t(__popcll(same));
    }
    base = __shfl(base, live ? __builtin_ctzll(same) : int(lane), kWave);
    place[j] = base + rank;
  }

  // Exclusive scans over the 256 bins, of the global totals and of this tile's
  // counts: within each of the first four waves, then across them.
  uint32_t incl_g = total, incl_l = mine;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t vg = __shfl_up(incl_g, o, kWave), vl = __shfl_up(incl_l, o, kWave);
    if (lane >= uint32_t(o)) { incl_g += vg; incl_l += vl; }
  }
  if (t < 256 && lane == kWave - 1) { s_part[wave] = incl_g; s_part[4 + wave] = incl_l; }
  __syncthreads();  // also: every wave's row of s_cnt is complete
  if (t < 256) {
    uint32_t slot = incl_g - total + before, first = incl_l - mine;
    for (uint32_t w = 0; w < wave; w++) { slot += s_part[w]; first += s_part[4 + w]; }
    s_slot[t] = slot;
    s_first[t] = first;
    uint32_t run = first;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) {
      const uint32_t c = s_cnt[w][t];
      s_cnt[w][t] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    if (x0 + j * kWave < n) {
      const uint32_t p = s_cnt[wave][bin[j]] + place[j];
      s_key[p] = key[j];
      s_id[p] = uint32_t(id[j]);
    }
  }
  __syncthreads();
  const uint32_t live_n = n - b0 < uint32_t(kSortTile) ? n - b0 : uint32_t(kSortTile);
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const uint32_t p = j * kSortThreads + t;
    if (p < live_n) {
      const uint32_t k = s_key[p];
      const int32_t i = int32_t(s_id[p]);
      const uint32_t b = 255u - ((k >> a.shift) & 255u);
      const uint32_t slot = s_slot[b] + (p - s_first[b]);
      if (a.msg) {
        // last pass: the indices that survive the cut go straight into the message
        if (slot < a.keep) reinterpret_cast<int32_t*>(a.msg + 4)[slot] = i;
      } else {
        a.keys_out[slot] = k;
        a.idx_out[slot] = i;
      }
    }
  }
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

// The four passes of the cut path: (keys_a, idx_a) hold the candidates in index
// order.  The last pass writes the indices of the `keep` largest into the
// message `msg`; a gather launch adds values and header and clears the residual.
int sort_and_cut(uint32_t* keys_a, int32_t* idx_a, uint32_t* keys_b, int32_t* idx_b, uint32_t* counts, uint32_t n,
                 uint8_t* msg, float* r, uint32_t keep, hipStream_t st) {
  constexpr int kStageBytes = 2 * kSortTile * int(sizeof(uint32_t));
  // The dynamic-LDS limit is a property of the function on one device: raise it once per device.
  static std::mutex attr_mu;
  static uint64_t attr_done = 0;  // bit d: done on device d (devices beyond 63 set it on every call)
  {
    int dev = 0;
    HPX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(attr_mu);
    if (dev >= 64 || !(attr_done >> dev & 1)) {
      HPX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gd_sort_pass_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kStageBytes));
      if (dev < 64) attr_done |= uint64_t(1) << dev;
    }
  }
  const uint32_t nblk = cdiv(n, kSortTile);
  for (int pass = 0; pass < 4; pass++) {
    SortArgs a;
    a.keys_in = keys_a; a.idx_in = idx_a; a.n = n; a.shift = pass * 8;
    a.counts = counts; a.nblk = nblk;
    a.keys_out = keys_b; a.idx_out = idx_b;
    a.msg = pass == 3 ? msg : nullptr;
    a.keep = keep;
    HPX_LAUNCH("gd_sort_count_kernel", gd_sort_count_kernel, dim3(nblk), dim3(kSortThreads), st, keys_a, n, a.shift, counts);
    if (hpx::g_prof_on) hpx::prof_begin("gd_sort_pass_kernel", st);
    hipLaunchKernelGGL(gd_sort_pass_kernel, dim3(nblk), dim3(kSortThreads), kStageBytes, st, a);
    if (hpx::g_prof_on) hpx::prof_end(st);
    HPX_HIP(hipGetLastError());
    std::swap(keys_a, keys_b);
    std::swap(idx_a, idx_b);
  }
  HPX_LAUNCH("gd_gather_kernel", gd_gather_kernel, dim3(cdiv(keep > 0 ? keep : 1, kThreads)), dim3(kThreads), st, msg, r, keep);
  HPX_HIP(hipGetLastError());
  return HPX_OK;
}

// One tensor.  With a residual (`residual` non-null): gd_body, s_percent = 1 - drop_ratio.  Without:
// dgc_with_auxiliary_body, where `grad` itself is thresholded and its selected entries cleared.
int gd_encode_one(float* grad, int32_t N, float* residual, uint8_t* out, double sample_rate, double s_percent,
                  uint64_t seed, hpx::Workspace* ws, hipStream_t st) {
  // size arithmetic of gd_body.h:112-115, :153 (dgc_body.h:79-80, :103)
  const int32_t sample_cnt = static_cast<int32_t>(std::ceil(N * sample_rate));
  const int32_t expected = static_cast<int32_t>(std::ceil(N * s_percent));
  const int32_t thr_index = static_cast<int32_t>(sample_cnt * s_percent);
  HPX_ARG(sample_cnt > 0 && thr_index >= 0 && thr_index < sample_cnt && expected >= 0,
          "sparsifier encode: N=%d sample_rate=%g kept fraction=%g give sample_cnt=%d threshold index=%d", N, sample_rate,
          s_percent, sample_cnt, thr_index);
  const float* g = grad;
  float* r = residual ? residual : grad;  // the array whose selected entries are read out and cleared

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
  // Room for the cut path (two copies of the candidates' keys and indices, and
  // the sort's counts) is laid out for a typical overshoot before anything is
  // launched: the expand kernel fills it without the host knowing the count.
  uint64_t cap64 = uint64_t(expected) * 2 > uint64_t(expected) + 65536 ? uint64_t(expected) * 2 : uint64_t(expected) + 65536;
  if (cap64 > n) cap64 = n;
  const uint32_t cap = static_cast<uint32_t>(cap64);
  struct CutLayout { size_t ka, kb, ia, ib, sc, end; };
  auto cut_layout = [](size_t at, uint64_t pairs) {
    CutLayout c;
    c.ka = at; at += align256(sizeof(uint32_t) * size_t(pairs));
    c.kb = at; at += align256(sizeof(uint32_t) * size_t(pairs));
    c.ia = at; at += align256(sizeof(int32_t) * size_t(pairs));
    c.ib = at; at += align256(sizeof(int32_t) * size_t(pairs));
    c.sc = at; at += align256(sizeof(uint32_t) * 256 * size_t(cdiv(pairs, kSortTile)));
    c.end = at;
    return c;
  };
  CutLayout cl = cut_layout(off, cap);
  int rc = hpx::ensure_workspace(ws, cl.end);
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

  SelArgs sa{g, residual, n, static_cast<uint32_t>(sample_cnt), static_cast<uint32_t>(seed), static_cast<uint32_t>(thr_index),
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
  if (residual)
    HPX_LAUNCH("gd_stream_kernel", gd_stream_kernel<true>, dim3(ntiles), dim3(kThreads), st, g, r, n, state, masks, blk_cnt);
  else
    HPX_LAUNCH("gd_stream_kernel", gd_stream_kernel<false>, dim3(ntiles), dim3(kThreads), st, g, r, n, state, masks, blk_cnt);
  uint32_t* h_total = reinterpret_cast<uint32_t*>(ws->pinned);
  HPX_LAUNCH("gd_scan_kernel", gd_scan_kernel, dim3(nchunks), dim3(kSelThreads), st, blk_cnt, blk_off, ntiles, chunk_tot,
             chunk_off, state, h_total);
  HPX_HIP(hipGetLastError());
  // Queued before the host knows the count: the finish if nothing has to be cut,
  // else the candidate list and keys of the cut path.
  const uint32_t lim = static_cast<uint32_t>(expected);
  HPX_LAUNCH("gd_expand_kernel", gd_expand_kernel, dim3(cdiv(ntiles, kThreads / kWave)), dim3(kThreads), st, masks, blk_off,
             chunk_off, ntiles, state, lim, out, r, reinterpret_cast<int32_t*>(base + cl.ia),
             reinterpret_cast<uint32_t*>(base + cl.ka), cap);
  HPX_HIP(hipGetLastError());
  HPX_HIP(hipStreamSynchronize(st));
  const uint32_t total = *reinterpret_cast<volatile uint32_t*>(h_total);
  if (total <= lim) return HPX_OK;

  // More candidates than `expected`: order them by |r| descending and keep the first `expected`.
  if (total > cap) {
    // Far more candidates than reserved for.  Growing would discard the masks;
    // build the larger block, carry them over and list the candidates again.
    cl = cut_layout(off, total);
    uint8_t* old = ws->dev;
    const size_t old_bytes = ws->dev_bytes;
    ws->dev = nullptr;
    ws->dev_bytes = 0;
    rc = hpx::ensure_workspace(ws, cl.end);
    if (rc != HPX_OK) { (void)hipFree(old); return rc; }
    HPX_HIP(hipMemcpyAsync(ws->dev, old, off < old_bytes ? off : old_bytes, hipMemcpyDeviceToDevice, st));
    HPX_HIP(hipStreamSynchronize(st));
    HPX_HIP(hipFree(old));
    base = ws->dev;
    state = reinterpret_cast<GdState*>(base + o_state);
    masks = reinterpret_cast<uint64_t*>(base + o_masks);
    blk_off = reinterpret_cast<uint32_t*>(base + o_off);
    chunk_off = reinterpret_cast<uint32_t*>(base + o_coff);
    HPX_LAUNCH("gd_expand_kernel", gd_expand_kernel, dim3(cdiv(ntiles, kThreads / kWave)), dim3(kThreads), st, masks, blk_off,
               chunk_off, ntiles, state, 0u, out, r, reinterpret_cast<int32_t*>(base + cl.ia),
               reinterpret_cast<uint32_t*>(base + cl.ka), total);
    HPX_HIP(hipGetLastError());
  }
  uint32_t* ka = reinterpret_cast<uint32_t*>(base + cl.ka);
  uint32_t* kb = reinterpret_cast<uint32_t*>(base + cl.kb);
  int32_t* ia = reinterpret_cast<int32_t*>(base + cl.ia);
  int32_t* ib = reinterpret_cast<int32_t*>(base + cl.ib);
  uint32_t* sc = reinterpret_cast<uint32_t*>(base + cl.sc);
  rc = sort_and_cut(ka, ia, kb, ib, sc, total, out, r, lim, st);
  if (rc != HPX_OK) return rc;
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
  if (const int rcc = hpx::reject_capture(st, "hpx_gd_encode")) return rcc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int worst = HPX_OK;
  for (int i = 0; i < count; i++) {
    const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
    const int rc = gd_encode_one(const_cast<float*>(grads[i]), Ns[i], residuals[i], outs[i], sample_rates[i],
                                 1 - drop_ratios[i], seed, ws, st);
    if (rc != HPX_OK && worst == HPX_OK) worst = rc;  // like the reference driver: report, go on
  }
  return worst;
}

namespace {
// gd_r_body (zero_fill: write mode clears the whole output first, gd_body.h:335-347)
// and dgc_r_body (no clearing, dgc_body.h:283-289).
int decode_messages(int count, const uint8_t* const* ins, const int32_t* in_sizes, float* const* outs,
                    const int32_t* out_sizes, const int32_t* is_add_tos, bool zero_fill, hpx_stream_t stream) {
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
  if (const int rcc = hpx::reject_capture(st, zero_fill ? "hpx_gd_decode" : "hpx_dgc_decode")) return rcc;
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
      if (n && zero_fill) {
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
}  // namespace

HPX_API int hpx_gd_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes, float* const* outs,
                          const int32_t* out_sizes, const int32_t* is_add_tos, hpx_stream_t stream) {
  return decode_messages(count, ins, in_sizes, outs, out_sizes, is_add_tos, true, stream);
}

HPX_API int hpx_dgc_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes, float* const* outs,
                           const int32_t* out_sizes, const int32_t* is_add_tos, hpx_stream_t stream) {
  return decode_messages(count, ins, in_sizes, outs, out_sizes, is_add_tos, false, stream);
}

HPX_API int hpx_dgc_encode(int count, float* const* grads, const int32_t* Ns, uint8_t* const* outs,
                           const double* sample_rates, const double* s_percents, const uint64_t* seeds,
                           hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_dgc_encode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(grads && Ns && outs && sample_rates && s_percents, "hpx_dgc_encode: null argument array");
  for (int i = 0; i < count; i++) {
    HPX_ARG(Ns[i] > 0, "hpx_dgc_encode: tensor %d has size %d (must be positive)", i, Ns[i]);
    HPX_ARG(grads[i] && outs[i], "hpx_dgc_encode: tensor %d has a null pointer", i);
    HPX_ARG((reinterpret_cast<uintptr_t>(outs[i]) & 3) == 0, "hpx_dgc_encode: output %d is not 4-byte aligned", i);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const int rcc = hpx::reject_capture(st, "hpx_dgc_encode")) return rcc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int worst = HPX_OK;
  for (int i = 0; i < count; i++) {
    const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
    const int rc = gd_encode_one(grads[i], Ns[i], nullptr, outs[i], sample_rates[i], s_percents[i], seed, ws, st);
    if (rc != HPX_OK && worst == HPX_OK) worst = rc;
  }
  return worst;
}

