// GradDrop ("DGC") sparsifier: residual accumulation, sampled threshold,
// order-preserving compaction, optional cut to the k largest, scatter decode.
//
// Semantics follow gd_body.h:102-232 (encode) and :283-353 (decode).  The
// reference makes a pass for R += G, a gather for the sample, a full sort of
// the sample, a two-pass copy_if and waits for the stream three times, tensor
// after tensor.  Here every phase is ONE launch for all tensors of a call (a
// table of tensors in the kernel arguments, as in the TBQ and TernGrad paths):
//
//   sample      |G[i]+R[i]| at the reference's LCG index stream, gathered
//               BEFORE the update (the same fp32 sum the update will store)
//   select      exact k-th largest of the sample by three radix-histogram
//               passes over the fp32 bit pattern (11+11+10 bits); no sort
//   stream      ONE pass over the tensor: r = g + r, store r, compare with the
//               threshold, wave64 ballot -> one 64-bit word per 64 elements
//               (bit i = element i), a popcount and the largest |r| per workgroup
//   scan        exclusive prefix of the per-workgroup counts within chunks of 4096,
//               the chunks' totals and largest |r|
//   expand      folds the chunk totals (each wave for itself), reports count,
//               threshold and largest |r| of each tensor to the host; bit words ->
//               ascending indices at the scanned offsets, values out, residual
//               entries zeroed, header written
//
// The stream pass moves 12 bytes per element (g, r in; r out) plus 1/8 byte of
// mask; everything else touches O(sample + selected) data.  The host learns the
// candidate counts from pinned memory while the expand launch is still running
// (it polls the words the expand launch writes first; no wait for the stream), and only
// for tensors with more than `expected` candidates queues the cut: a stable LSD
// radix sort by |r| (ties keep ascending index) over as many byte digits as the
// largest key has, whose last pass writes the message.  The expand launch has
// by then left the candidates and their keys where the sort wants them.
#include <cmath>
#include <vector>

#include <immintrin.h>

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
constexpr int kHistWords = kBins1 + kBins2 + kBins3;
constexpr int kCapLarge = 256;                   // tensors per launch table (17 KiB of kernel arguments)
constexpr int kCapSmall = 4;                     // calls with a few tensors pass a table of a few hundred bytes

struct GdState {
  uint32_t hits;      // provisional path: samples found above the provisional threshold so far
  uint32_t thr_bits;  // threshold as fp32 bits (provisional path: the provisional one until the exact one is known)
  uint32_t fallback;  // provisional path: 1 when the provisional threshold turned out to lie above the exact one
  uint32_t pad[61];
};
constexpr int kHitWays = 128;             // parts of the list of samples above the provisional threshold
constexpr uint32_t kPreSamples = 16384;  // samples the provisional threshold is taken from
constexpr uint32_t kFallback = 0xFFFFFFFEu;  // reported in place of a count: this tensor has to take the other path
constexpr int kScanChunk = 4096;   // per-tile counts scanned by one workgroup
constexpr int kMaxChunks = 128;    // 2^31 elements / kTile / kScanChunk

__host__ __device__ constexpr size_t align256(size_t x) { return (x + 255) & ~size_t(255); }
__host__ __device__ constexpr uint32_t cdiv(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }

// Where the pieces of one tensor's workspace block lie (the same arithmetic on the host and in the kernels).
struct GdLayout {
  size_t state, hist, samples, hitlist, masks, coarse, cnt, mx, off, ctot, cmax, coff, end;
};
__host__ __device__ inline GdLayout gd_layout(uint32_t n, uint32_t sample_cnt) {
  const size_t ntiles = cdiv(n, kTile);
  GdLayout l;
  size_t at = 0;
  l.state = at;   at += align256(sizeof(GdState));
  l.hist = at;    at += align256(sizeof(uint32_t) * kHistWords);
  l.samples = at; at += align256(sizeof(uint32_t) * size_t(sample_cnt));
  l.hitlist = at; at += align256(sizeof(uint32_t) * (size_t(sample_cnt) + size_t(256) * 128));  // provisional path, see gd_resample_kernel
  l.masks = at;   at += align256(sizeof(uint64_t) * ntiles * kWave);      // one bit per element
  l.coarse = at;  at += align256(sizeof(uint64_t) * ntiles);              // one bit per mask word: whether it has a bit set
  l.cnt = at;     at += align256(sizeof(uint32_t) * ntiles);              // candidates per tile
  l.mx = at;      at += align256(sizeof(uint32_t) * ntiles);              // largest |r| per tile, as bits
  l.off = at;     at += align256(sizeof(uint32_t) * ntiles);              // exclusive prefix within the chunk
  l.ctot = at;    at += align256(sizeof(uint32_t) * kMaxChunks);
  l.cmax = at;    at += align256(sizeof(uint32_t) * kMaxChunks);
  l.coff = at;    at += align256(sizeof(uint32_t) * kMaxChunks);
  l.end = at;
  return l;
}
// The cut path's buffers for up to `pairs` candidates: two copies of keys and indices, and the sort's counts.
constexpr int kSortThreads = 1024;
constexpr int kSortPer = 4;
constexpr int kSortTile = kSortThreads * kSortPer;   // tiles of 4096 pairs (8192: each launch of a pass 3 us longer)
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kSortBinsMax = 512;                    // bins of the widest digit the sort uses (9 bits)
struct CutLayout {
  size_t ka, kb, ia, ib, sc, end;
};
__host__ __device__ inline CutLayout cut_layout(uint64_t pairs) {
  CutLayout c;
  size_t at = 0;
  c.ka = at; at += align256(sizeof(uint32_t) * size_t(pairs));
  c.kb = at; at += align256(sizeof(uint32_t) * size_t(pairs));
  c.ia = at; at += align256(sizeof(int32_t) * size_t(pairs));
  c.ib = at; at += align256(sizeof(int32_t) * size_t(pairs));
  c.sc = at; at += align256(sizeof(uint32_t) * kSortBinsMax * size_t(cdiv(pairs, kSortTile)));
  c.end = at;
  return c;
}

// One tensor of a call.  64 bytes.
struct GdSeg {
  const float* g;      // the gradient
  float* r;            // the array whose entries are selected and cleared: the residual, or (without one) the gradient
  uint8_t* out;        // the message
  uint8_t* ws;         // this tensor's workspace block (gd_layout)
  uint8_t* cut;        // ... and its cut-path buffers (cut_layout)
  uint32_t n;
  uint32_t sample_cnt;
  uint32_t seed;       // low 32 bits of the 64-bit seed
  uint32_t thr_index;  // rank (descending, 0-based) of the threshold in the sample
  uint32_t limit;      // `expected`: more candidates than this are cut to this many
  uint32_t cap;        // pairs the cut-path buffers hold
};
static_assert(sizeof(GdSeg) == 64, "segment record");
// What the scan launch reports per tensor in pinned host memory.
constexpr int kReportWords = 4;  // count of candidates, threshold bits, bits of the largest |r|, unused
constexpr uint32_t kNotReported = 0xFFFFFFFFu;  // a count is < 2^31; as fp32 bits this is a NaN, which no threshold or |r| is
template <int CAP>
struct GdArgs {
  int32_t nseg;
  int32_t residual;             // 0: the sparsifier without residual (dgc_body.h)
  int32_t margin;               // provisional path: how many times the expected number of entries the provisional
                                // threshold lets through
  int32_t tile_start[CAP + 1];  // exclusive prefix of this launch's workgroups per tensor
  GdSeg seg[CAP];
  uint32_t* report;             // pinned host memory, kReportWords per tensor of this table
};
static_assert(sizeof(GdArgs<kCapLarge>) <= 18000, "kernel-argument budget");

__device__ __forceinline__ GdState* seg_state(const GdSeg& sg) { return reinterpret_cast<GdState*>(sg.ws); }

// Rank search in a descending cumulative histogram: returns the bin holding
// rank `rank_in` (0-based from the top) and the rank left inside that bin.
template <int BINS>
__device__ __forceinline__ void find_digit(const uint32_t* __restrict__ hist, uint32_t rank_in,
                                           uint32_t& digit, uint32_t& rank_out) {
  constexpr int PER = BINS / kSelThreads;
  static_assert(PER >= 1, "one bin per thread at least");
  constexpr int kWaves = kSelThreads / kWave;
  __shared__ uint32_t s_wave[kWaves];
  __shared__ uint32_t s_res[2];
  const int t = threadIdx.x;
  const uint32_t lane = t & (kWave - 1), wave = t / kWave;
  uint32_t h[PER], sum = 0;
#pragma unroll
  for (int j = 0; j < PER; j++) {
    h[j] = hist[BINS - 1 - (t * PER + j)];
    sum += h[j];
  }
  // Inclusive prefix over the threads in order: within each wave by shuffles, then the sixteen wave totals
  // (three workgroup barriers in all; a workgroup-wide scan through LDS, ten rounds of two barriers each, was
  // most of the time of the launches that call this).
  uint32_t incl = sum;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t v = __shfl_up(incl, o, kWave);
    if (lane >= uint32_t(o)) incl += v;
  }
  if (lane == kWave - 1) s_wave[wave] = incl;
  if (t == 0) { s_res[0] = 0; s_res[1] = 0; }
  __syncthreads();
  uint32_t before = 0;
#pragma unroll
  for (int w = 0; w < kWaves; w++) before += uint32_t(w) < wave ? s_wave[w] : 0u;
  const uint32_t excl = before + incl - sum;
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
// once.  The same launch clears the histograms of this call.
template <int CAP>
__global__ __launch_bounds__(kThreads) void gd_sample_kernel(const GdArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  uint32_t* hist = reinterpret_cast<uint32_t*>(sg.ws + l.hist);
  uint32_t* samples = reinterpret_cast<uint32_t*>(sg.ws + l.samples);
  const uint32_t x = uint32_t(tile - a.tile_start[s]) * kThreads + threadIdx.x;
  if (x < uint32_t(kHistWords)) hist[x] = 0;
  if (x < sg.sample_cnt) {
    const uint32_t i = sample_index(sg.seed, x, sg.n);
    // with a residual: |G[i] + R[i]|, the value the update is about to store; without (dgc_body.h:18-30): |G[i]|
    samples[x] = __float_as_uint(__builtin_fabsf(a.residual ? sg.g[i] + sg.r[i] : sg.g[i]));
  }
}

template <int PASS>
__device__ __forceinline__ void hist_accumulate(const uint32_t* __restrict__ samples, uint32_t sample_cnt, uint32_t block,
                                                uint32_t nblocks, uint32_t* s_hist, uint32_t prefix) {
  // PASS 1: all keys, digit = key >> 21.  PASS 2: keys with key>>21 == prefix,
  // digit = (key >> 10) & 2047.  PASS 3: keys with key>>10 == prefix, digit = key & 1023.
  const uint32_t stride = nblocks * kSelThreads;
  for (uint32_t x = block * kSelThreads + threadIdx.x; x < sample_cnt; x += stride) {
    const uint32_t key = samples[x];
    if (PASS == 1) {
      atomicAdd(&s_hist[key >> 21], 1u);
    } else if (PASS == 2) {
      if ((key >> 21) == prefix) atomicAdd(&s_hist[(key >> 10) & 2047u], 1u);
    } else {
      if ((key >> 10) == prefix) atomicAdd(&s_hist[key & 1023u], 1u);
    }
  }
}

template <int PASS, int CAP>
__global__ __launch_bounds__(kSelThreads) void gd_select_kernel(const GdArgs<CAP> a) {
  constexpr int BINS = PASS == 1 ? kBins1 : PASS == 2 ? kBins2 : kBins3;
  __shared__ uint32_t s_hist[BINS];
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  uint32_t* hist = reinterpret_cast<uint32_t*>(sg.ws + l.hist);
  for (int i = threadIdx.x; i < BINS; i += kSelThreads) s_hist[i] = 0;
  uint32_t prefix = 0;
  if (PASS >= 2) {
    uint32_t d1, rank;
    find_digit<kBins1>(hist, sg.thr_index, d1, rank);
    prefix = d1;
    if (PASS == 3) {
      uint32_t d2;
      find_digit<kBins2>(hist + kBins1, rank, d2, rank);
      prefix = (d1 << 11) | d2;
    }
  }
  __syncthreads();
  hist_accumulate<PASS>(reinterpret_cast<const uint32_t*>(sg.ws + l.samples), sg.sample_cnt,
                        uint32_t(tile - a.tile_start[s]), uint32_t(a.tile_start[s + 1] - a.tile_start[s]), s_hist, prefix);
  __syncthreads();
  uint32_t* gh = hist + (PASS == 1 ? 0 : PASS == 2 ? kBins1 : kBins1 + kBins2);
  for (int i = threadIdx.x; i < BINS; i += kSelThreads) {
    const uint32_t c = s_hist[i];
    if (c) atomicAdd(&gh[i], c);
  }
}

// One workgroup per tensor.
template <int CAP>
__global__ __launch_bounds__(kSelThreads) void gd_threshold_kernel(const GdArgs<CAP> a) {
  const GdSeg& sg = a.seg[blockIdx.x];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  const uint32_t* hist = reinterpret_cast<const uint32_t*>(sg.ws + l.hist);
  uint32_t d1, d2, d3, rank;
  find_digit<kBins1>(hist, sg.thr_index, d1, rank);
  find_digit<kBins2>(hist + kBins1, rank, d2, rank);
  find_digit<kBins3>(hist + kBins1 + kBins2, rank, d3, rank);
  if (threadIdx.x == 0) seg_state(sg)->thr_bits = (d1 << 21) | (d2 << 10) | d3;
}

// ---- the sampled threshold without the full gather (provisional path) -----------------------------------------
// The reference's threshold is the thr_index-th largest of a 1 % sample drawn at random positions: gathering it
// costs a 128-byte line of G and one of R per sample, a fifth of the traffic of the pass over the tensor itself,
// and it has to be finished before that pass can start.  This path starts the pass from a PROVISIONAL threshold
// instead - taken from the first kPreSamples samples only and set low enough (`margin` times the expected
// number of entries above it) that it all but certainly lies below the exact one - so the pass marks a superset
// of the candidates.  Every sample whose value exceeds the provisional threshold is then one whose bit the pass
// has set, so the exact threshold (the thr_index-th largest of ALL samples) is found among the samples whose bit is
// set: a gather over the bit mask (1 bit per element, cache-resident) and the values of the few that hit.  A last
// small pass clears the bits of the elements that do not exceed the exact threshold; scan and expand go on as
// ever.  Should fewer than thr_index + 1 samples exceed the provisional threshold (it was not below the exact one,
// or they tie), the tensor is reported as kFallback and the host sends it through the gather path, on the residual
// the pass has already updated.
//
// Rank `rank` (0-based from the top) of `count` keys in global memory, by one workgroup of kSelThreads lanes:
// three histogram passes of 11 + 11 + 10 bits in LDS.  Every lane returns the key.
__device__ __forceinline__ uint32_t select_rank(const uint32_t* __restrict__ keys, uint32_t count, uint32_t rank,
                                                uint32_t* s_hist) {
  uint32_t prefix = 0;
#pragma unroll 1
  for (int pass = 1; pass <= 3; pass++) {
    for (int i = threadIdx.x; i < kBins1; i += kSelThreads) s_hist[i] = 0;
    __syncthreads();
    for (uint32_t x = threadIdx.x; x < count; x += kSelThreads) {
      const uint32_t key = keys[x];
      if (pass == 1) atomicAdd(&s_hist[key >> 21], 1u);
      else if (pass == 2) { if ((key >> 21) == prefix) atomicAdd(&s_hist[(key >> 10) & 2047u], 1u); }
      else if ((key >> 10) == prefix) atomicAdd(&s_hist[key & 1023u], 1u);
    }
    __syncthreads();
    uint32_t d;
    if (pass == 3) find_digit<kBins3>(s_hist, rank, d, rank); else find_digit<kBins1>(s_hist, rank, d, rank);
    prefix = pass == 1 ? d : pass == 2 ? ((prefix << 11) | d) : ((prefix << 10) | d);
  }
  return prefix;
}

// The first kPreSamples samples, one per lane over many workgroups (one workgroup's gathers into arrays of
// hundreds of megabytes are bound by its CU's address translation: 16384 of them took it 90 us).
template <int CAP>
__global__ __launch_bounds__(kThreads) void gd_presample_kernel(const GdArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  uint32_t* samples = reinterpret_cast<uint32_t*>(sg.ws + l.samples);
  const uint32_t s0 = sg.sample_cnt < kPreSamples ? sg.sample_cnt : kPreSamples;
  const uint32_t x = uint32_t(tile - a.tile_start[s]) * kThreads + threadIdx.x;
  if (x < s0) {
    const uint32_t i = sample_index(sg.seed, x, sg.n);
    samples[x] = __float_as_uint(__builtin_fabsf(a.residual ? sg.g[i] + sg.r[i] : sg.g[i]));
  }
}

// One workgroup per tensor: the provisional threshold from those samples; clears what the later phases count in.
template <int CAP>
__global__ __launch_bounds__(kSelThreads) void gd_provisional_kernel(const GdArgs<CAP> a) {
  __shared__ uint32_t s_hist[kBins1];
  const GdSeg& sg = a.seg[blockIdx.x];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  const uint32_t* samples = reinterpret_cast<const uint32_t*>(sg.ws + l.samples);
  const uint32_t s0 = sg.sample_cnt < kPreSamples ? sg.sample_cnt : kPreSamples;
  // rank of the provisional threshold among the s0 samples: `margin` times where the exact one is expected
  uint64_t kp = 0;
  if (a.margin > 0) kp = (uint64_t(a.margin) * (uint64_t(sg.thr_index) + 1) * s0 + sg.sample_cnt - 1) / sg.sample_cnt + 8;
  if (kp > s0 - 1) kp = s0 - 1;
  const uint32_t key = select_rank(samples, s0, uint32_t(kp), s_hist);
  uint32_t* ways = reinterpret_cast<uint32_t*>(sg.ws + l.hist);
  if (threadIdx.x < uint32_t(kHitWays)) ways[threadIdx.x] = 0;
  if (threadIdx.x == 0) {
    GdState* st = seg_state(sg);
    st->thr_bits = key;
    st->hits = 0;
    st->fallback = 0;
  }
}

// All samples against the bit mask the pass left: the values of those whose bit is set are listed.  The list is
// kept in kHitWays parts, workgroup b appending to part b % kHitWays (one counter for all would take the few
// thousand appends one after the other, 37 ns each); a part has room for every sample its workgroups look at.
__host__ __device__ inline uint32_t hit_way_room(uint32_t sample_cnt) {
  const uint32_t blocks = cdiv(sample_cnt, kThreads);
  return cdiv(blocks, kHitWays) * uint32_t(kThreads);
}
template <int CAP>
__global__ __launch_bounds__(kThreads) void gd_resample_kernel(const GdArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  const uint64_t* __restrict__ masks = reinterpret_cast<const uint64_t*>(sg.ws + l.masks);
  const uint32_t blk = uint32_t(tile - a.tile_start[s]);
  const uint32_t way = blk % uint32_t(kHitWays);
  uint32_t* hits = reinterpret_cast<uint32_t*>(sg.ws + l.hitlist) + size_t(way) * hit_way_room(sg.sample_cnt);
  uint32_t* counter = reinterpret_cast<uint32_t*>(sg.ws + l.hist) + way;
  const uint32_t x = blk * kThreads + threadIdx.x;
  bool hit = false;
  uint32_t i = 0;
  if (x < sg.sample_cnt) {
    i = sample_index(sg.seed, x, sg.n);
    // first whether the element's mask word has any bit at all (one bit per word: the whole map stays in cache),
    // and only then the word itself
    const uint64_t* __restrict__ coarse = reinterpret_cast<const uint64_t*>(sg.ws + l.coarse);
    if ((coarse[i >> 12] >> ((i >> 6) & 63u)) & 1ull) hit = (masks[i >> 6] >> (i & 63u)) & 1ull;
  }
  const uint64_t m = __ballot(hit);
  if (m == 0) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t base = 0;
  if (lane == uint32_t(__builtin_ctzll(m))) base = atomicAdd(counter, uint32_t(__popcll(m)));
  base = __shfl(base, __builtin_ctzll(m), kWave);
  if (hit) hits[base + uint32_t(__popcll(m & ((1ull << lane) - 1ull)))] = __float_as_uint(__builtin_fabsf(sg.r[i]));
}

// One workgroup per tensor: the parts of the list are drawn together (into the samples' block, free by now), then
// the exact threshold is taken from them, or the other path called for.
template <int CAP>
__global__ __launch_bounds__(kSelThreads) void gd_exact_kernel(const GdArgs<CAP> a) {
  __shared__ uint32_t s_hist[kBins1];
  __shared__ uint32_t s_off[kHitWays + 1];
  const GdSeg& sg = a.seg[blockIdx.x];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  GdState* st = seg_state(sg);
  const uint32_t* ways = reinterpret_cast<const uint32_t*>(sg.ws + l.hist);
  if (threadIdx.x == 0) {
    uint32_t run = 0;
    for (int w = 0; w < kHitWays; w++) { s_off[w] = run; run += ways[w]; }
    s_off[kHitWays] = run;
  }
  __syncthreads();
  const uint32_t found = s_off[kHitWays];
  if (found <= sg.thr_index) {
    if (threadIdx.x == 0) st->fallback = 1;
    return;
  }
  const uint32_t* parts = reinterpret_cast<const uint32_t*>(sg.ws + l.hitlist);
  uint32_t* keys = reinterpret_cast<uint32_t*>(sg.ws + l.samples);
  const uint32_t room = hit_way_room(sg.sample_cnt);
  for (int w = threadIdx.x / kWave; w < kHitWays; w += kSelThreads / kWave) {
    const uint32_t c = s_off[w + 1] - s_off[w];
    for (uint32_t k = threadIdx.x & (kWave - 1); k < c; k += kWave) keys[s_off[w] + k] = parts[size_t(w) * room + k];
  }
  __syncthreads();
  const uint32_t key = select_rank(keys, found, sg.thr_index, s_hist);
  if (threadIdx.x == 0) st->thr_bits = key;
}

// The bits of the elements that exceed the provisional threshold but not the exact one are cleared, the tiles'
// counts corrected: a wave per tile, a mask word per lane, the value of a word's first set bit loaded for all
// lanes together.
template <int CAP>
__global__ __launch_bounds__(kThreads) void gd_recount_kernel(const GdArgs<CAP> a) {
  const int blk = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, blk);
  const GdSeg& sg = a.seg[s];
  const GdState* st = seg_state(sg);
  if (st->fallback) return;
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  uint64_t* __restrict__ masks = reinterpret_cast<uint64_t*>(sg.ws + l.masks);
  uint32_t* __restrict__ cnt = reinterpret_cast<uint32_t*>(sg.ws + l.cnt);
  const float* __restrict__ r = sg.r;
  const uint32_t ntiles = cdiv(sg.n, kTile);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t tile = uint32_t(blk - a.tile_start[s]) * (kThreads / kWave) + threadIdx.x / kWave;
  if (tile >= ntiles) return;
  if (cnt[tile] == 0) return;  // wave-uniform
  const float thr = __uint_as_float(st->thr_bits), nthr = -thr;
  const uint64_t old = masks[size_t(tile) * kWave + lane];
  const uint32_t e0 = tile * uint32_t(kTile) + lane * kWave;
  uint64_t m = old, keep = 0;
  const uint32_t b1 = m ? uint32_t(__builtin_ctzll(m)) : 0u;
  const float v1 = m ? r[e0 + b1] : 0.0f;
  if (m) {
    if (v1 > thr || v1 < nthr) keep |= 1ull << b1;
    m &= m - 1;
  }
  while (m) {
    const uint32_t b = uint32_t(__builtin_ctzll(m));
    m &= m - 1;
    const float v = r[e0 + b];
    if (v > thr || v < nthr) keep |= 1ull << b;
  }
  if (keep != old) masks[size_t(tile) * kWave + lane] = keep;
  uint32_t c = uint32_t(__popcll(keep));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, kWave);
  if (lane == 0) cnt[tile] = c;
}

// The one pass over the tensors.  Lane l of wave w handles elements
// base + w*1024 + c*64 + l for c = 0..15, so ballot number c is the mask word of
// 64 consecutive elements in natural bit order.
// RESIDUAL = false is the sparsifier without residual (dgc_body.h:110-117): the
// values are G itself, nothing is added and nothing is stored (4 bytes per element).
template <bool RESIDUAL, int CAP>
__global__ __launch_bounds__(kThreads) void gd_stream_kernel(const GdArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  const float* __restrict__ g = sg.g;
  float* __restrict__ r = sg.r;
  const uint32_t n = sg.n;
  uint64_t* __restrict__ masks = reinterpret_cast<uint64_t*>(sg.ws + l.masks);
  const uint32_t t = uint32_t(tile - a.tile_start[s]);
  const float thr = __uint_as_float(seg_state(sg)->thr_bits);
  const float nthr = -thr;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wave = threadIdx.x / kWave;
  const uint32_t base = t * uint32_t(kTile);
  const uint32_t wbase = base + wave * uint32_t(kWaveTile);
  uint32_t lo = 0, hi = 0, cnt = 0;
  float big = 0.0f;  // largest |x| this lane has seen
  float gv[kPerLane], rv[kPerLane];
  if (n - base >= uint32_t(kTile)) {
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
      big = __builtin_fmaxf(big, __builtin_fabsf(x));
      lo = lane == uint32_t(c) ? uint32_t(m) : lo;  // lane c keeps mask word c
      hi = lane == uint32_t(c) ? uint32_t(m >> 32) : hi;
    }
  } else {
    // The tile that holds the end of the tensor: all its loads first, as above (a load, add, store per
    // step would make this one workgroup wait for memory sixteen times in a row at the very end of the launch).
#pragma unroll
    for (int c = 0; c < kPerLane; c++) {
      const uint32_t e = wbase + c * kWave + lane;
      gv[c] = e < n ? g[e] : 0.0f;
      rv[c] = (RESIDUAL && e < n) ? r[e] : 0.0f;
    }
#pragma unroll
    for (int c = 0; c < kPerLane; c++) {
      const uint32_t e = wbase + c * kWave + lane;
      bool p = false;
      if (e < n) {
        const float x = RESIDUAL ? gv[c] + rv[c] : gv[c];
        if (RESIDUAL) r[e] = x;
        p = (x > thr) || (x < nthr);
        big = __builtin_fmaxf(big, __builtin_fabsf(x));
      }
      const uint64_t m = __ballot(p);
      cnt += __popcll(m);
      lo = lane == uint32_t(c) ? uint32_t(m) : lo;  // lane c keeps mask word c
      hi = lane == uint32_t(c) ? uint32_t(m >> 32) : hi;
    }
  }
  if (lane < kPerLane) masks[(size_t(wbase) >> 6) + lane] = (uint64_t(hi) << 32) | lo;
  // which of the wave's sixteen mask words have a bit set (lanes beyond the sixteenth hold zeros)
  const uint32_t any16 = uint32_t(__ballot((lo | hi) != 0u));
  uint32_t bigb = __float_as_uint(big);  // non-negative floats order like their bit patterns; a NaN is not an input
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { const uint32_t v = __shfl_xor(bigb, o, kWave); bigb = v > bigb ? v : bigb; }
  __shared__ uint32_t s_cnt[kThreads / kWave], s_big[kThreads / kWave], s_any[kThreads / kWave];
  if (lane == 0) { s_cnt[wave] = cnt; s_big[wave] = bigb; s_any[wave] = any16; }
  __syncthreads();
  if (threadIdx.x == 0) {
    reinterpret_cast<uint32_t*>(sg.ws + l.cnt)[t] = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
    reinterpret_cast<uint64_t*>(sg.ws + l.coarse)[t] =
        uint64_t(s_any[0]) | (uint64_t(s_any[1]) << 16) | (uint64_t(s_any[2]) << 32) | (uint64_t(s_any[3]) << 48);
    const uint32_t m01 = s_big[0] > s_big[1] ? s_big[0] : s_big[1], m23 = s_big[2] > s_big[3] ? s_big[2] : s_big[3];
    reinterpret_cast<uint32_t*>(sg.ws + l.mx)[t] = m01 > m23 ? m01 : m23;
  }
}

// Exclusive prefix of the per-tile counts within chunks of 4096 tiles: workgroup c of a tensor scans counts
// [c*4096, (c+1)*4096) into `off` (relative to its chunk) and leaves the chunk's total and largest |r|.
// The second level - at most 128 chunk totals per tensor - is folded by the expand launch itself, each
// wave for its own tiles, so no workgroup here waits for or counts the others.
template <int CAP>
__global__ __launch_bounds__(kSelThreads) void gd_scan_kernel(const GdArgs<CAP> a) {
  __shared__ uint32_t s_wave[kSelThreads / kWave], s_wmax[kSelThreads / kWave];
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  const uint32_t* __restrict__ cnt = reinterpret_cast<const uint32_t*>(sg.ws + l.cnt);
  const uint32_t* __restrict__ mxs = reinterpret_cast<const uint32_t*>(sg.ws + l.mx);
  uint32_t* __restrict__ off = reinterpret_cast<uint32_t*>(sg.ws + l.off);
  uint32_t* chunk_tot = reinterpret_cast<uint32_t*>(sg.ws + l.ctot);
  uint32_t* chunk_max = reinterpret_cast<uint32_t*>(sg.ws + l.cmax);
  const uint32_t n = cdiv(sg.n, kTile);                                   // tiles of this tensor
  const uint32_t chunk = uint32_t(tile - a.tile_start[s]);
  const uint32_t t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
  const uint32_t i0 = chunk * uint32_t(kScanChunk) + t * 4;
  uint32_t c[4], big = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    c[j] = (i0 + j < n) ? cnt[i0 + j] : 0u;
    const uint32_t m = (i0 + j < n) ? mxs[i0 + j] : 0u;
    big = m > big ? m : big;
  }
  const uint32_t sum = c[0] + c[1] + c[2] + c[3];
  uint32_t incl = sum;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t v = __shfl_up(incl, o, kWave);
    if (lane >= uint32_t(o)) incl += v;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { const uint32_t v = __shfl_xor(big, o, kWave); big = v > big ? v : big; }
  if (lane == kWave - 1) { s_wave[wave] = incl; s_wmax[wave] = big; }
  __syncthreads();
  uint32_t before = 0, all = 0, allmax = 0;
#pragma unroll
  for (uint32_t w = 0; w < kSelThreads / kWave; w++) {
    const uint32_t v = s_wave[w];
    if (w < wave) before += v;
    all += v;
    allmax = s_wmax[w] > allmax ? s_wmax[w] : allmax;
  }
  uint32_t run = before + incl - sum;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    if (i0 + j < n) off[i0 + j] = run;
    run += c[j];
  }
  if (t == 0) {
    chunk_tot[chunk] = all;
    chunk_max[chunk] = allmax;
  }
}

// Turns the per-tile bit masks into the ascending index list, kExpandTiles consecutive tiles
// per wave (their mask words, and then the values of their first candidates, are loaded
// together: a wave with one tile spent its time waiting for one load after the other, and
// the launch needed four rounds of such waves), at the offsets the scan produced.  Every wave
// folds the chunk totals for itself (at most 128 of them): the offset of its tiles' chunks and the
// tensor's candidate count; the wave of a tensor's first tile reports count, threshold and
// largest |r| to the host.  If the stream pass found at most `limit`
// candidates this is the finish (gd_body.h:193-229): indices, values and header
// are written and the residual entries cleared.  If it found more, the candidates
// and their keys (bits of |r|) go to the cut path's buffers instead and
// nothing else is touched; more than `cap` candidates do not fit those buffers
// and the kernel does nothing for that tensor (the host then calls it again with larger ones,
// limit = 0 and no report).
constexpr int kExpandTiles = 4;
constexpr int kExpandPerBlock = (kThreads / kWave) * kExpandTiles;  // tiles per workgroup
template <int CAP>
__global__ __launch_bounds__(kThreads) void gd_expand_kernel(const GdArgs<CAP> a) {
  const int blk = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, blk);
  const GdSeg& sg = a.seg[s];
  const GdLayout l = gd_layout(sg.n, sg.sample_cnt);
  const CutLayout cl = cut_layout(sg.cap);
  const GdState* st = seg_state(sg);
  const uint64_t* __restrict__ masks = reinterpret_cast<const uint64_t*>(sg.ws + l.masks);
  const uint32_t* __restrict__ tile_off = reinterpret_cast<const uint32_t*>(sg.ws + l.off);
  const uint32_t* __restrict__ chunk_tot = reinterpret_cast<const uint32_t*>(sg.ws + l.ctot);
  uint8_t* __restrict__ out = sg.out;
  float* __restrict__ r = sg.r;
  const uint32_t ntiles = cdiv(sg.n, kTile);
  const uint32_t nchunks = cdiv(ntiles, kScanChunk);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const uint32_t tile0 = (uint32_t(blk - a.tile_start[s]) * (kThreads / kWave) + wave) * kExpandTiles;

  // the masks of this wave's tiles: requested first, used last
  uint64_t m[kExpandTiles];
#pragma unroll
  for (int j = 0; j < kExpandTiles; j++) m[j] = tile0 + j < ntiles ? masks[size_t(tile0 + j) * kWave + lane] : 0ull;

  // chunk totals, two per lane: inclusive prefix over the lanes
  const uint32_t a0 = 2 * lane < nchunks ? chunk_tot[2 * lane] : 0u, a1 = 2 * lane + 1 < nchunks ? chunk_tot[2 * lane + 1] : 0u;
  uint32_t inc2 = a0 + a1;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t v = __shfl_up(inc2, o, kWave);
    if (lane >= uint32_t(o)) inc2 += v;
  }
  const uint32_t total = __builtin_amdgcn_readlane(inc2, kWave - 1);
  const uint32_t ex0 = inc2 - a0 - a1, ex1 = ex0 + a0;  // exclusive prefixes of chunks 2 * lane and 2 * lane + 1
  if (a.margin >= 0 && st->fallback) {
    // the provisional threshold was not below the exact one: nothing of what the masks hold may be used
    if (tile0 == 0 && a.report != nullptr && lane == 0) {
      uint32_t* rep = a.report + size_t(s) * kReportWords;
      __hip_atomic_store(rep + 0, kFallback, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      __hip_atomic_store(rep + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      __hip_atomic_store(rep + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    return;
  }
  if (tile0 == 0 && a.report != nullptr) {
    // Pinned host words the host polls (no copy command, no wait for the stream).  The host waits for each
    // of the three words to change, so plain system-scope stores do (a release would write the whole L2 back).
    const uint32_t* __restrict__ chunk_max = reinterpret_cast<const uint32_t*>(sg.ws + l.cmax);
    const uint32_t m0 = 2 * lane < nchunks ? chunk_max[2 * lane] : 0u, m1 = 2 * lane + 1 < nchunks ? chunk_max[2 * lane + 1] : 0u;
    uint32_t mm = m0 > m1 ? m0 : m1;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { const uint32_t v = __shfl_xor(mm, o, kWave); mm = v > mm ? v : mm; }
    if (lane == 0) {
      uint32_t* rep = a.report + size_t(s) * kReportWords;
      __hip_atomic_store(rep + 0, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      __hip_atomic_store(rep + 1, st->thr_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      __hip_atomic_store(rep + 2, mm, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
  const bool cut = total > sg.limit;
  if (cut && total > sg.cap) return;
  if (!cut && tile0 == 0 && lane == 0) *reinterpret_cast<int32_t*>(out) = int32_t(4 + total * 8);
  if (tile0 >= ntiles) return;

  // first place of every tile's candidates, then of this lane's within the tile
  uint32_t pos[kExpandTiles];
#pragma unroll
  for (int j = 0; j < kExpandTiles; j++) {
    const uint32_t tile = tile0 + j < ntiles ? tile0 + j : ntiles - 1;
    const uint32_t chunk = tile / kScanChunk;
    const uint32_t coff = __shfl((chunk & 1u) ? ex1 : ex0, int(chunk >> 1), kWave);
    const uint32_t c = __popcll(m[j]);
    uint32_t incl = c;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const uint32_t v = __shfl_up(incl, o, kWave);
      if (lane >= uint32_t(o)) incl += v;
    }
    pos[j] = coff + tile_off[tile] + incl - c;
  }
  // The first candidate of each of the lane's 64-element groups: their values are loaded together.
  uint32_t e1[kExpandTiles];
  float v1[kExpandTiles];
#pragma unroll
  for (int j = 0; j < kExpandTiles; j++) {
    e1[j] = (tile0 + j) * uint32_t(kTile) + lane * kWave + uint32_t(m[j] ? __builtin_ctzll(m[j]) : 0);
    v1[j] = m[j] ? r[e1[j]] : 0.0f;
  }
  if (cut) {
    int32_t* __restrict__ cand = reinterpret_cast<int32_t*>(sg.cut + cl.ia);
    uint32_t* __restrict__ keys = reinterpret_cast<uint32_t*>(sg.cut + cl.ka);
    const uint32_t thr_bits = st->thr_bits;
    // Sort key: distance of |r| above the threshold in fp32 bit patterns (same order as |r|;
    // the high digits of such keys are mostly zero, which lets the sort skip its last passes).
#pragma unroll
    for (int j = 0; j < kExpandTiles; j++) {
      if (m[j]) {
        cand[pos[j]] = int32_t(e1[j]);
        keys[pos[j]] = __float_as_uint(__builtin_fabsf(v1[j])) - thr_bits;
        pos[j]++;
        m[j] &= m[j] - 1;
      }
      const uint32_t e0 = (tile0 + j) * uint32_t(kTile) + lane * kWave;
      while (m[j]) {  // further candidates of the same group: rare
        const uint32_t e = e0 + uint32_t(__builtin_ctzll(m[j]));
        m[j] &= m[j] - 1;
        cand[pos[j]] = int32_t(e);
        keys[pos[j]] = __float_as_uint(__builtin_fabsf(r[e])) - thr_bits;
        pos[j]++;
      }
    }
    return;
  }
  int32_t* idx = reinterpret_cast<int32_t*>(out + 4);
  float* val = reinterpret_cast<float*>(out + 4 + size_t(total) * 4);
#pragma unroll
  for (int j = 0; j < kExpandTiles; j++) {
    if (m[j]) {
      idx[pos[j]] = int32_t(e1[j]);
      val[pos[j]] = v1[j];
      r[e1[j]] = 0.0f;
      pos[j]++;
      m[j] &= m[j] - 1;
    }
    const uint32_t e0 = (tile0 + j) * uint32_t(kTile) + lane * kWave;
    while (m[j]) {
      const uint32_t e = e0 + uint32_t(__builtin_ctzll(m[j]));
      m[j] &= m[j] - 1;
      idx[pos[j]] = int32_t(e);
      val[pos[j]] = r[e];
      r[e] = 0.0f;
      pos[j]++;
    }
  }
}

// ---- cut to the `expected` largest |r| (gd_body.h:176-187) ------------------
// Stable LSD radix sort of (key, index) pairs, 8 or 9 bits per pass (9 when that
// saves a pass: keys of 25 to 27 bits, as the configuration's heavy-tailed gradient
// gives, take three passes instead of four), descending (bin = BINS - 1 - digit).
// A pass is a count launch and a scatter launch over tiles of 4096 pairs
// (1024 lanes x 4), counts[tile * BINS + bin]; the last pass writes
// the message's index block instead of a sorted list.  All tensors of a call that
// have to be cut share these launches (a table of tensors in the kernel arguments);
// the number of passes is that of the tensor with the largest key (a pass over a
// digit that is zero in every key of a tensor leaves that tensor's order as it is).
// (All passes in one launch
// with grid-wide barriers was tried and lost: data handed between workgroups
// inside a launch needs device-scope accesses or whole-L2 fences, either of
// which costs more than the launches saved.)  (Counting a pass's digits where its
// input is written, with global atomics, saves the count launches but was five
// times slower: some 10^5 scattered atomics cost more than the launches.)
struct SortSeg {           // one tensor that is being cut; 64 bytes
  uint32_t* keys[2];       // the pass with parity p reads keys[p], idx[p] and writes keys[1 - p], idx[1 - p]
  int32_t* idx[2];
  uint32_t* counts;        // [tile][bins] of the current pass
  uint8_t* msg;            // the message: its index block gets the first `keep` indices from the last pass
  float* r;                // values are read from here, and cleared
  uint32_t n;              // candidates
  uint32_t keep;           // `expected`
};
static_assert(sizeof(SortSeg) == 64, "segment record");
template <int CAP>
struct SortArgs {
  int32_t nseg;
  int32_t shift;
  int32_t parity;
  int32_t last;            // this pass writes the messages
  int32_t tile_start[CAP + 1];
  SortSeg seg[CAP];
};
static_assert(sizeof(SortArgs<kCapLarge>) <= 18000, "kernel-argument budget");

// generate_S_value, gd_body.h:80-99, plus the header (gd_body.h:193-201), for
// messages whose k indices are already in place (the cut path).  A launch of its
// own with one lane per entry: done by the few workgroups of the last sort pass
// these random accesses to r took three times as long.  tile_start counts blocks of
// kThreads entries here.
template <int CAP>
__global__ __launch_bounds__(kThreads) void gd_gather_kernel(const SortArgs<CAP> a) {
  const int blk = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, blk);
  uint8_t* __restrict__ out = a.seg[s].msg;
  float* __restrict__ r = a.seg[s].r;
  const uint32_t k = a.seg[s].keep;
  const int32_t* idx = reinterpret_cast<const int32_t*>(out + 4);
  float* val = reinterpret_cast<float*>(out + 4 + size_t(k) * 4);
  const uint32_t x = uint32_t(blk - a.tile_start[s]) * kThreads + threadIdx.x;
  if (x == 0) *reinterpret_cast<int32_t*>(out) = int32_t(4 + k * 8);
  if (x < k) {
    const int32_t i = idx[x];
    val[x] = r[i];
    r[i] = 0.0f;
  }
}

// Lanes of the wave whose `bin` equals this lane's, among the lanes in `live`.
template <int BITS>
__device__ __forceinline__ uint64_t match_bin(uint32_t bin, bool live) {
  uint64_t same = __ballot(live);
#pragma unroll
  for (int b = 0; b < BITS; b++) {
    const uint64_t m = __ballot((bin >> b) & 1u);
    same &= ((bin >> b) & 1u) ? m : ~m;
  }
  return same;
}

// One LDS atomic per distinct bin of a wave's 64 keys, not one per key: the top
// digit of keys that are all just above one threshold is the same for nearly all
// of them, and 8192 atomics on one LDS word took longer than the rest of the pass.
template <int CAP, int BITS>
__global__ __launch_bounds__(kSortThreads) void gd_sort_count_kernel(const SortArgs<CAP> a) {
  constexpr uint32_t BINS = 1u << BITS;
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const uint32_t* __restrict__ keys = a.seg[s].keys[a.parity];
  const uint32_t n = a.seg[s].n;
  const int shift = a.shift;
  const uint32_t ltile = uint32_t(tile - a.tile_start[s]);
  uint32_t* __restrict__ counts = a.seg[s].counts;
  __shared__ uint32_t s_hist[BINS];
  const uint32_t t = threadIdx.x;
  const uint32_t lane = t & (kWave - 1);
  if (t < BINS) s_hist[t] = 0;
  const uint32_t b0 = ltile * uint32_t(kSortTile);
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
    const uint32_t bin = (BINS - 1) - ((key[j] >> shift) & (BINS - 1));
    const uint64_t same = match_bin<BITS>(bin, live);
    if (live && (same & ((uint64_t(1) << lane) - 1)) == 0) atomicAdd(&s_hist[bin], uint32_t(__popcll(same)));
  }
  __syncthreads();
  if (t < BINS) counts[size_t(ltile) * BINS + t] = s_hist[t];
}

// A wave owns 256 consecutive pairs of the tile and takes them 64 at a time, so
// the order wave, round, lane is the input order and equal digits keep it.  Per
// round the lanes of a wave that share a bin are found with ballots; the wave
// keeps its own running count per bin in its row of s_cnt (no workgroup barrier
// inside the loop).  One pass over the 16 rows gives every wave its first place
// per bin within the tile; the pairs are then put in that order in LDS, so that
// consecutive lanes write consecutive slots of a bin's run (scattering straight
// from registers costs one address per lane and made the pass twice as long).
template <int CAP, int BITS>
__global__ __launch_bounds__(kSortThreads) void gd_sort_pass_kernel(const SortArgs<CAP> a) {
  constexpr uint32_t BINS = 1u << BITS;
  constexpr uint32_t kBinWaves = BINS / kWave;    // waves whose lanes each look after one bin
  extern __shared__ uint32_t s_stage[];          // [kSortTile] keys, then [kSortTile] indices
  __shared__ uint32_t s_cnt[kSortWaves][BINS];   // per wave: pairs per bin, then the wave's first place per bin
  __shared__ uint32_t s_first[BINS];             // first place of the bin within the tile
  __shared__ uint32_t s_slot[BINS];              // first global slot of the bin's pairs of this tile
  __shared__ uint32_t s_part[2 * kBinWaves];
  uint32_t* s_key = s_stage;
  uint32_t* s_id = s_stage + kSortTile;
  const uint32_t t = threadIdx.x;
  const uint32_t lane = t & (kWave - 1), wave = t / kWave;
  const int gtile = blockIdx.x;
  const int sgi = find_segment<CAP>(a.tile_start, a.nseg, gtile);
  const SortSeg& sg = a.seg[sgi];
  const uint32_t n = sg.n;
  const uint32_t blk = uint32_t(gtile - a.tile_start[sgi]);                         // this tensor's tile ...
  const uint32_t nblk = uint32_t(a.tile_start[sgi + 1] - a.tile_start[sgi]);       // ... of so many
  const uint32_t* __restrict__ keys_in = sg.keys[a.parity];
  const int32_t* __restrict__ idx_in = sg.idx[a.parity];
  uint32_t* __restrict__ keys_out = sg.keys[1 - a.parity];
  int32_t* __restrict__ idx_out = sg.idx[1 - a.parity];
  const uint32_t* __restrict__ counts = sg.counts;
  uint8_t* __restrict__ msg = a.last ? sg.msg : nullptr;
  const uint32_t b0 = blk * uint32_t(kSortTile);
  const uint32_t x0 = b0 + wave * uint32_t(kSortPer * kWave) + lane;
  uint32_t key[kSortPer];
  int32_t id[kSortPer];
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const uint32_t x = x0 + j * kWave;
    key[j] = x < n ? keys_in[x] : 0u;
    id[j] = x < n ? idx_in[x] : 0;
  }
  // bin t (first BINS lanes): pairs in all tiles, in the tiles before this one, in this one.
  // The first 40 tiles (163,840 pairs) are read with independent loads.
  uint32_t total = 0, before = 0, mine = 0;
  if (t < BINS) {
    constexpr uint32_t kFlat = 40;
    uint32_t c[kFlat];
#pragma unroll
    for (uint32_t q = 0; q < kFlat; q++) c[q] = q < nblk ? counts[size_t(q) * BINS + t] : 0u;
#pragma unroll
    for (uint32_t q = 0; q < kFlat; q++) {
      total += c[q];
      before += q < blk ? c[q] : 0u;
      mine += q == blk ? c[q] : 0u;
    }
    for (uint32_t q = kFlat; q < nblk; q++) {
      const uint32_t v = counts[size_t(q) * BINS + t];
      total += v;
      before += q < blk ? v : 0u;
      mine += q == blk ? v : 0u;
    }
  }
  if (msg) {
    // Last pass: if every key has the same digit the input is already in order.
    if (__syncthreads_or(t < BINS && total == n)) {
#pragma unroll
      for (int j = 0; j < kSortPer; j++) {
        const uint32_t x = x0 + j * kWave;
        if (x < n && x < sg.keep) reinterpret_cast<int32_t*>(msg + 4)[x] = id[j];
      }
      return;
    }
  }
#pragma unroll
  for (uint32_t q = 0; q < kBinWaves; q++) s_cnt[wave][q * kWave + lane] = 0;  // own row: no barrier needed before use

  uint32_t place[kSortPer], bin[kSortPer];
#pragma unroll
  for (int j = 0; j < kSortPer; j++) {
    const bool live = x0 + j * kWave < n;
    bin[j] = (BINS - 1) - ((key[j] >> a.shift) & (BINS - 1));
    const uint64_t same = match_bin<BITS>(bin[j], live);
    const uint32_t rank = __popcll(same & ((uint64_t(1) << lane) - 1));
    uint32_t base = 0;
    if (live && rank == 0) {
      base = s_cnt[wave][bin[j]];
      s_cnt[wave][bin[j]] = base + uint32_t(__popcll(same));
    }
    base = __shfl(base, live ? __builtin_ctzll(same) : int(lane), kWave);
    place[j] = base + rank;
  }

  // Exclusive scans over the bins, of the global totals and of this tile's
  // counts: within each of the first BINS / 64 waves, then across them.
  uint32_t incl_g = total, incl_l = mine;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t vg = __shfl_up(incl_g, o, kWave), vl = __shfl_up(incl_l, o, kWave);
    if (lane >= uint32_t(o)) { incl_g += vg; incl_l += vl; }
  }
  if (t < BINS && lane == kWave - 1) { s_part[wave] = incl_g; s_part[kBinWaves + wave] = incl_l; }
  __syncthreads();  // also: every wave's row of s_cnt is complete
  if (t < BINS) {
    uint32_t slot = incl_g - total + before, first = incl_l - mine;
    for (uint32_t w = 0; w < wave; w++) { slot += s_part[w]; first += s_part[kBinWaves + w]; }
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
      const uint32_t b = (BINS - 1) - ((k >> a.shift) & (BINS - 1));
      const uint32_t slot = s_slot[b] + (p - s_first[b]);
      if (msg) {
        // last pass: the indices that survive the cut go straight into the message
        if (slot < sg.keep) reinterpret_cast<int32_t*>(msg + 4)[slot] = i;
      } else {
        keys_out[slot] = k;
        idx_out[slot] = i;
      }
    }
  }
}

// ---- decode -----------------------------------------------------------------
// The fill of a written tensor is a pure write stream: streaming stores, three workgroups per CU (hpx_common.h;
// 138 M elements: 119 -> 95 us for the whole call, 103 without the limit on the workgroups).
__global__ __launch_bounds__(kThreads) void gd_zero_kernel(float* __restrict__ out, uint32_t n) {
  const uint32_t stride = gridDim.x * kThreads * 4;
  for (uint32_t e = (blockIdx.x * kThreads + threadIdx.x) * 4; e < n; e += stride) {
    if (n - e >= 4) {
      st4_stream(out + e, make_float4(0.f, 0.f, 0.f, 0.f));
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

// One tensor of the cut path as the host sees it.
struct CutJob {
  SortSeg seg;
  int bits;  // significant bits of its largest key (at least 1)
};

// The sort's launches for digits of BITS bits: `passes` x (count launch, scatter launch), lowest digit first, the
// last scatter writing the index blocks of the messages.
template <int CAP, int BITS>
int sort_passes(SortArgs<CAP>& a, int passes, hipStream_t st) {
  constexpr int kStageBytes = 2 * kSortTile * int(sizeof(uint32_t));
  // The dynamic-LDS limit is a property of the function on one device: raise it once per device.
  static std::mutex attr_mu;
  static uint64_t attr_done = 0;  // bit d: done on device d (devices beyond 63 set it on every call)
  {
    int dev = 0;
    HPX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(attr_mu);
    if (dev >= 64 || !(attr_done >> dev & 1)) {
      HPX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&gd_sort_pass_kernel<CAP, BITS>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kStageBytes));
      if (dev < 64) attr_done |= uint64_t(1) << dev;
    }
  }
  const dim3 grid(uint32_t(a.tile_start[a.nseg]));
  for (int pass = 0; pass < passes; pass++) {
    a.shift = pass * BITS;
    a.parity = pass & 1;
    a.last = pass == passes - 1;
    HPX_LAUNCH("gd_sort_count_kernel", (gd_sort_count_kernel<CAP, BITS>), grid, dim3(kSortThreads), st, a);
    HPX_LAUNCH_LDS("gd_sort_pass_kernel", hpx::g_prof_on, (gd_sort_pass_kernel<CAP, BITS>), grid, dim3(kSortThreads), kStageBytes, st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

// The cut path for up to CAP tensors: the sort over all of them (as many digits as the largest key of any of
// them has; digits of 9 bits where that takes fewer passes than bytes), then one gather launch that adds values
// and headers and clears the residual entries.
template <int CAP>
int sort_and_cut(const CutJob* jobs, int count, hipStream_t st) {
  SortArgs<CAP> a;
  a.nseg = count;
  int bits = 1;
  a.tile_start[0] = 0;
  for (int i = 0; i < count; i++) {
    a.seg[i] = jobs[i].seg;
    a.tile_start[i + 1] = a.tile_start[i] + int32_t(cdiv(jobs[i].seg.n, kSortTile));
    bits = jobs[i].bits > bits ? jobs[i].bits : bits;
  }
  const int bytes = (bits + 7) / 8, nines = (bits + 8) / 9;
  const int rc = nines < bytes ? sort_passes<CAP, 9>(a, nines, st) : sort_passes<CAP, 8>(a, bytes, st);
  if (rc != HPX_OK) return rc;
  for (int i = 0; i < count; i++) {
    const uint32_t k = jobs[i].seg.keep;
    a.tile_start[i + 1] = a.tile_start[i] + int32_t(cdiv(k > 0 ? k : 1, kThreads));
  }
  HPX_LAUNCH("gd_gather_kernel", gd_gather_kernel<CAP>, dim3(uint32_t(a.tile_start[count])), dim3(kThreads), st, a);
  HPX_HIP(hipGetLastError());
  return HPX_OK;
}

// What the host works out per tensor before anything is launched (size arithmetic of gd_body.h:112-115, :153;
// dgc_body.h:79-80, :103).
struct Plan {
  GdSeg seg;
  size_t ws_bytes, cut_bytes;
  int index;  // position in the call
};

// The phases for up to CAP tensors, no host wait.  margin < 0: the threshold from the full gathered sample
// (sample, three histogram passes, rank search), then the pass, scan and expand.  margin >= 0: the provisional
// path (above): provisional threshold, the pass, the samples against the mask, exact threshold, recount, scan, expand.
template <int CAP>
int launch_phases(const Plan* plans, int count, bool residual, int margin, uint32_t* report, hipStream_t st) {
  GdArgs<CAP> a;
  a.nseg = count;
  a.residual = residual ? 1 : 0;
  a.margin = margin;
  a.report = report;
  for (int i = 0; i < count; i++) a.seg[i] = plans[i].seg;
  auto tiles = [&](auto per_tensor) {
    a.tile_start[0] = 0;
    for (int i = 0; i < count; i++) a.tile_start[i + 1] = a.tile_start[i] + int32_t(per_tensor(a.seg[i]));
    return dim3(uint32_t(a.tile_start[count]));
  };
  auto sel_blocks = [](const GdSeg& sg) {
    const uint32_t b = cdiv(sg.sample_cnt, kSelThreads * 8);
    return b > uint32_t(kSelBlocksMax) ? uint32_t(kSelBlocksMax) : b;
  };
  auto stream_pass = [&]() {
    const dim3 g = tiles([](const GdSeg& sg) { return cdiv(sg.n, kTile); });
    if (residual)
      HPX_LAUNCH("gd_stream_kernel", (gd_stream_kernel<true, CAP>), g, dim3(kThreads), st, a);
    else
      HPX_LAUNCH("gd_stream_kernel", (gd_stream_kernel<false, CAP>), g, dim3(kThreads), st, a);
  };
  dim3 grid;
  if (margin < 0) {
    grid = tiles([](const GdSeg& sg) { return cdiv(sg.sample_cnt > uint32_t(kHistWords) ? sg.sample_cnt : uint32_t(kHistWords), kThreads); });
    HPX_LAUNCH("gd_sample_kernel", gd_sample_kernel<CAP>, grid, dim3(kThreads), st, a);
    grid = tiles(sel_blocks);
    HPX_LAUNCH("gd_select_kernel", (gd_select_kernel<1, CAP>), grid, dim3(kSelThreads), st, a);
    HPX_LAUNCH("gd_select_kernel", (gd_select_kernel<2, CAP>), grid, dim3(kSelThreads), st, a);
    HPX_LAUNCH("gd_select_kernel", (gd_select_kernel<3, CAP>), grid, dim3(kSelThreads), st, a);
    HPX_LAUNCH("gd_threshold_kernel", gd_threshold_kernel<CAP>, dim3(uint32_t(count)), dim3(kSelThreads), st, a);
    stream_pass();
  } else {
    grid = tiles([](const GdSeg& sg) { return cdiv(sg.sample_cnt < kPreSamples ? sg.sample_cnt : kPreSamples, kThreads); });
    HPX_LAUNCH("gd_presample_kernel", gd_presample_kernel<CAP>, grid, dim3(kThreads), st, a);
    HPX_LAUNCH("gd_provisional_kernel", gd_provisional_kernel<CAP>, dim3(uint32_t(count)), dim3(kSelThreads), st, a);
    stream_pass();
    grid = tiles([](const GdSeg& sg) { return cdiv(sg.sample_cnt, kThreads); });
    HPX_LAUNCH("gd_resample_kernel", gd_resample_kernel<CAP>, grid, dim3(kThreads), st, a);
    HPX_LAUNCH("gd_exact_kernel", gd_exact_kernel<CAP>, dim3(uint32_t(count)), dim3(kSelThreads), st, a);
    grid = tiles([](const GdSeg& sg) { return cdiv(cdiv(sg.n, kTile), kThreads / kWave); });
    HPX_LAUNCH("gd_recount_kernel", gd_recount_kernel<CAP>, grid, dim3(kThreads), st, a);
  }
  grid = tiles([](const GdSeg& sg) { return cdiv(cdiv(sg.n, kTile), kScanChunk); });
  HPX_LAUNCH("gd_scan_kernel", gd_scan_kernel<CAP>, grid, dim3(kSelThreads), st, a);
  HPX_HIP(hipGetLastError());
  // Queued before the host knows the counts: the finish where nothing has to be cut,
  // else the candidate list and keys of the cut path.
  grid = tiles([](const GdSeg& sg) { return cdiv(cdiv(sg.n, kTile), kExpandPerBlock); });
  HPX_LAUNCH("gd_expand_kernel", gd_expand_kernel<CAP>, grid, dim3(kThreads), st, a);
  HPX_HIP(hipGetLastError());
  return HPX_OK;
}

// Waits until the expand launch has reported every tensor of `count` (the words are in pinned host memory and
// the kernel writes them with system-scope stores as the first thing it does, so they arrive while the stream
// is still busy with that launch).  Polls memory; every 20 us or so it also asks whether the stream has drained, which ends the
// wait if the words can only be seen once the kernels have finished, or if a launch failed.
int wait_reports(volatile uint32_t* report, int count, hipStream_t st) {
  for (int t = 0; t < count; t++) {
    volatile uint32_t* word = report + size_t(t) * kReportWords;
    uint32_t spins = 0;
    auto pending = [word]() { return word[0] == kNotReported || word[1] == kNotReported || word[2] == kNotReported; };
    while (pending()) {
      _mm_pause();
      if ((++spins & 511u) == 0) {
        const hipError_t e = hipStreamQuery(st);
        if (e == hipErrorNotReady) { (void)hipGetLastError(); continue; }
        if (e != hipSuccess) {
          hpx::set_error("sparsifier encode: the stream failed: %s", hipGetErrorString(e));
          return HPX_ERR_HIP;
        }
        if (pending()) {  // everything has run and still no report
          hpx::set_error("sparsifier encode: tensor %d was not reported by the scan launch", t);
          return HPX_ERR_HIP;
        }
      }
    }
  }
  __atomic_thread_fence(__ATOMIC_ACQUIRE);
  return HPX_OK;
}

constexpr int kMaxPerWait = int((hpx::kPinnedFlagOffset) / (kReportWords * sizeof(uint32_t)));  // tensors whose reports fit the pinned block

// `count` tensors.  With residuals (`residuals` non-null): gd_body, s_percent = 1 - drop_ratio.  Without:
// dgc_with_auxiliary_body, where the gradient itself is thresholded and its selected entries cleared.
// A tensor whose parameters make no sense is reported and skipped, like the reference driver's
// print-and-continue; the others are encoded.
int gd_encode_batch(int count, float* const* grads, const int32_t* Ns, float* const* residuals, uint8_t* const* outs,
                    const double* sample_rates, const double* s_percents, const uint64_t* seeds, hpx::Workspace* ws,
                    hipStream_t st) {
  int worst = HPX_OK;
  std::vector<Plan> plans;
  plans.reserve(count);
  size_t ws_total = 0;
  for (int i = 0; i < count; i++) {
    const int32_t N = Ns[i];
    const int32_t sample_cnt = static_cast<int32_t>(std::ceil(N * sample_rates[i]));
    const int32_t expected = static_cast<int32_t>(std::ceil(N * s_percents[i]));
    const int32_t thr_index = static_cast<int32_t>(sample_cnt * s_percents[i]);
    if (!(sample_cnt > 0 && thr_index >= 0 && thr_index < sample_cnt && expected >= 0)) {
      hpx::set_error("sparsifier encode: tensor %d: N=%d sample_rate=%g kept fraction=%g give sample_cnt=%d threshold index=%d", i,
                     N, sample_rates[i], s_percents[i], sample_cnt, thr_index);
      if (worst == HPX_OK) worst = HPX_ERR_ARG;
      continue;
    }
    Plan p;
    const uint32_t n = static_cast<uint32_t>(N);
    // Room for the cut path is laid out for a typical overshoot before anything is
    // launched: the expand kernel fills it without the host knowing the count.
    uint64_t cap64 = uint64_t(expected) * 2 > uint64_t(expected) + 65536 ? uint64_t(expected) * 2 : uint64_t(expected) + 65536;
    if (cap64 > n) cap64 = n;
    const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
    p.seg.g = grads[i];
    p.seg.r = residuals ? residuals[i] : grads[i];
    p.seg.out = outs[i];
    p.seg.ws = nullptr;
    p.seg.cut = nullptr;
    p.seg.n = n;
    p.seg.sample_cnt = static_cast<uint32_t>(sample_cnt);
    p.seg.seed = static_cast<uint32_t>(seed);
    p.seg.thr_index = static_cast<uint32_t>(thr_index);
    p.seg.limit = static_cast<uint32_t>(expected);
    p.seg.cap = static_cast<uint32_t>(cap64);
    p.ws_bytes = gd_layout(n, p.seg.sample_cnt).end;
    p.cut_bytes = cut_layout(cap64).end;
    p.index = i;
    ws_total += p.ws_bytes + p.cut_bytes;
    plans.push_back(p);
  }
  if (plans.empty()) return worst;
  int rc = hpx::ensure_workspace(ws, ws_total);
  if (rc != HPX_OK) return rc;
  {
    size_t at = 0;
    for (Plan& p : plans) {
      p.seg.ws = ws->dev + at;  at += p.ws_bytes;
      p.seg.cut = ws->dev + at; at += p.cut_bytes;
    }
  }
  volatile uint32_t* report = reinterpret_cast<volatile uint32_t*>(ws->pinned);
  const int total = int(plans.size());
  // The provisional path pays where the gather of the full sample is long: from a few hundred thousand samples on.
  uint64_t all_samples = 0;
  for (const Plan& p : plans) all_samples += p.seg.sample_cnt;
  const int64_t prov_min = hpx::option(hpx::kOptGdProvisionalMinSamples);
  const int64_t prov_margin = hpx::option(hpx::kOptGdProvisionalMargin);
  const int margin = (prov_min >= 0 && all_samples >= uint64_t(prov_min) && prov_margin >= 0) ? int(prov_margin > 1000 ? 1000 : prov_margin) : -1;
  auto reset_reports = [&](int n_) {
    for (int t = 0; t < n_; t++)
      for (int w = 0; w < 3; w++) report[size_t(t) * kReportWords + w] = kNotReported;
    __atomic_thread_fence(__ATOMIC_RELEASE);
  };
  for (int first = 0; first < total; first += kMaxPerWait) {
    const int batch = total - first < kMaxPerWait ? total - first : kMaxPerWait;
    reset_reports(batch);
    for (int k = 0; k < batch; k += kCapLarge) {
      const int m = batch - k < kCapLarge ? batch - k : kCapLarge;
      uint32_t* rep = const_cast<uint32_t*>(report) + size_t(k) * kReportWords;
      rc = m <= kCapSmall ? launch_phases<kCapSmall>(&plans[first + k], m, residuals != nullptr, margin, rep, st)
                          : launch_phases<kCapLarge>(&plans[first + k], m, residuals != nullptr, margin, rep, st);
      if (rc != HPX_OK) return rc;
    }
    rc = wait_reports(report, batch, st);
    if (rc != HPX_OK) return rc;
    // What the tensors reported, kept on the host: the pinned words serve again below.
    std::vector<uint32_t> rep_host(size_t(batch) * kReportWords);
    for (size_t w = 0; w < rep_host.size(); w++) rep_host[w] = report[w];
    if (margin >= 0) {
      // Tensors whose provisional threshold was not below the exact one: through the gather path, on the array
      // the pass has already updated (it holds G + R now: sampled and thresholded as it is, nothing added again).
      std::vector<int> fb;
      for (int t = 0; t < batch; t++)
        if (rep_host[size_t(t) * kReportWords] == kFallback) fb.push_back(t);
      if (!fb.empty()) {
        std::vector<Plan> again;
        for (int t : fb) {
          Plan p = plans[first + t];
          p.seg.g = p.seg.r;
          again.push_back(p);
        }
        ws->gd_fallbacks += fb.size();
        reset_reports(int(again.size()));
        for (size_t k = 0; k < again.size(); k += kCapLarge) {
          const int m = int(again.size() - k < size_t(kCapLarge) ? again.size() - k : size_t(kCapLarge));
          uint32_t* rep = const_cast<uint32_t*>(report) + k * kReportWords;
          rc = m <= kCapSmall ? launch_phases<kCapSmall>(&again[k], m, false, -1, rep, st)
                              : launch_phases<kCapLarge>(&again[k], m, false, -1, rep, st);
          if (rc != HPX_OK) return rc;
        }
        rc = wait_reports(report, int(again.size()), st);
        if (rc != HPX_OK) return rc;
        for (size_t j = 0; j < fb.size(); j++)
          for (int w = 0; w < kReportWords; w++) rep_host[size_t(fb[j]) * kReportWords + w] = report[j * kReportWords + w];
      }
    }
    // More candidates than `expected`: order them by |r| descending and keep the first `expected`
    // (gd_body.h:176-187), all such tensors of the batch together.
    std::vector<CutJob> jobs;
    std::vector<int> overflow;   // jobs whose candidates are more than their buffers were laid out for
    size_t aux_need = 0;
    for (int t = 0; t < batch; t++) {
      const GdSeg& sg = plans[first + t].seg;
      const uint32_t found = rep_host[size_t(t) * kReportWords];
      if (found <= sg.limit) continue;
      const uint32_t thr_bits = rep_host[size_t(t) * kReportWords + 1], max_bits = rep_host[size_t(t) * kReportWords + 2];
      // keys are |r| bits minus threshold bits: the largest tells how many byte digits are in use
      const uint32_t max_key = max_bits > thr_bits ? max_bits - thr_bits : 0u;
      CutJob job;
      job.bits = max_key ? 32 - __builtin_clz(max_key) : 1;
      job.seg.msg = sg.out;
      job.seg.r = sg.r;
      job.seg.n = found;
      job.seg.keep = sg.limit;
      job.seg.counts = nullptr;
      if (found > sg.cap) {
        overflow.push_back(int(jobs.size()));
        aux_need += cut_layout(found).end;
        job.seg.keys[0] = reinterpret_cast<uint32_t*>(uintptr_t(first + t));  // the plan, until the block exists
      } else {
        const CutLayout cl = cut_layout(sg.cap);
        job.seg.keys[0] = reinterpret_cast<uint32_t*>(sg.cut + cl.ka);
        job.seg.keys[1] = reinterpret_cast<uint32_t*>(sg.cut + cl.kb);
        job.seg.idx[0] = reinterpret_cast<int32_t*>(sg.cut + cl.ia);
        job.seg.idx[1] = reinterpret_cast<int32_t*>(sg.cut + cl.ib);
        job.seg.counts = reinterpret_cast<uint32_t*>(sg.cut + cl.sc);
      }
      jobs.push_back(job);
    }
    if (!overflow.empty()) {
      // Far more candidates than reserved for: list them again into a block of their own.
      rc = hpx::ensure_aux(ws, aux_need);
      if (rc != HPX_OK) return rc;
      size_t at = 0;
      for (int j : overflow) {
        CutJob& job = jobs[j];
        const Plan& plan = plans[size_t(reinterpret_cast<uintptr_t>(job.seg.keys[0]))];
        const CutLayout cl = cut_layout(job.seg.n);
        uint8_t* cut = ws->aux + at;
        at += cl.end;
        job.seg.keys[0] = reinterpret_cast<uint32_t*>(cut + cl.ka);
        job.seg.keys[1] = reinterpret_cast<uint32_t*>(cut + cl.kb);
        job.seg.idx[0] = reinterpret_cast<int32_t*>(cut + cl.ia);
        job.seg.idx[1] = reinterpret_cast<int32_t*>(cut + cl.ib);
        job.seg.counts = reinterpret_cast<uint32_t*>(cut + cl.sc);
        GdArgs<kCapSmall> a;
        a.nseg = 1;
        a.residual = residuals != nullptr;
        a.margin = -1;
        a.report = nullptr;  // the host has its report
        a.seg[0] = plan.seg;
        a.seg[0].cut = cut;
        a.seg[0].cap = job.seg.n;
        a.seg[0].limit = 0u;
        a.tile_start[0] = 0;
        a.tile_start[1] = int32_t(cdiv(cdiv(plan.seg.n, kTile), kExpandPerBlock));
        HPX_LAUNCH("gd_expand_kernel", gd_expand_kernel<kCapSmall>, dim3(uint32_t(a.tile_start[1])), dim3(kThreads), st, a);
        HPX_HIP(hipGetLastError());
      }
    }
    for (size_t k = 0; k < jobs.size(); k += kCapLarge) {
      const int m = int(jobs.size() - k < size_t(kCapLarge) ? jobs.size() - k : size_t(kCapLarge));
      rc = m <= kCapSmall ? sort_and_cut<kCapSmall>(&jobs[k], m, st) : sort_and_cut<kCapLarge>(&jobs[k], m, st);
      if (rc != HPX_OK) return rc;
    }
  }
  return worst;
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
  std::vector<double> kept(count);
  for (int i = 0; i < count; i++) kept[i] = 1 - drop_ratios[i];  // s_percent, gd_body.h:112
  return gd_encode_batch(count, const_cast<float* const*>(grads), Ns, residuals, outs, sample_rates, kept.data(), seeds, ws, st);
}

HPX_API int64_t hpx_gd_fallbacks(hpx_stream_t stream) {
  hpx::clear_error();
  hpx::Workspace* ws = hpx::workspace_record(static_cast<hipStream_t>(stream));
  if (!ws) return -1;
  std::lock_guard<std::mutex> lock(ws->mu);
  return int64_t(ws->gd_fallbacks);
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
  // the headers are read back into the pinned block, whose last words belong to the barrier kernels' expiry flag
  HPX_ARG(size_t(count) * sizeof(int32_t) <= hpx::kPinnedFlagOffset, "hpx_gd_decode: more than %zu messages in one call",
          hpx::kPinnedFlagOffset / sizeof(int32_t));
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
        HPX_LAUNCH_LDS("gd_zero_kernel", hpx::g_prof_on, gd_zero_kernel, dim3(blocks), dim3(kThreads), hpx::kWriteStreamPadLds3, st, outs[i], n);
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
  return gd_encode_batch(count, grads, Ns, nullptr, outs, sample_rates, s_percents, seeds, ws, st);
}
