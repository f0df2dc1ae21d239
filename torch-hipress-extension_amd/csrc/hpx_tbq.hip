// TBQ: threshold quantisation with residual feedback, 2-bit codes, 4 per byte.
//
// Semantics follow the reference's `compress` functor (tbq_body.h:57-88) and
// its decoders (tbq_body.h:22-55).  Both directions are pure streams: each
// lane owns one 4-element group (one packed byte) per step and a wave touches
// 1 KiB of contiguous gradient per load instruction.  A whole bucket of
// tensors is described by a table passed in the kernel-argument segment, so a
// call needs no device-side setup, no workspace and no host synchronisation;
// the partial last group of a tensor is packed in the same kernel (the
// reference round-trips it through the host, tbq_body.h:114-155).
#include <unordered_map>
#include <vector>

#include "hpx_common.h"

namespace {
using namespace hpx;

constexpr int kThreads = 256;
constexpr int kIters = 4;                           // groups per lane
constexpr int kTileGroups = kThreads * kIters;      // 1024 bytes of codes
constexpr int kCapLarge = 256;  // 9 KiB of kernel arguments: a 200-tensor bucket is one launch
constexpr int kCapSmall = 8;    // calls with a few tensors pass a table of a few hundred bytes

struct EncSeg {
  const float* g;
  float* r;
  uint8_t* out;
  int32_t n;
  float thr;
};
template <int CAP>
struct EncArgs {
  int32_t nseg;
  int32_t tile_start[CAP + 1];
  EncSeg seg[CAP];
};
struct DecSeg {
  float* out;
  const uint8_t* in;
  int32_t n;
  float thr;
  int32_t add;
  int32_t pad;
};
template <int CAP>
struct DecArgs {
  int32_t nseg;
  int32_t stream_store;  // see kStreamStoreMaxBytes
  int32_t tile_start[CAP + 1];
  DecSeg seg[CAP];
};
static_assert(sizeof(EncArgs<kCapLarge>) <= 9600 && sizeof(DecArgs<kCapLarge>) <= 9600, "kernel-argument budget");

struct __attribute__((packed, aligned(1))) u32u {
  uint32_t v;
};

// One element of the reference rule; returns the 2-bit code.
__device__ __forceinline__ uint32_t tbq_code(float g, float& r, float thr) {
  r += g;
  uint32_t c = 1;
  if (r >= thr) {
    c = 2;
    r -= thr;
  } else if (r <= -thr) {
    c = 0;
    r += thr;
  }
  return c;
}

__device__ __forceinline__ uint32_t tbq_code4(const float4& g, float4& r, float thr) {
  uint32_t q = tbq_code(g.x, r.x, thr);
  q |= tbq_code(g.y, r.y, thr) << 2;
  q |= tbq_code(g.z, r.z, thr) << 4;
  q |= tbq_code(g.w, r.w, thr) << 6;
  return q;
}

// Tiles are laid on absolute addresses: a workgroup's 16 KiB of residual (encode) or output (decode)
// starts on a 16 KiB boundary whatever the tensor's base address is, because a tile that straddles such a
// boundary streams measurably slower (7 % at an offset of 8 KiB).  The groups before the first boundary,
// `head` of them, form a short first tile.  Host and kernels use the same two functions.
__host__ __device__ inline uint32_t tbq_head_groups(const void* p, uint32_t total_groups) {
  const uint32_t to_boundary = (16384u - (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)) & 16383u)) & 16383u;
  const uint32_t h = (to_boundary + 15u) >> 4;  // groups of 16 bytes
  return h >= total_groups ? 0u : h;
}
__host__ __device__ inline uint32_t tbq_tiles(const void* p, uint32_t n) {
  const uint32_t total = (n + 3u) >> 2;
  const uint32_t head = tbq_head_groups(p, total);
  return (head ? 1u : 0u) + (total - head + uint32_t(kTileGroups) - 1u) / uint32_t(kTileGroups);
}
// Groups [gbeg, glim) of tile t (glim may lie past the end of the tensor for its last tile).
__device__ __forceinline__ void tbq_tile_range(const void* p, uint32_t n, uint32_t t, uint32_t& gbeg, uint32_t& glim) {
  const uint32_t head = tbq_head_groups(p, (n + 3u) >> 2);
  if (head && t == 0) {
    gbeg = 0;
    glim = head;
  } else {
    gbeg = head + (t - (head ? 1u : 0u)) * uint32_t(kTileGroups);
    glim = gbeg + uint32_t(kTileGroups);
  }
}

template <int CAP>
__global__ __launch_bounds__(kThreads) void tbq_encode_kernel(const EncArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const float* __restrict__ gp = a.seg[s].g;
  float* __restrict__ rp = a.seg[s].r;
  uint8_t* __restrict__ op = a.seg[s].out;
  const uint32_t n = static_cast<uint32_t>(a.seg[s].n);
  const float thr = a.seg[s].thr;
  const uint32_t full = n >> 2;  // complete groups
  uint32_t gbeg, glim;
  tbq_tile_range(rp, n, static_cast<uint32_t>(tile - a.tile_start[s]), gbeg, glim);
  const uint32_t g0 = gbeg + threadIdx.x;

  if (glim - gbeg == uint32_t(kTileGroups) && glim <= full) {
    // Whole tile inside the tensor.  A wave owns kIters * 64 consecutive groups, i.e. 256 consecutive
    // bytes of codes, and writes them as ONE dword per lane (a 256-byte store per wave) instead of four
    // single-byte stores per lane.
    static_assert(kIters == 4, "the code gather below pairs the four steps with the four lanes of a quad");
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t gw = g0 - threadIdx.x + (threadIdx.x / kWave) * uint32_t(kIters * kWave);  // the wave's first group
    float4 gv[kIters], rv[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const size_t e = size_t(gw + k * kWave + lane) * 4;
      gv[k] = ld4_stream(gp + e);
      rv[k] = ld4_stream(rp + e);
    }
    uint32_t d[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      uint32_t b = tbq_code4(gv[k], rv[k], thr) << (8 * (lane & 3));
      st4_stream(rp + size_t(gw + k * kWave + lane) * 4, rv[k]);
      b |= __shfl_xor(b, 1, kWave);
      b |= __shfl_xor(b, 2, kWave);
      d[k] = b;  // every lane of quad m: the four bytes of groups gw + 64k + 4m .. +3, i.e. dword 16k + m of the wave
    }
    // Lane 4m + k of a quad offers dword 16k + m; lane l fetches dword l from lane 4 (l % 16) + l / 16.
    const uint32_t i = lane & 3;
    const uint32_t offer = i == 0 ? d[0] : i == 1 ? d[1] : i == 2 ? d[2] : d[3];
    const uint32_t dw = __shfl(offer, int(4 * (lane & 15) + (lane >> 4)), kWave);
    reinterpret_cast<u32u*>(op + gw + 4 * lane)->v = dw;  // messages start at any byte
    return;
  }
  // First (short) or last tile of the tensor: bounds-checked, and the lane owning the
  // partial group leaves the fields past the end at code 1.  All loads first: the last
  // tile of the last tensor is the tail of the launch.
  const uint32_t lim = glim < full ? glim : full;  // complete groups of this tile end here
  float4 gt[kIters], rt[kIters];
#pragma unroll
  for (int k = 0; k < kIters; k++) {
    const uint32_t grp = g0 + k * kThreads;
    if (grp < lim) {
      gt[k] = ld4(gp + size_t(grp) * 4);
      rt[k] = ld4(rp + size_t(grp) * 4);
    }
  }
#pragma unroll
  for (int k = 0; k < kIters; k++) {
    const uint32_t grp = g0 + k * kThreads;
    const size_t e = size_t(grp) * 4;
    if (grp < lim) {
      float4 gv = gt[k], rv = rt[k];
      const uint32_t q = tbq_code4(gv, rv, thr);
      st4(rp + e, rv);
      op[grp] = static_cast<uint8_t>(q);
    } else if (grp == full && grp < glim && (n & 3)) {
      uint32_t q = 85;
      for (uint32_t j = 0; j < (n & 3); j++) {
        float r = rp[e + j];
        const uint32_t c = tbq_code(gp[e + j], r, thr);
        rp[e + j] = r;
        q = (q & ~(3u << (2 * j))) | (c << (2 * j));
      }
      op[grp] = static_cast<uint8_t>(q);
    }
  }
}

__device__ __forceinline__ float4 tbq_values(uint32_t q, float thr) {
  // (float(code) - 1) * thr, tbq_body.h:36
  return make_float4((static_cast<float>(q & 3) - 1) * thr, (static_cast<float>((q >> 2) & 3) - 1) * thr,
                     (static_cast<float>((q >> 4) & 3) - 1) * thr, (static_cast<float>((q >> 6) & 3) - 1) * thr);
}

// STREAM: the stores of a written (not added-to) tensor carry the non-temporal hint.  A template parameter and not
// a run-time flag: with both kinds of store in one function the compiler folds them into one plain store.
template <bool ADD, bool STREAM>
__device__ __forceinline__ void tbq_decode_tile(const DecSeg& sg, uint32_t t) {
  float* __restrict__ op = sg.out;
  const uint8_t* __restrict__ ip = sg.in;
  const uint32_t n = static_cast<uint32_t>(sg.n);
  const float thr = sg.thr;
  const uint32_t full = n >> 2;
  uint32_t gbeg, glim;
  tbq_tile_range(op, n, t, gbeg, glim);
  const uint32_t g0 = gbeg + threadIdx.x;
  if (glim - gbeg == uint32_t(kTileGroups) && glim <= full) {
    // Whole tile inside the tensor.  A wave owns kIters * 64 consecutive groups - 4 KiB of the tensor, 256
    // consecutive bytes of codes, which it fetches with ONE load (a dword per lane); the lanes pick their
    // bytes out of it with cross-lane reads.  (A byte load per group and lane, the workgroup walking the
    // tile 4 KiB at a time, took 84 us for 110 M elements where this takes 66.)
    static_assert(kIters * kWave == kWave * 4, "a wave fetches exactly 256 code bytes, one dword per lane: four groups of four elements per lane");
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t gw = gbeg + (threadIdx.x / kWave) * uint32_t(kIters * kWave);  // the wave's first group
    const uint32_t dw = as_global(reinterpret_cast<const u32u*>(ip + gw + lane * 4))->v;  // messages start at any byte
    float4 acc[kIters];
    if (ADD) {
#pragma unroll
      for (int k = 0; k < kIters; k++) acc[k] = ld4_stream(op + size_t(gw + k * kWave + lane) * 4);
    }
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const uint32_t q = (__shfl(dw, k * (kWave / 4) + lane / 4, kWave) >> (8 * (lane & 3))) & 0xFFu;
      float4 v = tbq_values(q, thr);
      float* o = op + size_t(gw + k * kWave + lane) * 4;
      if (ADD) {
        v.x += acc[k].x; v.y += acc[k].y; v.z += acc[k].z; v.w += acc[k].w;
      }
      if (ADD || STREAM) st4_stream(o, v); else st4(o, v);  // an in-place update always streams
      __asm__ volatile("" ::: "memory");  // one store per step, in order
    }
    return;
  }
  const uint32_t lim = glim < full ? glim : full;  // complete groups of this (first or last) tile end here
  uint32_t qt[kIters];
  float4 ot[kIters];
#pragma unroll
  for (int k = 0; k < kIters; k++) {  // all loads first: the last tile of the last tensor is the tail of the launch
    const uint32_t grp = g0 + k * kThreads;
    if (grp < lim) {
      qt[k] = ip[grp];
      if (ADD) ot[k] = ld4(op + size_t(grp) * 4);
    }
  }
#pragma unroll
  for (int k = 0; k < kIters; k++) {
    const uint32_t grp = g0 + k * kThreads;
    const size_t e = size_t(grp) * 4;
    if (grp < lim) {
      float4 v = tbq_values(qt[k], thr);
      if (ADD) {
        const float4 o = ot[k];
        v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
      }
      st4(op + e, v);
    } else if (grp == full && grp < glim && (n & 3)) {
      const uint32_t q = ip[grp];
      for (uint32_t j = 0; j < (n & 3); j++) {
        const float v = (static_cast<float>((q >> (2 * j)) & 3) - 1) * thr;
        op[e + j] = ADD ? v + op[e + j] : v;
      }
    }
  }
}

template <int CAP>
__global__ __launch_bounds__(kThreads) void tbq_decode_kernel(const DecArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const uint32_t t = static_cast<uint32_t>(tile - a.tile_start[s]);
  if (a.seg[s].add)
    tbq_decode_tile<true, true>(a.seg[s], t);
  else if (a.stream_store)
    tbq_decode_tile<false, true>(a.seg[s], t);
  else
    tbq_decode_tile<false, false>(a.seg[s], t);
}

// ---- several messages into one tensor ---------------------------------------
// The reference's root path hands tbq_r_body the same output tensor once per
// gathered message (hp_cuda.cpp:241-259, is_add_to = 1) and the messages are
// applied one after the other.  Here all messages of a tensor are applied in one
// pass: the tensor is read once, every message contributes its byte per group in
// call order (same sequence of fp32 additions, so the sums are bit-identical),
// and the tensor is written once.
constexpr int kMultiSegs = 64;
constexpr int kMultiSlots = 448;
constexpr int kMultiSlotsPerSeg = 32;  // a tensor's messages are staged in LDS; more of them go to a later launch
struct MSeg {
  float* out;
  int32_t n;
  int32_t first_slot;
  int32_t nslots;
  int32_t pad;
};
struct MSlot {
  const uint8_t* in;
  float thr;
  int32_t add;
};
struct MArgs {
  int32_t nseg;
  int32_t tile_start[kMultiSegs + 1];
  MSeg seg[kMultiSegs];
  MSlot slot[kMultiSlots];
};
static_assert(sizeof(MArgs) <= 9600, "kernel-argument budget");
// The same for tensors whose messages lie at a fixed distance from each other, share one threshold and are all
// added (the first one may also overwrite): the gathered slots of the reference's communication buffer
// (hp_cuda.cpp:241-259), of which the root leaves out its own - one gap of twice the distance is part of the form.  A tensor then takes 40 bytes of table whatever its number of messages, and a bucket of
// 200 tensors with 7 messages each is ONE launch instead of four.
constexpr int kStrideSegs = 208;
struct SSeg {
  float* out;
  const uint8_t* in0;  // the first message
  int64_t stride;      // bytes from one message to the next
  int32_t n;
  float thr;
  int16_t nslots;
  int16_t add0;        // the first message is added to what the tensor holds
  int16_t skip;        // messages from this one on lie one distance further (the root's own slot is left out); -1: none
  int16_t pad;
};
struct SArgs {
  int32_t nseg;
  int32_t tile_start[kStrideSegs + 1];
  SSeg seg[kStrideSegs];
};
static_assert(sizeof(SSeg) == 40 && sizeof(SArgs) <= 9600, "kernel-argument budget");

// What the two tables have in common for the kernel: the tensor of a tile, and its messages in LDS.
__device__ __forceinline__ int multi_segment(const MArgs& a, int tile) { return find_segment<kMultiSegs>(a.tile_start, a.nseg, tile); }
__device__ __forceinline__ int multi_segment(const SArgs& a, int tile) { return find_segment<kStrideSegs>(a.tile_start, a.nseg, tile); }
__device__ __forceinline__ int multi_slots(const MArgs& a, int s, const uint8_t** s_in, float* s_thr, int32_t* s_add) {
  const int s0 = a.seg[s].first_slot, ns = a.seg[s].nslots;
  if (int(threadIdx.x) < ns) {
    s_in[threadIdx.x] = a.slot[s0 + threadIdx.x].in;
    s_thr[threadIdx.x] = a.slot[s0 + threadIdx.x].thr;
    s_add[threadIdx.x] = a.slot[s0 + threadIdx.x].add;
  }
  return ns;
}
__device__ __forceinline__ int multi_slots(const SArgs& a, int s, const uint8_t** s_in, float* s_thr, int32_t* s_add) {
  const int ns = a.seg[s].nslots;
  if (int(threadIdx.x) < ns) {
    const int skip = a.seg[s].skip;
    s_in[threadIdx.x] = a.seg[s].in0 + int64_t(int(threadIdx.x) + ((skip >= 0 && int(threadIdx.x) >= skip) ? 1 : 0)) * a.seg[s].stride;
    s_thr[threadIdx.x] = a.seg[s].thr;
    s_add[threadIdx.x] = threadIdx.x == 0 ? int32_t(a.seg[s].add0) : 1;
  }
  return ns;
}

template <typename Args>
__global__ __launch_bounds__(kThreads) void tbq_decode_multi_kernel(const Args a) {
  __shared__ const uint8_t* s_in[kMultiSlotsPerSeg];
  __shared__ float s_thr[kMultiSlotsPerSeg];
  __shared__ int32_t s_add[kMultiSlotsPerSeg];
  const int tile = blockIdx.x;
  const int s = multi_segment(a, tile);
  float* __restrict__ op = a.seg[s].out;
  const uint32_t n = static_cast<uint32_t>(a.seg[s].n);
  const int ns = multi_slots(a, s, s_in, s_thr, s_add);
  __syncthreads();
  const bool need_old = s_add[0] != 0;
  const uint32_t full = n >> 2;
  const uint32_t g0 = static_cast<uint32_t>(tile - a.tile_start[s]) * kTileGroups + threadIdx.x;
  if (g0 - threadIdx.x + kTileGroups <= full) {
    // Whole tile inside the tensor.  A wave owns kIters * 64 consecutive groups, i.e. that many
    // consecutive bytes of every message: each message costs the wave ONE load (a dword per lane)
    // and the lanes pick their bytes out of it with cross-lane reads, instead of one byte load per
    // group and message (28 loads per lane for 7 messages; the address pipeline, not memory,
    // was the limit).  The old values and up to 8 messages are requested together, then folded in
    // message order.
    static_assert(kIters * kWave == kWave * 4, "a wave fetches exactly 256 code bytes of a message, one dword per lane");
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t gw = g0 - threadIdx.x + (threadIdx.x / kWave) * uint32_t(kIters * kWave);  // the wave's first group
    float4 acc[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++)
      acc[k] = need_old ? ld4_stream(op + size_t(gw + k * kWave + lane) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j0 = 0; j0 < ns; j0 += 8) {
      uint32_t dw[8];
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        dw[jj] = 0u;
        if (j0 + jj < ns && lane < uint32_t(kIters * kWave / 4)) {
          dw[jj] = as_global(reinterpret_cast<const u32u*>(s_in[j0 + jj] + gw + lane * 4))->v;  // messages start at any byte
        }
      }
      uint32_t q[8][kIters];
#pragma unroll
      for (int jj = 0; jj < 8; jj++)
#pragma unroll
        for (int k = 0; k < kIters; k++)
          q[jj][k] = (__shfl(dw[jj], k * (kWave / 4) + lane / 4, kWave) >> (8 * (lane & 3))) & 0xFFu;
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        if (j0 + jj < ns) {
          const float thr = s_thr[j0 + jj];
          const bool add = s_add[j0 + jj] != 0;
#pragma unroll
          for (int k = 0; k < kIters; k++) {
            const float4 v = tbq_values(q[jj][k], thr);
            if (add) {
              acc[k].x = v.x + acc[k].x; acc[k].y = v.y + acc[k].y; acc[k].z = v.z + acc[k].z; acc[k].w = v.w + acc[k].w;
            } else {
              acc[k] = v;
            }
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      st4_stream(op + size_t(gw + k * kWave + lane) * 4, acc[k]);
      __asm__ volatile("" ::: "memory");
    }
    return;
  }
  // The tile that holds the end of the tensor.  Its whole groups are handled like the ones above, one byte
  // load per group and message, with the loads of all of a lane's groups and of up to 8 messages in flight
  // together; only the last, partial group goes element by element.  (Done element by element for the whole
  // tile, every element waited for its own loads, message after message: up to 16 x (1 + messages) memory
  // latencies in a row in ONE workgroup, tens of microseconds that the rest of the grid could not hide.)
  float4 acc[kIters];
  bool live[kIters];
#pragma unroll
  for (int k = 0; k < kIters; k++) {
    const uint32_t grp = g0 + k * kThreads;
    live[k] = grp < full;
    acc[k] = (live[k] && need_old) ? ld4(op + size_t(grp) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  for (int j0 = 0; j0 < ns; j0 += 8) {
    uint32_t q[8][kIters];
#pragma unroll
    for (int jj = 0; jj < 8; jj++)
#pragma unroll
      for (int k = 0; k < kIters; k++) {
        q[jj][k] = 85u;
        if (j0 + jj < ns && live[k]) q[jj][k] = as_global(s_in[j0 + jj])[g0 + k * kThreads];
      }
#pragma unroll
    for (int jj = 0; jj < 8; jj++) {
      if (j0 + jj < ns) {
        const float thr = s_thr[j0 + jj];
        const bool add = s_add[j0 + jj] != 0;
#pragma unroll
        for (int k = 0; k < kIters; k++) {
          const float4 v = tbq_values(q[jj][k], thr);
          if (add) {
            acc[k].x = v.x + acc[k].x; acc[k].y = v.y + acc[k].y; acc[k].z = v.z + acc[k].z; acc[k].w = v.w + acc[k].w;
          } else {
            acc[k] = v;
          }
        }
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kIters; k++)
    if (live[k]) st4(op + size_t(g0 + k * kThreads) * 4, acc[k]);
  // the partial group, if the tensor has one and it belongs to this lane
  const uint32_t rest = n & 3u;
  if (rest && full >= g0 && (full - g0) % kThreads == 0 && (full - g0) / kThreads < uint32_t(kIters)) {
    const size_t e = size_t(full) * 4;
    float tail[3];
    for (uint32_t i = 0; i < rest; i++) tail[i] = need_old ? op[e + i] : 0.f;
    for (int j = 0; j < ns; j++) {
      const uint32_t q = as_global(s_in[j])[full];
      const float thr = s_thr[j];
      const bool add = s_add[j] != 0;
      for (uint32_t i = 0; i < rest; i++) {
        const float v = (static_cast<float>((q >> (2 * i)) & 3) - 1) * thr;
        tail[i] = add ? v + tail[i] : v;
      }
    }
    for (uint32_t i = 0; i < rest; i++) op[e + i] = tail[i];
  }
}

inline int32_t tiles_for(int32_t n) {
  const int64_t groups = (int64_t(n) + 3) >> 2;
  return static_cast<int32_t>((groups + kTileGroups - 1) / kTileGroups);
}

template <int CAP>
int launch_encode(int count, const float* const* grads, const int32_t* sizes, float* const* residuals,
                  uint8_t* const* outs, const float* thresholds, hipStream_t st) {
  EncArgs<CAP> a;
  int i = 0;
  while (i < count) {
    a.nseg = 0;
    a.tile_start[0] = 0;
    while (i < count && a.nseg < CAP) {
      const int32_t n = sizes[i];
      HPX_ARG(n >= 0, "hpx_tbq_encode: tensor %d has negative size %d", i, n);
      if (n > 0) {
        HPX_ARG(grads[i] && residuals[i] && outs[i], "hpx_tbq_encode: tensor %d has a null pointer", i);
        const int32_t t = static_cast<int32_t>(tbq_tiles(residuals[i], static_cast<uint32_t>(n)));
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;  // next launch
        a.seg[a.nseg] = EncSeg{grads[i], residuals[i], outs[i], n, thresholds[i]};
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
      }
      i++;
    }
    if (a.nseg == 0) continue;
    // A bucket's launch is held to three workgroups per CU (unused LDS, hpx_common.h): with the 256-entry table every
    // workgroup starts with a search, and fewer of them at a time serve the stream better (200 tensors, 110 M
    // elements: 214 -> 207 us); a launch of a few tensors is left as it is (201 us either way).
    const int pad = CAP > kCapSmall ? hpx::kWriteStreamPadLds3 : 0;
    HPX_LAUNCH_LDS("tbq_encode_kernel", hpx::g_prof_on, tbq_encode_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), pad, st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

template <int CAP>
int launch_decode(int count, float* const* outs, const int32_t* sizes, const uint8_t* const* ins,
                  const float* thresholds, const int32_t* is_add_tos, hipStream_t st) {
  DecArgs<CAP> a;
  size_t out_bytes = 0;
  for (int k = 0; k < count; k++) out_bytes += sizes[k] > 0 ? size_t(sizes[k]) * 4 : 0;
  a.stream_store = out_bytes <= hpx::stream_store_max_bytes();
  int i = 0;
  while (i < count) {
    a.nseg = 0;
    a.tile_start[0] = 0;
    bool any_add = false;
    while (i < count && a.nseg < CAP) {
      const int32_t n = sizes[i];
      HPX_ARG(n >= 0, "hpx_tbq_decode: tensor %d has negative size %d", i, n);
      if (n > 0) {
        HPX_ARG(outs[i] && ins[i], "hpx_tbq_decode: tensor %d has a null pointer", i);
        const int32_t t = static_cast<int32_t>(tbq_tiles(outs[i], static_cast<uint32_t>(n)));
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;
        a.seg[a.nseg] = DecSeg{outs[i], ins[i], n, thresholds[i], is_add_tos[i] != 0, 0};
        any_add = any_add || is_add_tos[i] != 0;
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
      }
      i++;
    }
    if (a.nseg == 0) continue;
    // write mode throughout: a pure write stream, held to three workgroups per CU (hpx_common.h)
    const int pad = (a.stream_store && !any_add) ? hpx::kWriteStreamPadLds3 : 0;
    HPX_LAUNCH_LDS("tbq_decode_kernel", hpx::g_prof_on, tbq_decode_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), pad, st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

// Plans the launches of a multi-message decode.  Messages are visited in call order; each launch takes up to
// kMultiSegs tensors and up to kMultiSlotsPerSeg messages per tensor (kMultiSlots in all).  A message that does not
// fit is left for a later launch together with every later message of the same tensor, so the messages of a tensor
// are always applied in call order (launches are ordered by the stream); tensors do not overlap, so the order
// between different tensors is immaterial.
struct MultiGroup {
  float* out;
  int32_t n;
  std::vector<int> msgs;
};
template <typename TilesFn>
std::vector<MultiGroup> plan_multi_launch(int count, float* const* outs, const int32_t* sizes, std::vector<char>& done,
                                          TilesFn tiles_of) {
  std::vector<MultiGroup> groups;
  std::unordered_map<float*, int> index;  // tensor -> group, or -1 once the tensor is closed for this launch
  int used_slots = 0;
  int64_t tiles = 0;
  for (int j = 0; j < count; j++) {
    if (done[j]) continue;
    auto it = index.find(outs[j]);
    if (it != index.end()) {
      if (it->second < 0) continue;
      MultiGroup& g = groups[it->second];
      if (used_slots == kMultiSlots || int(g.msgs.size()) == kMultiSlotsPerSeg) { it->second = -1; continue; }
      g.msgs.push_back(j);
    } else {
      if (used_slots == kMultiSlots || int(groups.size()) == kMultiSegs || tiles + tiles_of(sizes[j]) > INT32_MAX) {
        index[outs[j]] = -1;
        continue;
      }
      index[outs[j]] = int(groups.size());
      groups.push_back(MultiGroup{outs[j], sizes[j], {j}});
      tiles += tiles_of(sizes[j]);
    }
    used_slots++;
    done[j] = 1;
  }
  return groups;
}

// Fills the table of the fixed-distance form when the whole call fits it: at most kStrideSegs tensors, every
// tensor's messages (in call order) at one distance from each other, with one threshold, and all but the first
// added.  Arguments have been checked.
bool plan_strided(int count, float* const* outs, const int32_t* sizes, const uint8_t* const* ins, const float* thresholds,
                  const int32_t* is_add_tos, SArgs& a) {
  std::unordered_map<float*, int> index;
  std::vector<const uint8_t*> last(kStrideSegs, nullptr);
  a.nseg = 0;
  for (int j = 0; j < count; j++) {
    if (sizes[j] == 0) continue;
    auto it = index.find(outs[j]);
    if (it == index.end()) {
      if (a.nseg == kStrideSegs) return false;
      index[outs[j]] = a.nseg;
      a.seg[a.nseg] = SSeg{outs[j], ins[j], 0, sizes[j], thresholds[j], 1, int16_t(is_add_tos[j] != 0), -1, 0};
      last[a.nseg] = ins[j];
      a.nseg++;
      continue;
    }
    SSeg& g = a.seg[it->second];
    const int64_t step = static_cast<int64_t>(reinterpret_cast<intptr_t>(ins[j]) - reinterpret_cast<intptr_t>(last[it->second]));  // addresses, not elements of one array
    if (g.nslots == kMultiSlotsPerSeg || is_add_tos[j] == 0 || thresholds[j] != g.thr || sizes[j] != g.n) return false;
    if (g.nslots == 1) g.stride = step;
    else if (step == g.stride) {}
    else if (g.skip < 0 && step == 2 * g.stride) g.skip = g.nslots;                                   // the gap
    else if (g.skip < 0 && g.nslots == 2 && 2 * step == g.stride) { g.stride = step; g.skip = 1; }    // the gap came first
    else return false;
    last[it->second] = ins[j];
    g.nslots++;
  }
  int64_t tiles = 0;
  a.tile_start[0] = 0;
  for (int k = 0; k < a.nseg; k++) {
    tiles += tiles_for(a.seg[k].n);
    if (tiles > INT32_MAX) return false;
    a.tile_start[k + 1] = int32_t(tiles);
  }
  return a.nseg > 0;
}

int launch_decode_multi(int count, float* const* outs, const int32_t* sizes, const uint8_t* const* ins,
                        const float* thresholds, const int32_t* is_add_tos, hipStream_t st) {
  std::vector<char> done(count, 0);
  int left = 0;
  for (int j = 0; j < count; j++) {
    HPX_ARG(sizes[j] >= 0, "hpx_tbq_decode: tensor %d has negative size %d", j, sizes[j]);
    if (sizes[j] == 0) { done[j] = 1; continue; }
    HPX_ARG(outs[j] && ins[j], "hpx_tbq_decode: tensor %d has a null pointer", j);
    left++;
  }
  if (left == 0) return HPX_OK;
  {
    SArgs sa;
    if (plan_strided(count, outs, sizes, ins, thresholds, is_add_tos, sa)) {
      HPX_LAUNCH("tbq_decode_multi_kernel", tbq_decode_multi_kernel<SArgs>, dim3(sa.tile_start[sa.nseg]), dim3(kThreads), st, sa);
      HPX_HIP(hipGetLastError());
      return HPX_OK;
    }
  }
  MArgs a;
  while (left > 0) {
    const std::vector<MultiGroup> groups = plan_multi_launch(count, outs, sizes, done, tiles_for);
    a.nseg = 0;
    a.tile_start[0] = 0;
    int nslots = 0;
    for (const MultiGroup& g : groups) {
      a.seg[a.nseg] = MSeg{g.out, g.n, nslots, static_cast<int32_t>(g.msgs.size()), 0};
      for (int m : g.msgs) a.slot[nslots++] = MSlot{ins[m], thresholds[m], is_add_tos[m] != 0};
      a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + tiles_for(g.n);
      a.nseg++;
    }
    if (nslots == 0) { hpx::set_error("hpx_tbq_decode: could not place the remaining messages"); return HPX_ERR_ARG; }
    left -= nslots;
    HPX_LAUNCH("tbq_decode_multi_kernel", tbq_decode_multi_kernel<MArgs>, dim3(a.tile_start[a.nseg]), dim3(kThreads), st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

}  // namespace

HPX_API int hpx_tbq_encode(int count, const float* const* grads, const int32_t* sizes,
                           float* const* residuals, uint8_t* const* outs, const float* thresholds,
                           hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_tbq_encode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(grads && sizes && residuals && outs && thresholds, "hpx_tbq_encode: null argument array");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (count <= kCapSmall) return launch_encode<kCapSmall>(count, grads, sizes, residuals, outs, thresholds, st);
  return launch_encode<kCapLarge>(count, grads, sizes, residuals, outs, thresholds, st);
}

HPX_API int hpx_tbq_decode(int count, float* const* outs, const int32_t* sizes,
                           const uint8_t* const* ins, const float* thresholds,
                           const int32_t* is_add_tos, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_tbq_decode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(outs && sizes && ins && thresholds && is_add_tos, "hpx_tbq_decode: null argument array");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (hpx::classify_outputs(count, outs, sizes)) {
    case 0: break;
    case 1:  // several messages accumulate into the same tensor(s): one pass per tensor
      return launch_decode_multi(count, outs, sizes, ins, thresholds, is_add_tos, st);
    default: {  // partially overlapping outputs: keep the reference's one-message-at-a-time order
      for (int i = 0; i < count; i++) {
        const int rc = launch_decode<kCapSmall>(1, outs + i, sizes + i, ins + i, thresholds + i, is_add_tos + i, st);
        if (rc != HPX_OK) return rc;
      }
      return HPX_OK;
    }
  }
  if (count <= kCapSmall) return launch_decode<kCapSmall>(count, outs, sizes, ins, thresholds, is_add_tos, st);
  return launch_decode<kCapLarge>(count, outs, sizes, ins, thresholds, is_add_tos, st);
}
