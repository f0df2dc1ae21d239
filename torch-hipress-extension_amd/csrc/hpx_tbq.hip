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
  const uint32_t g0 = static_cast<uint32_t>(tile - a.tile_start[s]) * kTileGroups + threadIdx.x;

  if (g0 - threadIdx.x + kTileGroups <= full) {
    float4 gv[kIters], rv[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const size_t e = size_t(g0 + k * kThreads) * 4;
      gv[k] = ld4_stream(gp + e);
      rv[k] = ld4_stream(rp + e);
    }
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const uint32_t grp = g0 + k * kThreads;
      const uint32_t q = tbq_code4(gv[k], rv[k], thr);
      st4_stream(rp + size_t(grp) * 4, rv[k]);
      op[grp] = static_cast<uint8_t>(q);
    }
    return;
  }
  // Last tile of the tensor: bounds-checked, and the lane owning the partial
  // group leaves the fields past the end at code 1.
#pragma unroll
  for (int k = 0; k < kIters; k++) {
    const uint32_t grp = g0 + k * kThreads;
    const size_t e = size_t(grp) * 4;
    if (grp < full) {
      float4 gv = ld4(gp + e), rv = ld4(rp + e);
      const uint32_t q = tbq_code4(gv, rv, thr);
      st4(rp + e, rv);
      op[grp] = static_cast<uint8_t>(q);
    } else if (grp == full && (n & 3)) {
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

template <bool ADD>
__device__ __forceinline__ void tbq_decode_tile(const DecSeg& sg, uint32_t g0, bool stream_store) {
  float* __restrict__ op = sg.out;
  const uint8_t* __restrict__ ip = sg.in;
  const uint32_t n = static_cast<uint32_t>(sg.n);
  const float thr = sg.thr;
  const uint32_t full = n >> 2;
  if (g0 - threadIdx.x + kTileGroups <= full) {
    uint32_t q[kIters];
    float4 acc[kIters];
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const uint32_t grp = g0 + k * kThreads;
      q[k] = ip[grp];
      if (ADD) acc[k] = ld4_stream(op + size_t(grp) * 4);
    }
#pragma unroll
    for (int k = 0; k < kIters; k++) {
      const uint32_t grp = g0 + k * kThreads;
      float4 v = tbq_values(q[k], thr);
      if (ADD) {
        v.x += acc[k].x; v.y += acc[k].y; v.z += acc[k].z; v.w += acc[k].w;
        st4_stream(op + size_t(grp) * 4, v);  // in-place update: streaming store
      } else if (stream_store) {
        st4_stream(op + size_t(grp) * 4, v);
      } else {
        st4(op + size_t(grp) * 4, v);
      }
    }
    return;
  }
#pragma unroll
  for (int k = 0; k < kIters; k++) {
    const uint32_t grp = g0 + k * kThreads;
    const size_t e = size_t(grp) * 4;
    if (grp < full) {
      float4 v = tbq_values(ip[grp], thr);
      if (ADD) {
        const float4 o = ld4(op + e);
        v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
      }
      st4(op + e, v);
    } else if (grp == full && (n & 3)) {
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
  const uint32_t g0 = static_cast<uint32_t>(tile - a.tile_start[s]) * kTileGroups + threadIdx.x;
  if (a.seg[s].add)
    tbq_decode_tile<true>(a.seg[s], g0, true);
  else
    tbq_decode_tile<false>(a.seg[s], g0, a.stream_store != 0);
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
        const int32_t t = tiles_for(n);
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;  // next launch
        a.seg[a.nseg] = EncSeg{grads[i], residuals[i], outs[i], n, thresholds[i]};
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
      }
      i++;
    }
    if (a.nseg == 0) continue;
    HPX_LAUNCH("tbq_encode_kernel", tbq_encode_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), st, a);
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
    while (i < count && a.nseg < CAP) {
      const int32_t n = sizes[i];
      HPX_ARG(n >= 0, "hpx_tbq_decode: tensor %d has negative size %d", i, n);
      if (n > 0) {
        HPX_ARG(outs[i] && ins[i], "hpx_tbq_decode: tensor %d has a null pointer", i);
        const int32_t t = tiles_for(n);
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;
        a.seg[a.nseg] = DecSeg{outs[i], ins[i], n, thresholds[i], is_add_tos[i] != 0, 0};
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
      }
      i++;
    }
    if (a.nseg == 0) continue;
    HPX_LAUNCH("tbq_decode_kernel", tbq_decode_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), st, a);
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
  if (count <= kCapSmall) return launch_decode<kCapSmall>(count, outs, sizes, ins, thresholds, is_add_tos, st);
  return launch_decode<kCapLarge>(count, outs, sizes, ins, thresholds, is_add_tos, st);
}
