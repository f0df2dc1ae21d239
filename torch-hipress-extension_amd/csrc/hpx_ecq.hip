// ECQ: error-compensated b-bit quantiser with a history H (b in {2, 4, 8}).
//
// The reference holds this codec as a body without driver or caller
// (ecq_body.h:157-286 encode, :342-423 decode).  As written it keeps its
// |G + alpha*H| scratch at the start of the output buffer and writes the packed
// bytes over it from byte 10 while later elements are still to be read, and its
// quantise loop leaves the last payload byte alone.  Under the device or OpenMP
// policy that is a race; under the serial policy it is deterministic, and that
// behaviour is what these kernels reproduce bit for bit, computing |G + alpha*H|
// where it is needed instead of keeping it in the output buffer:
//
//   max        one pass: max over x of float(fabs(double(G[x]) + alpha*double(H[x])))
//   quantise   one pass: byte x < M - 1 (M = ceil(N / dpb)) draws from the reference's
//              LCG seeded with seed + x; per element f = (gh + max) * gap_inverse,
//              code = uint8(f + u), H = float(beta*H + (f - code)*gap); codes are
//              OR-ed LSB-first.  If max < 1e-6 the bytes are 0 and H *= beta.
//
// What the aliasing does in the serial order, and is reproduced: a payload byte
// stored at 10 + x lands in scratch element (10 + x) / 4, which for 4-bit codes
// (element 2) and 8-bit codes (elements 2 and 3) has not been read yet, so those
// elements are read with the stored byte(s) in them: the first four bytes are
// worked out by one lane over a 16-byte copy of the scratch; the LAST payload byte
// is never written by the loop and keeps byte (9 + M) % 4 of scratch element
// (9 + M) / 4 if that element exists (else the caller's byte stays), and the
// history of the last byte's elements stays as it was.
// Codes come out of |.|, so every decoded value is >= 0: the reference's ECQ loses
// the sign, and so does this one.
#include <climits>
#include <cmath>
#include <cstring>

#include "hpx_common.h"

namespace {
using namespace hpx;

constexpr int kThreads = 256;
constexpr int kMaxTile = kThreads * 16;   // elements per workgroup of the max pass
constexpr int kWays = 128;                // words a tensor's workgroups fold their maxima into
constexpr int kBytesPerLane = 4;          // payload bytes per lane of the quantise pass

struct EcqArgs {
  const float* g;
  float* h;
  uint8_t* out;
  uint32_t* ways;   // kWays words, zero before the max pass
  double alpha, beta;
  uint32_t n;
  uint32_t seed;    // low 32 bits of seed (+ byte index) reach the LCG
  int32_t bits;
};

// fabs(G + alpha*H) as the reference computes and stores it (ecq_body.h:58): double arithmetic, kept as float.
__device__ __forceinline__ float gh_of(float g, float h, double alpha) {
  return static_cast<float>(fabs(static_cast<double>(g) + alpha * static_cast<double>(h)));
}

__global__ __launch_bounds__(kThreads) void ecq_clear_kernel(uint32_t* __restrict__ p, uint32_t words) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i < words) p[i] = 0u;
}

__global__ __launch_bounds__(kThreads) void ecq_max_kernel(const EcqArgs a) {
  const uint32_t n = a.n;
  const uint32_t e0 = blockIdx.x * uint32_t(kMaxTile);
  float m = 0.0f;  // the values are >= 0
  if (n - e0 >= uint32_t(kMaxTile)) {
    float4 gv[4], hv[4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      gv[k] = ld4(a.g + size_t(e0) + size_t(k * kThreads + threadIdx.x) * 4);
      hv[k] = ld4(a.h + size_t(e0) + size_t(k * kThreads + threadIdx.x) * 4);
    }
#pragma unroll
    for (int k = 0; k < 4; k++) {
      m = __builtin_fmaxf(m, gh_of(gv[k].x, hv[k].x, a.alpha));
      m = __builtin_fmaxf(m, gh_of(gv[k].y, hv[k].y, a.alpha));
      m = __builtin_fmaxf(m, gh_of(gv[k].z, hv[k].z, a.alpha));
      m = __builtin_fmaxf(m, gh_of(gv[k].w, hv[k].w, a.alpha));
    }
  } else {
    for (uint32_t e = e0 + threadIdx.x; e < n; e += kThreads) m = __builtin_fmaxf(m, gh_of(a.g[e], a.h[e], a.alpha));
  }
  uint32_t mb = __float_as_uint(m);  // non-negative floats order like their bit patterns
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { const uint32_t v = __shfl_xor(mb, o, kWave); mb = v > mb ? v : mb; }
  __shared__ uint32_t s_m[kThreads / kWave];
  if ((threadIdx.x & (kWave - 1)) == 0) s_m[threadIdx.x / kWave] = mb;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t v = s_m[0];
    for (int i = 1; i < kThreads / kWave; i++) v = s_m[i] > v ? s_m[i] : v;
    atomicMax(a.ways + (blockIdx.x % kWays), v);
  }
}

// static_cast<uint8_t>(float) as the reference's x86-64 build performs it: truncation to int32 (NaN and values
// outside int32 give 0x80000000), low byte kept.  Inside [0, 256) that is the C++ conversion; outside it C++ leaves
// the result open, and the body gets there when scratch elements 2 and 3 are read back with payload bytes in them.
__device__ __forceinline__ uint32_t u8_of_float_x86(float v) {
  const int32_t i = (v >= -2147483648.0f && v < 2147483648.0f) ? static_cast<int32_t>(v) : INT32_MIN;
  return static_cast<uint32_t>(i) & 0xFFu;
}

// One payload byte: dpb elements starting at element `head`; gh[] are their scratch values.  Returns the byte
// and updates the history (ecq_body.h:105-131).
template <int B>
__device__ __forceinline__ uint32_t ecq_byte(const float (&gh)[8 / B], float (&h)[8 / B], float max_gh, float gap,
                                             float gap_inverse, double beta, uint32_t seed_plus_x) {
  constexpr int DPB = 8 / B;
  uint32_t q = 0;
  uint32_t x = seed_plus_x;
  x = kLcgA * x + kLcgC;  // srand discards one draw
#pragma unroll
  for (int j = 0; j < DPB; j++) {
    x = kLcgA * x + kLcgC;
    const float u = static_cast<float>(static_cast<double>(x) / 4294967295.0);
    const float f = (gh[j] + max_gh) * gap_inverse;
    const uint32_t t = u8_of_float_x86(f + u);  // uint8(f + r()), :117
    q |= (t << (B * j)) & 0xFFu;
    h[j] = static_cast<float>(beta * static_cast<double>(h[j]) + static_cast<double>((f - static_cast<float>(t)) * gap));
  }
  return q;
}

template <int B>
__global__ __launch_bounds__(kThreads) void ecq_quant_kernel(const EcqArgs a) {
  constexpr int DPB = 8 / B;
  __shared__ uint32_t s_max;
  if (threadIdx.x < kWave) {
    uint32_t v = 0;
    for (int w = threadIdx.x; w < kWays; w += kWave) { const uint32_t t = a.ways[w]; v = t > v ? t : v; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { const uint32_t t = __shfl_xor(v, o, kWave); v = t > v ? t : v; }
    if (threadIdx.x == 0) s_max = v;
  }
  __syncthreads();
  const float max_gh = __uint_as_float(s_max);
  const uint32_t n = a.n;
  const uint32_t M = (n + DPB - 1) / DPB;
  const uint32_t loop_bytes = M - 1;  // the reference's loop leaves the last byte alone (:222, :240)
  const float s = static_cast<float>((1 << (B - 1)) - 1);
  const bool zero = max_gh < 1e-6;  // float against the double constant, as :206
  const float gap = max_gh / s;
  const float gap_inverse = static_cast<float>(1.0 / static_cast<double>(gap));
  uint8_t* __restrict__ Q = a.out + 10;
  // The last payload byte keeps what the scratch held at byte 9 + M: byte (9 + M) % 4 of |G + alpha*H| of element
  // (9 + M) / 4, taken BEFORE any history update.  The lane that owns that element's byte stores it.
  const uint64_t keep_pos = uint64_t(9) + M;
  const bool keep = keep_pos < uint64_t(4) * n;
  const uint32_t keep_elem = uint32_t(keep_pos >> 2);

  if (blockIdx.x == 0 && threadIdx.x == 0) {
    // header (:262-272)
    const int32_t out_true_size = int32_t(10 + M);
    const uint32_t mb = __float_as_uint(max_gh);
    for (int i = 0; i < 4; i++) {
      a.out[i] = uint8_t(uint32_t(out_true_size) >> (8 * i));
      a.out[4 + i] = uint8_t(mb >> (8 * i));
    }
    a.out[8] = uint8_t(B);
    a.out[9] = uint8_t(M * DPB - n);
    // Bytes 0..3 in the serial order, over a copy of the first 16 bytes of the scratch: a byte stored at 10 + x
    // changes scratch element (10 + x) / 4 before it is read (4-bit codes: element 2; 8-bit codes: 2 and 3).
    uint32_t scratch[4];
    for (uint32_t e = 0; e < 4; e++) scratch[e] = e < n ? __float_as_uint(gh_of(a.g[e], a.h[e], a.alpha)) : 0u;
    for (uint32_t x = 0; x < 4 && x < M; x++) {
      float gh[DPB], h[DPB];
      for (int j = 0; j < DPB; j++) {
        const uint32_t e = x * DPB + j;
        h[j] = e < n ? a.h[e] : 0.0f;
        gh[j] = e < 4 ? __uint_as_float(scratch[e]) : (e < n ? gh_of(a.g[e], h[j], a.alpha) : 0.0f);
        if (keep && e == keep_elem && e >= 4) a.out[keep_pos] = uint8_t(__float_as_uint(gh[j]) >> (8 * (keep_pos & 3)));
      }
      uint32_t q = 0;
      if (zero) {  // update_H_with_0 covers all N elements (:216-225), the last byte's too
        for (int j = 0; j < DPB; j++) h[j] = static_cast<float>(static_cast<double>(h[j]) * a.beta);
      } else if (x < loop_bytes) {
        q = ecq_byte<B>(gh, h, max_gh, gap, gap_inverse, a.beta, a.seed + x);
      }
      if (zero || x < loop_bytes)
        for (int j = 0; j < DPB; j++)
          if (x * DPB + j < n) a.h[x * DPB + j] = h[j];
      if (x < loop_bytes) {
        Q[x] = uint8_t(q);
        const uint32_t at = 10 + x;
        if (at < 16) scratch[at >> 2] = (scratch[at >> 2] & ~(0xFFu << (8 * (at & 3)))) | (q << (8 * (at & 3)));
      }
    }
    // (a kept byte below position 16 is one the loop never stores to, so the copy still holds the original)
    if (keep && keep_elem < 4) a.out[keep_pos] = uint8_t(scratch[keep_elem] >> (8 * (keep_pos & 3)));
  }

#pragma unroll
  for (int k = 0; k < kBytesPerLane; k++) {
    const uint32_t x = blockIdx.x * uint32_t(kThreads * kBytesPerLane) + k * kThreads + threadIdx.x;
    if (x < 4 || x >= M) continue;  // bytes 0..3: done above
    float gh[DPB], h[DPB];
    const size_t e0 = size_t(x) * DPB;
#pragma unroll
    for (int j = 0; j < DPB; j++) {
      const bool in = e0 + j < n;  // only the last byte can reach past the end
      h[j] = in ? a.h[e0 + j] : 0.0f;
      gh[j] = in ? gh_of(a.g[e0 + j], h[j], a.alpha) : 0.0f;
      if (keep && e0 + j == keep_elem) a.out[keep_pos] = uint8_t(__float_as_uint(gh[j]) >> (8 * (keep_pos & 3)));
    }
    if (zero) {
#pragma unroll
      for (int j = 0; j < DPB; j++)
        if (e0 + j < n) a.h[e0 + j] = static_cast<float>(static_cast<double>(h[j]) * a.beta);
      if (x < loop_bytes) Q[x] = 0;
      continue;
    }
    if (x >= loop_bytes) continue;  // the last byte: not quantised, its history left as it was
    const uint32_t q = ecq_byte<B>(gh, h, max_gh, gap, gap_inverse, a.beta, a.seed + x);
#pragma unroll
    for (int j = 0; j < DPB; j++) a.h[e0 + j] = h[j];
    Q[x] = uint8_t(q);
  }
}

struct EcqDecArgs {
  const uint8_t* in;
  float* out;
  uint32_t n;       // elements to write
  float max_abs;
  int32_t bits;
  int32_t add;
};

__global__ __launch_bounds__(kThreads) void ecq_decode_kernel(const EcqDecArgs a) {
  const uint32_t bits = uint32_t(a.bits), dpb = 8u / bits, mask = (1u << bits) - 1u;
  const float s = static_cast<float>((1 << (a.bits - 1)) - 1);
  const float gap = a.max_abs / s;
  const uint8_t* __restrict__ Q = a.in + 10;
  const uint32_t stride = gridDim.x * kThreads;
  for (uint32_t x = blockIdx.x * kThreads + threadIdx.x; x < a.n; x += stride) {
    const uint32_t q = (uint32_t(Q[x / dpb]) >> ((x % dpb) * bits)) & mask;
    const float v = static_cast<float>(int(q)) * gap - a.max_abs;  // qval*gap - max_abs_G, :302
    a.out[x] = a.add ? a.out[x] + v : v;                           // G[x] += ..., :332
  }
}

inline uint32_t cdiv(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }

}  // namespace

HPX_API int hpx_ecq_encode(int count, const float* const* Gs, const int32_t* Ns, float* const* Hs, uint8_t* const* outs,
                           const int32_t* out_sizes, const double* alphas, const double* betas, const int32_t* bitwidths,
                           const uint64_t* seeds, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_ecq_encode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(Gs && Ns && Hs && outs && out_sizes && alphas && betas && bitwidths, "hpx_ecq_encode: null argument array");
  for (int i = 0; i < count; i++) {
    const int32_t b = bitwidths[i];
    if (b != 2 && b != 4 && b != 8) {  // the reference aborts here (ecq_body.h:172-175)
      hpx::set_error("bitwidth's range: {2,4,8}\tInput bitwidth=%d", b);
      return HPX_ERR_BODY;
    }
    HPX_ARG(Ns[i] > 0, "hpx_ecq_encode: tensor %d has size %d (must be positive)", i, Ns[i]);
    HPX_ARG(Gs[i] && Hs[i] && outs[i], "hpx_ecq_encode: tensor %d has a null pointer", i);
    const int64_t need = 10 + (int64_t(Ns[i]) + 8 / b - 1) / (8 / b);
    HPX_ARG(out_sizes[i] >= need, "hpx_ecq_encode: tensor %d needs %lld output bytes, got %d", i, static_cast<long long>(need),
            out_sizes[i]);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the workspace may have to grow (a wait for the stream, hipFree, hipMalloc): not something a graph can record
  if (const int rcc = hpx::reject_capture(st, "hpx_ecq_encode")) return rcc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  const size_t words = size_t(count) * kWays;
  int rc = hpx::ensure_workspace(ws, words * sizeof(uint32_t));
  if (rc != HPX_OK) return rc;
  uint32_t* ways = reinterpret_cast<uint32_t*>(ws->dev);
  HPX_LAUNCH("ecq_clear_kernel", ecq_clear_kernel, dim3(cdiv(words, kThreads)), dim3(kThreads), st, ways, uint32_t(words));
  for (int i = 0; i < count; i++) {
    const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
    EcqArgs a{Gs[i], Hs[i], outs[i], ways + size_t(i) * kWays, alphas[i], betas[i], static_cast<uint32_t>(Ns[i]),
              static_cast<uint32_t>(seed), bitwidths[i]};
    HPX_LAUNCH("ecq_max_kernel", ecq_max_kernel, dim3(cdiv(a.n, kMaxTile)), dim3(kThreads), st, a);
    const uint32_t M = cdiv(a.n, 8 / a.bits);
    const dim3 grid(cdiv(M, kThreads * kBytesPerLane));
    switch (a.bits) {
      case 2: HPX_LAUNCH("ecq_quant_kernel", ecq_quant_kernel<2>, grid, dim3(kThreads), st, a); break;
      case 4: HPX_LAUNCH("ecq_quant_kernel", ecq_quant_kernel<4>, grid, dim3(kThreads), st, a); break;
      default: HPX_LAUNCH("ecq_quant_kernel", ecq_quant_kernel<8>, grid, dim3(kThreads), st, a); break;
    }
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

HPX_API int hpx_ecq_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes, float* const* outs,
                           const int32_t* out_sizes, const int32_t* is_add_tos, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_ecq_decode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(ins && in_sizes && outs && out_sizes && is_add_tos, "hpx_ecq_decode: null argument array");
  HPX_ARG(size_t(count) * 16 <= hpx::kPinnedFlagOffset, "hpx_ecq_decode: more than %zu messages in one call", hpx::kPinnedFlagOffset / 16);
  for (int i = 0; i < count; i++)
    HPX_ARG(ins[i] && outs[i] && in_sizes[i] >= 10 && out_sizes[i] >= 0, "hpx_ecq_decode: message %d: null pointer, or fewer than 10 bytes", i);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const int rcc = hpx::reject_capture(st, "hpx_ecq_decode")) return rcc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int rc = hpx::ensure_workspace(ws, 0);
  if (rc != HPX_OK) return rc;
  // headers first, one wait, as the reference copies them to the host (ecq_body.h:352-358)
  uint8_t* heads = ws->pinned;
  for (int i = 0; i < count; i++) HPX_HIP(hipMemcpyAsync(heads + size_t(i) * 16, ins[i], 10, hipMemcpyDeviceToHost, st));
  HPX_HIP(hipStreamSynchronize(st));
  for (int i = 0; i < count; i++) {
    const uint8_t* hd = heads + size_t(i) * 16;
    int32_t used;
    float max_abs;
    std::memcpy(&used, hd, 4);
    std::memcpy(&max_abs, hd + 4, 4);
    const int32_t bits = hd[8], unused = hd[9];
    if (bits != 2 && bits != 4 && bits != 8) {
      hpx::set_error("hpx_ecq_decode: message %d has bitwidth %d", i, bits);
      return HPX_ERR_BODY;
    }
    HPX_ARG(used >= 10 && used <= in_sizes[i], "hpx_ecq_decode: message %d says %d bytes, %d provided", i, used, in_sizes[i]);
    const int64_t N = int64_t(used - 10) * (8 / bits) - unused;
    if (out_sizes[i] < N) {  // the reference aborts here (ecq_body.h:386-390)
      hpx::set_error("Output space too small: out_float_size < N.  %d vs. %lld", out_sizes[i], static_cast<long long>(N));
      return HPX_ERR_BODY;
    }
    if (N <= 0) continue;
    EcqDecArgs a{ins[i], outs[i], static_cast<uint32_t>(N), max_abs, bits, is_add_tos[i] != 0};
    uint32_t blocks = cdiv(uint64_t(N), kThreads * 4);
    if (blocks > 65536) blocks = 65536;
    HPX_LAUNCH("ecq_decode_kernel", ecq_decode_kernel, dim3(blocks), dim3(kThreads), st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}
