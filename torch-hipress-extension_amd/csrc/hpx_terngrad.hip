// TernGrad path: b-bit uniform min/max quantiser (b in {1,2,4,8}) with optional
// stochastic rounding, 10-byte header, codes packed LSB-first.
//
// Semantics follow terngrad_body.h:162-307 (encode) and :309-409 (decode).
// Encode is three launches with no host round trip: a min/max reduction to
// per-tile partials; one workgroup per tensor that folds them, derives the
// scalars (gap, 1/gap) on the device and writes the header; then the
// quantise-and-pack stream.  Decode parses the header on the device.
//
// Bit-exactness notes
//   * (x - min) * gi + u is three separately rounded fp32 operations (the
//     library is built with -ffp-contract=off).
//   * gi = float(1.0 / (double(gap) + 1e-8)), terngrad_body.h:206.
//   * The reference seeds its LCG per output byte with seed + byte index and
//     draws once per slot after one discarded draw (terngrad_body.h:88-96), so
//     slot j of byte i uses x = A_{j+2} * (seed + i) + C_{j+2}: a lane stepping
//     through bytes at a fixed stride advances each draw by a constant.
//   * u = float(double(x) / 4294967295.0) is evaluated without fp64 (which
//     runs at a quarter of the fp32 rate and made the quantise pass
//     ALU-bound): with A = float(x & ~0xFF) and lo = float(x & 0xFF),
//     u = (A + fma(A, 0x1.ffff88p-33, lo)) * 2^-32 for all 2^32 inputs
//     (checked exhaustively on the CPU).  A + lo alone is RNE(x); the fused
//     term adds the quotient's excess over x * 2^-32, which turns ties into
//     round-up, and the constant is chosen so that the two inputs where the
//     fp64 quotient itself lands on a tie (0xFFFFFD7F, 0xFFFFFF7F) come out
//     as the reference's double rounding leaves them.
//   * min and max are the FIRST smallest / largest element as
//     thrust::minmax_element returns them, which only matters for the sign of
//     a zero extreme; it is recovered from the first zero of the tensor.
#include <atomic>
#include <cstdlib>
#include <mutex>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "hpx_common.h"

// Reduction slots of hpx_terngrad_encode_noalloc: 192 tensors x 3 x 128 words of 8 bytes = 576 KiB, held by
// every GPU the library runs on until the process ends.  In host code this name only stands for the
// symbol; the device address comes from hipGetSymbolAddress (scratch_address below).
static __device__ __align__(256) unsigned long long scratch[192 * 3 * 128];

namespace {
using namespace hpx;

constexpr int kThreads = 256;
constexpr int kCapLarge = 192;  // tensors per launch table (about 7 KiB of kernel arguments)
constexpr int kCapSmall = 8;    // calls with a few tensors pass a table of a few hundred bytes
constexpr int kRedIters = 4;                                 // float4 loads per lane (16 KiB per workgroup: with 8 the
                                                             // pass over 25.5 M elements took 28 us instead of 24.6, with 16: 39.6)
constexpr int kRedTile = kThreads * kRedIters * 4;           // 4096 elements
constexpr int kQIters = 4;                                   // units per lane
constexpr int kDIters = 4;                                   // 4-element groups per lane in decode
constexpr int kDecTile = kThreads * kDIters * 4;

// Per tensor, 3 x kSlotWays epoch-tagged slots: first the largest ordered key of x, then the
// largest complemented key (i.e. the minimum), then the largest complemented
// index of a tile that holds a zero (i.e. the first such tile).
constexpr int kSlotWays = 128;  // a multiple of 64 (the size of `scratch` above is written out from this and kCapLarge); with 64 the min/max pass over one 25.5 M tensor took 24.1 us, with 128 or 256: 20.2
constexpr int kSlotsPerTensor = 3 * kSlotWays;

struct EncSeg {
  const float* x;
  uint8_t* out;
  int32_t n;
  int32_t out_size;
  uint32_t seed;  // only the low 32 bits of seed + byte index reach the LCG
  uint8_t bits;
  uint8_t random;
  uint16_t pad;
};
template <int CAP>
struct EncArgs {
  int32_t nseg;
  int32_t tile_start[CAP + 1];
  EncSeg seg[CAP];
  uint64_t* slots;      // kSlotsPerTensor words per segment of this launch
  uint32_t epoch;       // tag of this call; slots carrying an older tag are stale
};
struct __attribute__((packed, aligned(1))) u32u {
  uint32_t v;
};
struct DecSeg {
  float* out;
  const uint8_t* in;
  int32_t out_size;
  int32_t in_size;
  int32_t add;
  int32_t pad;
};
template <int CAP>
struct DecArgs {
  int32_t nseg;
  int32_t stream_store;  // see kStreamStoreMaxBytes
  int32_t tile_start[CAP + 1];
  DecSeg seg[CAP];
  uint32_t* status;
};
static_assert(sizeof(EncArgs<kCapLarge>) <= 9600 && sizeof(DecArgs<kCapLarge>) <= 9600, "kernel-argument budget");

// Reductions over the 64 lanes of a wave through the lane-permuting forms of the move instruction (no LDS
// round trips): within quads, within rows of 16, then row 0 into row 1 and row 2 into row 3, then rows 0-1
// into rows 2-3; lane 63 holds the result and hands it to every lane.
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
  static_assert(sizeof(T) == 4, "32-bit values");
  auto perm = [](T x, auto ctrl, auto rows) {
    const int xi = __builtin_bit_cast(int, x);
    // lanes whose row is not named keep their own value
    return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(xi, xi, decltype(ctrl)::value, decltype(rows)::value, 0xF, false));
  };
  using std::integral_constant;
  v = op(v, perm(v, integral_constant<int, 0xB1>{}, integral_constant<int, 0xF>{}));   // quad_perm [1,0,3,2]
  v = op(v, perm(v, integral_constant<int, 0x4E>{}, integral_constant<int, 0xF>{}));   // quad_perm [2,3,0,1]
  v = op(v, perm(v, integral_constant<int, 0x141>{}, integral_constant<int, 0xF>{}));  // row_half_mirror
  v = op(v, perm(v, integral_constant<int, 0x140>{}, integral_constant<int, 0xF>{}));  // row_mirror
  v = op(v, perm(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{}));  // row_bcast:15 into rows 1 and 3
  v = op(v, perm(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{}));  // row_bcast:31 into rows 2 and 3
  return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_min(float v) {
  return wave_reduce(v, [](float a, float b) { return b < a ? b : a; });
}
__device__ __forceinline__ float wave_max(float v) {
  return wave_reduce(v, [](float a, float b) { return b > a ? b : a; });
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
  return wave_reduce(v, [](uint32_t a, uint32_t b) { return b < a ? b : a; });
}

// Block-wide (min, max, min-u32) over 4 waves.  Result valid in every thread.
__device__ __forceinline__ void block_reduce(float& mn, float& mx, uint32_t& z) {
  __shared__ float s_mn[kThreads / kWave], s_mx[kThreads / kWave];
  __shared__ uint32_t s_z[kThreads / kWave];
  mn = wave_min(mn);
  mx = wave_max(mx);
  z = wave_min_u32(z);
  const int w = threadIdx.x / kWave;
  __syncthreads();  // protects reuse of the shared arrays between calls
  if ((threadIdx.x & (kWave - 1)) == 0) { s_mn[w] = mn; s_mx[w] = mx; s_z[w] = z; }
  __syncthreads();
  mn = s_mn[0]; mx = s_mx[0]; z = s_z[0];
#pragma unroll
  for (int i = 1; i < kThreads / kWave; i++) {
    mn = s_mn[i] < mn ? s_mn[i] : mn;
    mx = s_mx[i] > mx ? s_mx[i] : mx;
    z = s_z[i] < z ? s_z[i] : z;
  }
}

__device__ __forceinline__ void acc3(float v, float& mn, float& mx, float& am) {
  mn = v < mn ? v : mn;
  mx = v > mx ? v : mx;
  const float a = __builtin_fabsf(v);
  am = a < am ? a : am;
}

// Three-operand minimum / maximum: one instruction for two elements, where the comparison-and-select
// form above costs the compiler three issue slots per element (compare, a wait for the condition, select).
// A NaN operand is ignored, as the comparisons ignore it; which zero wins among +0 and -0 does not matter,
// because the sign of a zero extreme is settled from the first zero of the tensor.
__device__ __forceinline__ float vmin3(float a, float b, float c) {
  float r;
  __asm__("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float vmax3(float a, float b, float c) {
  float r;
  __asm__("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float vmin3_abs(float a, float b, float c) {  // min(a, |b|, |c|)
  float r;
  __asm__("v_min3_f32 %0, %1, |%2|, |%3|" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// 16 bytes per lane from global memory straight into LDS, without passing through registers: lane i's
// piece lands at lds_wave_base + 16 * i (the base must be the same in every lane); lanes that are switched
// off leave their 16 bytes of LDS as they were.  The load counts as a vector-memory load (vmcnt) and returns
// in order with the others; the address needs 4-byte alignment only.  Non-temporal, like ld4_stream.
//
// Written out as instructions, so that the compiler does not know of it: told of loads into LDS in flight,
// it makes every LDS access wait for all of them, and every use of an ordinary load that follows them too
// (it no longer trusts the order of returns), which serialises the whole pass.  Unaware of them, its counted
// waits for the ordinary loads stay right as long as these loads are requested BEFORE those (returns are in
// order, so a wait for "at most N younger loads outstanding" also covers everything older).  The caller
// answers for the rest: wait_vector_loads() before anything reads the LDS the loads fill.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is reserved, and naming it is still how the compiler learns that it changes
__device__ __forceinline__ void ld4_stream_to_lds(const float* p, float4* lds_wave_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)lds_wave_base)));
  __asm__ volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(p), "s"(base) : "memory", "m0");
}
#pragma clang diagnostic pop
// Waits for every vector-memory load of the wave, LDS-bound ones included.
__device__ __forceinline__ void wait_vector_loads() { __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// A row of a register ring: requested into the very registers that held the row before (the operand is tied, so the
// register allocator has no choice to make and nothing to spill), and waited for by count.  The compiler does not
// know that the registers are written later than the request: between ring_request(row) and ring_wait(row) the row
// must not be touched, and ring_wait's count must not exceed the number of vector-memory instructions that are
// certain to have been issued after the request (loads and stores complete in the order of their issue).
typedef float ring_f32x4 __attribute__((ext_vector_type(4)));
template <int OFFSET>
__device__ __forceinline__ void ring_request(float4& row, const float* uniform_base, uint32_t byte_offset) {
  ring_f32x4 t = {row.x, row.y, row.z, row.w};
  __asm__ volatile("global_load_dwordx4 %0, %1, %2 offset:%3 nt ; ring request" : "+v"(t) : "v"(byte_offset), "s"(uniform_base), "n"(OFFSET) : "memory");
  row = make_float4(t.x, t.y, t.z, t.w);
}
template <int COUNT>
__device__ __forceinline__ void ring_wait(float4& row) {
  ring_f32x4 t = {row.x, row.y, row.z, row.w};
  __asm__ volatile("s_waitcnt vmcnt(%1) ; ring wait %0" : "+v"(t) : "n"(COUNT) : "memory");
  row = make_float4(t.x, t.y, t.z, t.w);
}

// min, max and min |x| over four elements: six instructions.
__device__ __forceinline__ void acc3x4(const float4& v, float& mn, float& mx, float& am) {
  mn = vmin3(mn, v.x, v.y); mx = vmax3(mx, v.x, v.y); am = vmin3_abs(am, v.x, v.y);
  mn = vmin3(mn, v.z, v.w); mx = vmax3(mx, v.z, v.w); am = vmin3_abs(am, v.z, v.w);
}

// Order-preserving map of a float onto unsigned integers, and back.
__device__ __forceinline__ uint32_t okey(float f) {
  const uint32_t b = __float_as_uint(f);
  return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ float from_okey(uint32_t k) {
  return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xFFFFFFFFu));
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  return wave_reduce(v, [](uint32_t a, uint32_t b) { return b > a ? b : a; });
}

// Pass 1 of encode.  Each workgroup reduces one kRedTile-element tile and folds its
// result into one of kSlotWays slots of its tensor with a 64-bit atomic max on
// (epoch << 32 | key).  Tiles spread over the slots, so about n_tiles/kSlotWays atomics
// meet on one address over the whole run of the kernel (same-address atomics
// from different workgroups cost ~37 ns each), and because a newer epoch beats
// any older word the slots are never cleared.  The quantise kernel folds the
// slots itself, so no separate reduction launch is needed.
template <int CAP>
__global__ __launch_bounds__(kThreads) void terngrad_minmax_kernel(const EncArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const float* __restrict__ xp = a.seg[s].x;
  const uint32_t n = static_cast<uint32_t>(a.seg[s].n);
  const uint32_t t = static_cast<uint32_t>(tile - a.tile_start[s]);
  const uint32_t e0 = t * uint32_t(kRedTile);

  float mn = __builtin_inff(), mx = -__builtin_inff(), am = __builtin_inff();
  if (n - e0 >= uint32_t(kRedTile)) {
    float4 v[kRedIters];
#pragma unroll
    for (int k = 0; k < kRedIters; k++) v[k] = ld4(xp + size_t(e0) + size_t(k * kThreads + threadIdx.x) * 4);
#pragma unroll
    for (int k = 0; k < kRedIters; k++) acc3x4(v[k], mn, mx, am);
  } else {
    for (uint32_t e = e0 + threadIdx.x; e < n; e += kThreads) acc3(xp[e], mn, mx, am);
  }
  uint32_t z = (am == 0.0f) ? 0u : 1u;  // 0 when this tile holds a zero
  block_reduce(mn, mx, z);
  if (threadIdx.x == 0) {
    unsigned long long* sl = reinterpret_cast<unsigned long long*>(a.slots) + size_t(s) * kSlotsPerTensor + (t % kSlotWays);
    const unsigned long long ep = static_cast<unsigned long long>(a.epoch) << 32;
    atomicMax(sl, ep | okey(mx));
    atomicMax(sl + kSlotWays, ep | (~okey(mn)));
    if (z == 0u) atomicMax(sl + 2 * kSlotWays, ep | (0xFFFFFFFFu - t));
  }
}

// 1 / (gap + 1e-8) in fp64, rounded to fp32 (terngrad_body.h:204-206).
__device__ __forceinline__ float inverse_gap(float mn, float mx, uint32_t bits) {
  const float gap = (mx - mn) / (float(1 << bits) - 1.0f);
  return static_cast<float>(1.0 / (static_cast<double>(gap) + 1e-8));
}

// The 10-byte header: bitwidth, tail, min, max (terngrad_body.h:219-224).
__device__ __forceinline__ void write_header(uint8_t* o, uint32_t bits, uint32_t n, float mn, float mx) {
  const uint32_t dpb = 8u / bits;
  uint32_t tail = n % dpb;
  tail = tail == 0 ? 0 : dpb - tail;
  const uint32_t mb = __float_as_uint(mn), xb = __float_as_uint(mx);
  o[0] = uint8_t(bits);
  o[1] = uint8_t(tail);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    o[2 + i] = uint8_t(mb >> (8 * i));
    o[6 + i] = uint8_t(xb >> (8 * i));
  }
}

// Prologue of the quantise kernel: folds the tensor's slots into min and max
// (thrust::minmax_element semantics: a zero extreme takes the sign of the first
// zero element of the tensor), derives gap and 1/(gap + 1e-8) as the reference
// does (terngrad_body.h:204-206) and, in the workgroup of the tensor's first tile,
// writes the 10-byte header (terngrad_body.h:219-224).  Every workgroup repeats
// this; it reads 3 KB from L2.
template <int CAP>
__device__ __forceinline__ void load_scalars(const EncArgs<CAP>& a, int s, bool first_tile, float& mn_out, float& gi_out) {
  __shared__ uint32_t s_k[3];
  const float* __restrict__ xp = a.seg[s].x;
  const uint32_t n = static_cast<uint32_t>(a.seg[s].n);
  if (threadIdx.x < kWave) {
    const unsigned long long* sl = reinterpret_cast<const unsigned long long*>(a.slots) + size_t(s) * kSlotsPerTensor + threadIdx.x;
    uint32_t kx = 0u, kn = 0u, kz = 0u;
#pragma unroll
    for (int w = 0; w < kSlotWays / kWave; w++) {
      const unsigned long long vx = sl[w * kWave], vn = sl[kSlotWays + w * kWave], vz = sl[2 * kSlotWays + w * kWave];
      const uint32_t x1 = (uint32_t(vx >> 32) == a.epoch) ? uint32_t(vx) : 0u;
      const uint32_t n1 = (uint32_t(vn >> 32) == a.epoch) ? uint32_t(vn) : 0u;
      const uint32_t z1 = (uint32_t(vz >> 32) == a.epoch) ? uint32_t(vz) : 0u;
      kx = x1 > kx ? x1 : kx;
      kn = n1 > kn ? n1 : kn;
      kz = z1 > kz ? z1 : kz;
    }
    kx = wave_max_u32(kx);
    kn = wave_max_u32(kn);
    kz = wave_max_u32(kz);
    if (threadIdx.x == 0) { s_k[0] = kx; s_k[1] = kn; s_k[2] = kz; }
  }
  __syncthreads();
  float mx = from_okey(s_k[0]), mn = from_okey(~s_k[1]);
  const uint32_t kz = s_k[2];
  if ((mn == 0.0f || mx == 0.0f) && kz != 0u) {
    const uint32_t b0 = (0xFFFFFFFFu - kz) * uint32_t(kRedTile);
    const uint32_t b1 = (n - b0 < uint32_t(kRedTile)) ? n : b0 + uint32_t(kRedTile);
    uint32_t first = 0xFFFFFFFFu;
    for (uint32_t e = b0 + threadIdx.x; e < b1; e += kThreads)
      if (xp[e] == 0.0f && e < first) first = e;
    float d0 = 0.f, d1 = 0.f;
    block_reduce(d0, d1, first);
    if (first != 0xFFFFFFFFu) {
      const float zv = xp[first];
      if (mn == 0.0f) mn = zv;
      if (mx == 0.0f) mx = zv;
    }
  }
  const uint32_t bits = a.seg[s].bits;
  gi_out = inverse_gap(mn, mx, bits);
  mn_out = mn;
  if (first_tile && threadIdx.x == 0) write_header(a.seg[s].out, bits, n, mn, mx);
}

// 2^32 * float(double(x) / 4294967295.0), in fp32 only (see the file header).
__device__ __forceinline__ float u01_scaled(uint32_t x) {
  const float hi = static_cast<float>(x & 0xFFFFFF00u);  // 24 significant bits: exact
  const float lo = static_cast<float>(x & 0xFFu);
  return hi + __builtin_fmaf(hi, 0x1.ffff88p-33f, lo);
}

template <int B, bool RANDOM>
__device__ __forceinline__ uint32_t quant_one(float x, float mn, float gi, uint32_t draw) {
  float th = (x - mn) * gi;
  int32_t t;
  if (RANDOM) {
    th = __builtin_fmaf(u01_scaled(draw), 0x1p-32f, th);  // th + u: the scaling by 2^-32 is exact
    t = static_cast<int32_t>(th);  // truncation, terngrad_body.h:94
  } else {
    t = static_cast<int32_t>(__builtin_rintf(th));  // nearbyint, terngrad_body.h:53
  }
  return static_cast<uint32_t>(t) & 0xFFu;
}

// The codes of one unit as its packed bytes.  Within a byte codes are OR-ed without masking
// (terngrad_body.h:95): a code that reaches 1<<B spills into the next slot of the SAME byte.  Shifting
// distributes over OR, so the byte is built from its last slot down, one shift-and-or per slot.
template <int B, int UNIT>
__device__ __forceinline__ uint32_t pack_codes(const uint32_t (&t)[UNIT]) {
  constexpr int DPB = 8 / B;
  uint32_t packed = 0;
#pragma unroll
  for (int jb = 0; jb < UNIT / DPB; jb++) {
    uint32_t p = t[jb * DPB + DPB - 1];
#pragma unroll
    for (int j = DPB - 2; j >= 0; j--) p = (p << B) | t[jb * DPB + j];
    packed |= (UNIT / DPB > 1 ? (p & 0xFFu) : p) << (8 * jb);  // a single byte is cut by its store
  }
  return packed;
}

// Quantises one unit held in registers and returns its BPU packed bytes; advances
// the lane's draws by `stride_bytes` output bytes.
template <int B, bool RANDOM, int UNIT = (8 / B > 4 ? 8 / B : 4)>
__device__ __forceinline__ uint32_t quant_unit(const float4 (&v)[UNIT / 4], float mn, float gi, uint32_t (&draw)[UNIT],
                                               uint32_t stride_bytes) {
  constexpr int DPB = 8 / B;
  uint32_t t[UNIT];
#pragma unroll
  for (int q = 0; q < UNIT; q++) {
    const float4 f = v[q / 4];
    const float x = (q & 3) == 0 ? f.x : (q & 3) == 1 ? f.y : (q & 3) == 2 ? f.z : f.w;
    t[q] = quant_one<B, RANDOM>(x, mn, gi, RANDOM ? draw[q] : 0u);
    if (RANDOM) draw[q] += lcg_mul(q % DPB + 2) * stride_bytes;
  }
  return pack_codes<B, UNIT>(t);
}

// Unit u of a tensor whose end may fall inside it: element-wise from memory.
template <int B, bool RANDOM, int UNIT = (8 / B > 4 ? 8 / B : 4)>
__device__ __forceinline__ void quant_unit_ragged(const EncSeg& sg, float mn, float gi, uint32_t u,
                                                  const uint32_t (&draw)[UNIT]) {
  constexpr int DPB = 8 / B;
  constexpr int BPU = UNIT / DPB;
  const float* __restrict__ xp = sg.x;
  uint8_t* __restrict__ pay = sg.out + 10;
  const uint32_t n = static_cast<uint32_t>(sg.n);
  const uint32_t nbytes = n / DPB;  // bytes the reference's transform covers
  for (int jb = 0; jb < BPU; jb++) {
    const uint32_t byte = u * BPU + jb;
    const size_t e = size_t(byte) * DPB;
    if (byte < nbytes) {
      uint32_t qv = 0;
      for (int j = 0; j < DPB; j++) {
        const uint32_t t = quant_one<B, RANDOM>(xp[e + j], mn, gi, RANDOM ? draw[jb * DPB + j] : 0u);
        qv |= t << (B * j);
      }
      pay[byte] = uint8_t(qv);
    } else if (byte == nbytes && (n % DPB)) {
      // Partial last byte: always round-to-nearest, stored at the last byte
      // of the caller's buffer (terngrad_body.h:288-296).
      uint32_t qv = 0;
      for (uint32_t j = 0; j < n % DPB; j++) qv |= quant_one<B, false>(xp[e + j], mn, gi, 0u) << (B * j);
      sg.out[sg.out_size - 1] = uint8_t(qv);
    }
  }
}

// One tile of the quantise stream.  A unit is UNIT = max(4, 8/B) consecutive
// elements owned by one lane per step; it packs into BPU = UNIT*B/8 bytes.
template <int B, bool RANDOM>
__device__ __forceinline__ void quant_tile(const EncSeg& sg, const float mn, const float gi, uint32_t tile_in_seg) {
  constexpr int DPB = 8 / B;
  constexpr int UNIT = DPB > 4 ? DPB : 4;
  constexpr int BPU = UNIT / DPB;
  constexpr uint32_t kStrideBytes = uint32_t(kThreads) * BPU;
  const float* __restrict__ xp = sg.x;
  uint8_t* __restrict__ pay = sg.out + 10;
  const uint32_t n = static_cast<uint32_t>(sg.n);
  const uint32_t u0 = tile_in_seg * uint32_t(kThreads * kQIters) + threadIdx.x;

  // Draw for slot j of byte (u*BPU + jb): A_{j+2} * (seed + byte) + C_{j+2}.
  uint32_t draw[UNIT];
  if (RANDOM) {
    const uint32_t x0 = sg.seed + u0 * BPU;
#pragma unroll
    for (int q = 0; q < UNIT; q++) {
      const int jb = q / DPB, j = q % DPB;
      draw[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
    }
  }

  const uint32_t units_total = (n + UNIT - 1) / UNIT;
  const uint32_t tile_u0 = u0 - threadIdx.x;
  if (uint64_t(tile_u0 + kThreads * kQIters) * UNIT <= n) {
    float4 v[kQIters][UNIT / 4];
#pragma unroll
    for (int k = 0; k < kQIters; k++)
#pragma unroll
      for (int h = 0; h < UNIT / 4; h++)
        v[k][h] = ld4_stream(xp + size_t(u0 + k * kThreads) * UNIT + h * 4);
#pragma unroll
    for (int k = 0; k < kQIters; k++) {
      const uint32_t packed = quant_unit<B, RANDOM>(v[k], mn, gi, draw, kStrideBytes);
#pragma unroll
      for (int jb = 0; jb < BPU; jb++) pay[size_t(u0 + k * kThreads) * BPU + jb] = uint8_t(packed >> (8 * jb));
    }
    return;
  }
  // Tile holding the end of the tensor.
  for (int k = 0; k < kQIters; k++) {
    const uint32_t u = u0 + k * kThreads;
    if (u < units_total) quant_unit_ragged<B, RANDOM>(sg, mn, gi, u, draw);
    if (RANDOM) {
#pragma unroll
      for (int q = 0; q < UNIT; q++) draw[q] += lcg_mul(q % DPB + 2) * kStrideBytes;
    }
  }
}

template <int B>
__device__ __forceinline__ void quant_dispatch(const EncSeg& sg, float mn, float gi, uint32_t t) {
  if (sg.random) quant_tile<B, true>(sg, mn, gi, t); else quant_tile<B, false>(sg, mn, gi, t);
}

// tile_start here counts quantise tiles (kThreads*kQIters units each).
template <int CAP>
__global__ __launch_bounds__(kThreads) void terngrad_quant_kernel(const EncArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const uint32_t t = static_cast<uint32_t>(tile - a.tile_start[s]);
  float mn, gi;
  load_scalars<CAP>(a, s, t == 0, mn, gi);
  switch (a.seg[s].bits) {
    case 1: quant_dispatch<1>(a.seg[s], mn, gi, t); break;
    case 2: quant_dispatch<2>(a.seg[s], mn, gi, t); break;
    case 4: quant_dispatch<4>(a.seg[s], mn, gi, t); break;
    default: quant_dispatch<8>(a.seg[s], mn, gi, t); break;
  }
}

// ---- resident encode ------------------------------------------------------------
// One launch for one large tensor.  The chip's register files and LDS together
// hold more than 128 MB, so a tensor of up to ~33M elements can stay on chip
// between the min/max pass and the quantise pass: every workgroup (one per CU,
// 1024 lanes) loads its contiguous share once, up to 24 float4 per lane into registers
// and the rest into LDS, publishes its extremes, waits at a grid-wide barrier and
// then quantises out of registers.  The tensor is read from HBM once instead of
// twice.
//
// The barrier is the exchange of hpx_common.h (records tagged with the number of
// the launch, `gen`; nothing is ever reset).  All workgroups of the grid
// must be resident together, which holds because the grid is at most one workgroup per
// CU and a workgroup fits a CU by construction; other work sharing the GPU only
// delays the barrier.  The wait is bounded by `spin_limit` ticks of the 100 MHz
// wall clock: on expiry the workgroup raises *host_flag and leaves, so the grid
// always drains.
constexpr int kResThreads = 1024;
constexpr int kResRegGroups = 24;  // float4 per lane held in registers ...
// ... except at 1 bit with stochastic rounding, whose eight draws per lane need the room.
// Rows of prepared random addends when the LDS has room for them (8 float4 per lane).
constexpr int res_pre_rows(int bits) { return bits == 1 ? 4 : 8; }
constexpr int res_reg_groups(int bits, bool random) { return (bits == 1 && random) ? 14 : kResRegGroups; }
constexpr int kResLdsGroups = 8;   // float4 per lane of the tensor held in LDS (128 KiB per workgroup)
constexpr int kResLdsTotalGroups = 9;  // ... and what the workgroup may use altogether (144 KiB): the rest holds prepared draws
struct ResArgs {
  EncSeg seg;
  uint32_t chunk_units;  // units per workgroup, a multiple of kWave
  uint32_t reg_rows;     // rows of 64 units a wave holds in registers: all the kernel has room for when the share
                         // fills them, otherwise just enough of them, so that a smaller share still spreads over all waves
  uint32_t lds_rows;     // rows of kResThreads units kept in LDS
  uint32_t pre_rows;     // register rows whose random addends are prepared during pass 1: 0 or res_pre_rows(bits)
  uint32_t stream_u0;    // a tensor larger than the chip: the first unit that is NOT kept on chip (= the workgroups'
                         // shares together); each workgroup streams `stream_units` units from there on twice, once
  uint32_t stream_units; // for the extremes and once to quantise them; a multiple of kWave.  0: everything is on chip
  uint32_t gen;          // generation of this launch, counted from 1: the tag of its records
  uint64_t* bar;         // exchange memory (kBarTotalWords); only ever holds (gen << 32 | key) words
  uint32_t* host_flag;   // pinned host word, set to 1 when the barrier wait expires
  uint64_t spin_limit;
  uint64_t* stamps;      // measurement aid, normally null: four wall-clock readings per workgroup (phase_stamp below)
  uint32_t* done;        // pinned host words, one per workgroup: set to `gen` by a workgroup that got through the barrier
};

// Measurement aid (hpx_terngrad_phase_stamps): while a buffer is set, every workgroup of a resident launch leaves
// four readings of the 100 MHz wall clock in it: [0] on entry, before its first load is requested; [1] when all its
// waves have their share loaded and reduced; [2] when it has the global extremes (the grid-wide exchange is behind
// it); [3] when all its waves have issued their last store.  One scalar branch per reading when no buffer is set.
__device__ __forceinline__ void phase_stamp(uint64_t* stamps, int k) {
  if (stamps && threadIdx.x == 0) stamps[size_t(blockIdx.x) * 4 + k] = wall_clock64();
}

__device__ __forceinline__ void acc_zero(float v, uint32_t idx, float& mn, float& mx, uint32_t& fz) {
  mn = v < mn ? v : mn;
  mx = v > mx ? v : mx;
  fz = (v == 0.0f && idx < fz) ? idx : fz;
}
__device__ __forceinline__ void acc_zero4(float4 v, uint32_t idx, float& mn, float& mx, uint32_t& fz) {
  acc_zero(v.x, idx, mn, mx, fz); acc_zero(v.y, idx + 1, mn, mx, fz);
  acc_zero(v.z, idx + 2, mn, mx, fz); acc_zero(v.w, idx + 3, mn, mx, fz);
}

// quant_unit for a unit whose random addends (2^32 * u per element) were prepared earlier.
template <int B, int UNIT = (8 / B > 4 ? 8 / B : 4)>
__device__ __forceinline__ uint32_t quant_unit_prepared(const float4 (&v)[UNIT / 4], const float4 (&s)[UNIT / 4], float mn,
                                                        float gi) {
  uint32_t t[UNIT];
#pragma unroll
  for (int q = 0; q < UNIT; q++) {
    const float4 f = v[q / 4], g = s[q / 4];
    const float x = (q & 3) == 0 ? f.x : (q & 3) == 1 ? f.y : (q & 3) == 2 ? f.z : f.w;
    const float sc = (q & 3) == 0 ? g.x : (q & 3) == 1 ? g.y : (q & 3) == 2 ? g.z : g.w;
    float th = (x - mn) * gi;
    th = __builtin_fmaf(sc, 0x1p-32f, th);
    t[q] = static_cast<uint32_t>(static_cast<int32_t>(th)) & 0xFFu;
  }
  return pack_codes<B, UNIT>(t);
}

// PRE: register rows whose random addends are prepared during pass 1 (a compile-time count, so that pass 2
// stays one straight block the scheduler can interleave across rows; a per-row branch cost as much as the
// prepared rows saved).
//
// STREAMED: the tensor is larger than the chip can hold.  The workgroups' shares (the first stream_u0 units) stay on
// chip as described; the rest is dealt out in contiguous pieces of stream_units units per workgroup and streamed
// twice by the same launch: before the share is loaded, for its extremes, and again to be quantised.  The second
// time round it passes through a ring made of the first sixteen register rows themselves: a row is requested for
// the streamed part the moment its row of the share has been quantised, so memory is busy again from the first
// row of pass 2 on, while the rest of the share (arithmetic only) is still being worked on.  The tensor's head is
// read once, the rest twice: 4 (2 - share/n) bytes per element where the two-launch encode reads 8.
constexpr int kResStreamIters = 8;  // units per lane and round of a streaming loop (128 KiB per workgroup in flight at 2 bits)

template <int B, bool RANDOM, int PRE, bool STREAMED = false>
__global__ __launch_bounds__(kResThreads) void terngrad_resident_kernel(const ResArgs a) {
  constexpr int DPB = 8 / B;
  constexpr int UNIT = DPB > 4 ? DPB : 4;
  constexpr int H = UNIT / 4;
  constexpr int BPU = UNIT / DPB;
  constexpr int KU = res_reg_groups(B, RANDOM) / H;  // unit rows held in registers
  constexpr int kWaves = kResThreads / kWave;
  extern __shared__ float4 s_rows[];  // [lds_rows][H][kResThreads]
  __shared__ float s_mn[kWaves], s_mx[kWaves];
  __shared__ uint32_t s_fz[kWaves];
  __shared__ uint32_t s_q[kBarWaves][4];  // per quarter of the grid: the three keys, then 1 if its wait ended in time

  phase_stamp(a.stamps, 0);
  const float* __restrict__ xp = a.seg.x;
  const uint32_t n = static_cast<uint32_t>(a.seg.n);
  const uint32_t full_units = n / UNIT;
  const uint32_t wg_u0 = blockIdx.x * a.chunk_units;
  const uint32_t wg_lim = wg_u0 + a.chunk_units;
  const uint32_t wg_end = wg_lim < full_units ? wg_lim : full_units;  // <= wg_u0 for a workgroup without a share
  // A wave's register rows are 24 consecutive 64-unit pieces (24 KiB of contiguous
  // input per wave: measurably faster than rows spread over the workgroup's
  // share); the LDS rows follow all register rows.
  constexpr uint32_t rs = kWave;
  const uint32_t R = a.reg_rows;  // KU whenever there are LDS rows
  const uint32_t u0 = wg_u0 + (threadIdx.x / kWave) * (R * kWave) + (threadIdx.x & (kWave - 1));
  const uint32_t l0 = wg_u0 + KU * kResThreads + threadIdx.x;
  constexpr uint32_t stride_bytes = rs * BPU;
  const float qnan = __builtin_nanf("");  // compares false both ways: ignored by min and max

  // ---- pass 1: load the share, reduce ------------------------------------------
  // All loads of the lane are requested at once: the LDS rows, which go straight into LDS and cost no
  // registers on the way (lanes past the end of the share keep whatever their slot held: every later
  // reader checks the bound), then its register rows.  While
  // they are in flight and the ALUs idle, the random addends of the first PRE register rows, which
  // depend on position and seed only, go into the LDS the tensor does not need; pass 2 (ALU-bound:
  // nothing left to overlap with) then skips 6 of its 11 operations per element for those rows.
  // Then each register row is reduced as it arrives (min, max and min |x| of every element; the
  // index of the first zero is only worked out by lanes that met one), so that only the last
  // rows' work is left when the last byte has landed.  This is one straight block per case - a
  // workgroup whose register rows are all whole, and the others - because behind a join of the
  // two the compiler no longer knows the order of the loads and waits for all of them at once.
  // STREAMED: pass 2 streams through two buffers of SW float4 per lane.  They are the first 2 SW register rows
  // themselves: a row is requested again, for the streamed part, as soon as its share of the head has been quantised,
  // so that memory works through the whole of pass 2 and the buffers cost no registers of their own.
  constexpr int SW = STREAMED ? kResStreamIters / H : 1;  // float4 per lane and round: the same at every width
  constexpr int KV = (STREAMED && 2 * SW > KU) ? 2 * SW : KU;
  float4 v[KV][H];
#pragma unroll
  for (int k = KU; k < KV; k++)
#pragma unroll
    for (int h = 0; h < H; h++) v[k][h] = make_float4(0.f, 0.f, 0.f, 0.f);
  float4* s_pre = s_rows + size_t(a.lds_rows) * H * kResThreads;
  float mn = __builtin_inff(), mx = -__builtin_inff(), am = __builtin_inff();
  uint32_t fz = 0xFFFFFFFFu;
  // The part of the tensor that does not stay on chip, first time through: extremes and first zero only.
  const uint32_t st_u0 = STREAMED ? a.stream_u0 + blockIdx.x * a.stream_units : 0u;
  const uint32_t st_lim = st_u0 + (STREAMED ? a.stream_units : 0u);
  const uint32_t st_end = STREAMED ? (st_u0 >= full_units ? st_u0 : (st_lim < full_units ? st_lim : full_units)) : 0u;
  if (STREAMED) {
    for (uint32_t t0 = st_u0; t0 < st_end; t0 += uint32_t(kResStreamIters) * kResThreads) {
      float4 w[kResStreamIters][H];
#pragma unroll
      for (int k = 0; k < kResStreamIters; k++) {
        const uint32_t u = t0 + k * kResThreads + threadIdx.x;
#pragma unroll
        for (int h = 0; h < H; h++)
          w[k][h] = u < st_end ? ld4_stream(xp + size_t(u) * UNIT + h * 4) : make_float4(qnan, qnan, qnan, qnan);
      }
      float amt = __builtin_inff();
#pragma unroll
      for (int k = 0; k < kResStreamIters; k++)
#pragma unroll
        for (int h = 0; h < H; h++) acc3x4(w[k][h], mn, mx, amt);
      if (amt == 0.0f) {  // a zero among this lane's elements of the round: note where (rare)
        float d0 = 0.f, d1 = 0.f;
#pragma unroll
        for (int k = 0; k < kResStreamIters; k++)
#pragma unroll
          for (int h = 0; h < H; h++) acc_zero4(w[k][h], (t0 + k * kResThreads + threadIdx.x) * UNIT + h * 4, d0, d1, fz);
      }
    }
  }
  const bool whole_rows = wg_u0 + uint32_t(KU * kResThreads) <= wg_end;
  const uint32_t wave_lane0 = __builtin_amdgcn_readfirstlane(threadIdx.x & ~uint32_t(kWave - 1));
  for (uint32_t r = 0; r < a.lds_rows; r++) {
    const uint32_t u = l0 + r * kResThreads;
    if (u < wg_end) {
#pragma unroll
      for (int h = 0; h < H; h++) ld4_stream_to_lds(xp + size_t(u) * UNIT + h * 4, s_rows + (r * H + h) * kResThreads + wave_lane0);
    }
  }
  auto pass1 = [&](auto whole) {
#pragma unroll
    for (int k = 0; k < KU; k++) {
      const uint32_t u = u0 + k * rs;
#pragma unroll
      for (int h = 0; h < H; h++)
        v[k][h] = (decltype(whole)::value || (uint32_t(k) < R && u < wg_end)) ? ld4_stream(xp + size_t(u) * UNIT + h * 4)
                                                         : make_float4(qnan, qnan, qnan, qnan);
    }
    __builtin_amdgcn_sched_barrier(0);  // every load is requested before any other work: nothing moves across this line
    if (RANDOM && PRE > 0) {
      uint32_t d[UNIT];
      const uint32_t x0 = a.seg.seed + u0 * BPU;
#pragma unroll
      for (int q = 0; q < UNIT; q++) {
        const int jb = q / DPB, j = q % DPB;
        d[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
      }
      for (uint32_t k = 0; k < uint32_t(PRE); k++) {
#pragma unroll
        for (int h = 0; h < H; h++)
          s_pre[(k * H + h) * kResThreads + threadIdx.x] =
              make_float4(u01_scaled(d[4 * h]), u01_scaled(d[4 * h + 1]), u01_scaled(d[4 * h + 2]), u01_scaled(d[4 * h + 3]));
#pragma unroll
        for (int q = 0; q < UNIT; q++) d[q] += lcg_mul(q % DPB + 2) * stride_bytes;
      }
    }
#pragma unroll
    for (int k = 0; k < KU; k++)
#pragma unroll
      for (int h = 0; h < H; h++) acc3x4(v[k][h], mn, mx, am);
  };
  if (whole_rows) pass1(std::true_type{}); else pass1(std::false_type{});
  if (a.lds_rows > 0) wait_vector_loads();  // the LDS rows were requested first and have long landed
  for (uint32_t r = 0; r < a.lds_rows; r++) {
    if (l0 + r * kResThreads < wg_end) {
#pragma unroll
      for (int h = 0; h < H; h++) acc3x4(s_rows[(r * H + h) * kResThreads + threadIdx.x], mn, mx, am);
    }
  }
  if (am == 0.0f) {
    float d0 = 0.f, d1 = 0.f;
#pragma unroll
    for (int k = 0; k < KU; k++)
#pragma unroll
      for (int h = 0; h < H; h++) acc_zero4(v[k][h], (u0 + k * rs) * UNIT + h * 4, d0, d1, fz);
    for (uint32_t r = 0; r < a.lds_rows; r++) {  // this lane's own LDS rows
      if (l0 + r * kResThreads < wg_end) {
#pragma unroll
        for (int h = 0; h < H; h++)
          acc_zero4(s_rows[(r * H + h) * kResThreads + threadIdx.x], (l0 + r * kResThreads) * UNIT + h * 4, d0, d1, fz);
      }
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0)
    for (uint32_t e = full_units * UNIT; e < n; e++) acc_zero(xp[e], e, mn, mx, fz);

  mn = wave_min(mn);
  mx = wave_max(mx);
  fz = wave_min_u32(fz);
  if ((threadIdx.x & (kWave - 1)) == 0) {
    s_mn[threadIdx.x / kWave] = mn; s_mx[threadIdx.x / kWave] = mx; s_fz[threadIdx.x / kWave] = fz;
  }
  __syncthreads();
  phase_stamp(a.stamps, 1);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  if (wave < uint32_t(kBarWaves)) {
    // Each wave that takes part in the exchange folds the workgroup's sixteen results for itself.
    const uint32_t i = threadIdx.x & (kWaves - 1);
    mn = wave_min(s_mn[i]);
    mx = wave_max(s_mx[i]);
    fz = wave_min_u32(s_fz[i]);
    const bool has = mx >= mn;  // false only for a workgroup whose share is empty
    // largest key of x; largest complemented key (the minimum); complemented index of the first zero, 0 for none
    uint32_t k0 = has ? okey(mx) : 0u, k1 = has ? ~okey(mn) : 0u, k2 = fz != 0xFFFFFFFFu ? 0xFFFFFFFEu - fz : 0u;
    const bool ok = grid_exchange(a.bar, a.gen, a.spin_limit, wave, k0, k1, k2);
    if ((threadIdx.x & (kWave - 1)) == 0) {
      if (!ok) __hip_atomic_store(a.host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      s_q[wave][0] = k0; s_q[wave][1] = k1; s_q[wave][2] = k2;
      s_q[wave][3] = ok ? 1u : 0u;
    }
  }
  __syncthreads();
  uint32_t kx = 0u, kn = 0u, kz = 0u, oks = 1u;
#pragma unroll
  for (int q = 0; q < kBarWaves; q++) {
    kx = s_q[q][0] > kx ? s_q[q][0] : kx;
    kn = s_q[q][1] > kn ? s_q[q][1] : kn;
    kz = s_q[q][2] > kz ? s_q[q][2] : kz;
    oks &= s_q[q][3];
  }
  if (oks == 0u) return;
  // this workgroup will write its part of the message: the host may forget the launch once all have said so
  if (threadIdx.x == 0) __hip_atomic_store(a.done + blockIdx.x, a.gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  phase_stamp(a.stamps, 2);

  // ---- pass 2: quantise from registers -------------------------------------------
  mx = from_okey(kx);
  mn = from_okey(~kn);
  if ((mn == 0.0f || mx == 0.0f) && kz != 0u) {
    // thrust::minmax_element returns the first extreme: a zero extreme carries the
    // sign of the first zero of the tensor.
    const float zv = xp[0xFFFFFFFEu - kz];
    if (mn == 0.0f) mn = zv;
    if (mx == 0.0f) mx = zv;
  }
  const float gi = inverse_gap(mn, mx, B);
  if (blockIdx.x == 0 && threadIdx.x == 0) write_header(a.seg.out, B, n, mn, mx);

  uint8_t* __restrict__ pay = a.seg.out + 10;
  uint32_t draw[UNIT];
  if (RANDOM) {
    const uint32_t x0 = a.seg.seed + u0 * BPU + uint32_t(PRE) * stride_bytes;  // first row that draws for itself
#pragma unroll
    for (int q = 0; q < UNIT; q++) {
      const int jb = q / DPB, j = q % DPB;
      draw[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
    }
  }
  constexpr uint32_t kRound = uint32_t(SW) * kResThreads;
  // STREAMED: rows 0 .. 2 SW - 1 of `v` are a ring for the streamed part.  A row's address is a uniform pointer plus
  // a 32-bit lane offset, and the request is unconditional: a lane past the end of the workgroup's piece reads the
  // piece's last unit (any unit of the tensor, for a workgroup without a piece) and the value is never stored.
  constexpr int RG = 2 * SW;
  const uint32_t lane_off = threadIdx.x * (UNIT * 4);
  const uint32_t st_last = (st_end > st_u0 ? st_end : full_units) - 1u;  // uniform; STREAMED tensors have units
  auto fetch_row = [&](int k, uint32_t r0) {  // r0, uniform: the row's first unit
    const uint32_t b0 = r0 < st_last ? r0 : st_last;
    const uint32_t room = (st_last - b0) * (UNIT * 4);
    const float* rowp = xp + size_t(b0) * UNIT;
    const uint32_t off = lane_off < room ? lane_off : room;
    ring_request<0>(v[k][0], rowp, off);
    if (H > 1) ring_request<16>(v[k][H - 1], rowp, off);
  };
  // A workgroup whose register rows are all whole (every one but the last with a share) stores
  // without a bounds check per row: the checks cost a branch each.
  auto register_rows = [&](auto whole) {
#pragma unroll
    for (int k = 0; k < KU; k++) {
      const uint32_t u = u0 + k * rs;
      uint32_t packed;
      if (RANDOM && k < PRE) {
        float4 sc[H];
#pragma unroll
        for (int h = 0; h < H; h++) sc[h] = s_pre[(k * H + h) * kResThreads + threadIdx.x];
        packed = quant_unit_prepared<B>(v[k], sc, mn, gi);
      } else {
        packed = quant_unit<B, RANDOM>(v[k], mn, gi, draw, stride_bytes);
      }
      if (decltype(whole)::value || (uint32_t(k) < R && u < wg_end)) {
#pragma unroll
        for (int jb = 0; jb < BPU; jb++) pay[size_t(u) * BPU + jb] = uint8_t(packed >> (8 * jb));
      }
      if (STREAMED && k < RG) fetch_row(k, st_u0 + uint32_t(k) * kResThreads);  // the row is free: first trip of the ring
    }
  };
  // (a tensor that is streamed fills every workgroup's share)
  if (STREAMED || whole_rows) register_rows(std::true_type{}); else register_rows(std::false_type{});
  if (STREAMED) {
#pragma unroll
    for (int k = KU; k < RG; k++) fetch_row(k, st_u0 + uint32_t(k) * kResThreads);
  }
  if (RANDOM) {
    uint32_t x0 = a.seg.seed + l0 * BPU;
    // Keeps the compiler from preparing these draws before the register rows are
    // done, where they would cost registers the rows need.
    __asm__ volatile("" : "+v"(x0));
#pragma unroll
    for (int q = 0; q < UNIT; q++) {
      const int jb = q / DPB, j = q % DPB;
      draw[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
    }
  }
  for (uint32_t r = 0; r < a.lds_rows; r++) {
    const uint32_t u = l0 + r * kResThreads;
    float4 f[H];
#pragma unroll
    for (int h = 0; h < H; h++) f[h] = s_rows[(r * H + h) * kResThreads + threadIdx.x];
    const uint32_t packed = quant_unit<B, RANDOM>(f, mn, gi, draw, uint32_t(kResThreads) * BPU);
    if (u < wg_end) {
#pragma unroll
      for (int jb = 0; jb < BPU; jb++) pay[size_t(u) * BPU + jb] = uint8_t(packed >> (8 * jb));
    }
  }
  // The part of the tensor that did not stay on chip, second time through: quantise it.
  if (STREAMED) {
    if (RANDOM) {
      const uint32_t x0 = a.seg.seed + (st_u0 + threadIdx.x) * BPU;
#pragma unroll
      for (int q = 0; q < UNIT; q++) {
        const int jb = q / DPB, j = q % DPB;
        draw[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
      }
    }
    // One trip round the ring per iteration: a row is waited for, quantised, stored and requested again for the
    // next trip.  Of the rows requested after it, RG - 1 are certain to have been issued when a row is waited for
    // (the stores between them are not counted: a wave none of whose lanes stores skips the instruction).
    auto half = [&](auto base, uint32_t t0) {
#pragma unroll
      for (int k = decltype(base)::value; k < decltype(base)::value + SW; k++) {
        const uint32_t u = t0 + k * kResThreads + threadIdx.x;
#pragma unroll
        for (int h = 0; h < H; h++) ring_wait<(RG - 1) * H>(v[k][h]);
        const uint32_t packed = quant_unit<B, RANDOM>(v[k], mn, gi, draw, uint32_t(kResThreads) * BPU);
        if (u < st_end) {
#pragma unroll
          for (int jb = 0; jb < BPU; jb++) pay[size_t(u) * BPU + jb] = uint8_t(packed >> (8 * jb));
        }
        fetch_row(k, t0 + uint32_t(RG + k) * kResThreads);
      }
    };
    for (uint32_t t0 = st_u0; t0 < st_end; t0 += 2 * kRound) {
      half(std::integral_constant<int, 0>{}, t0);
      if (t0 + kRound >= st_end) break;
      half(std::integral_constant<int, SW>{}, t0);
    }
    // Requests of the last trips are still on their way: the ring's registers stay taken until they have landed.
#pragma unroll
    for (int k = 0; k < RG; k++)
#pragma unroll
      for (int h = 0; h < H; h++) ring_wait<0>(v[k][h]);
  }
  // The unit that holds the end of the tensor, if the length is not a whole number of units.
  if (blockIdx.x == 0 && threadIdx.x == 0 && full_units * UNIT < n) {
    uint32_t d[UNIT];
#pragma unroll
    for (int q = 0; q < UNIT; q++) {
      const int jb = q / DPB, j = q % DPB;
      d[q] = lcg_mul(j + 2) * (a.seg.seed + full_units * BPU + jb) + lcg_add(j + 2);
    }
    quant_unit_ragged<B, RANDOM>(a.seg, mn, gi, full_units, d);
  }
  if (a.stamps) {  // uniform
    __syncthreads();
    phase_stamp(a.stamps, 3);
  }
}

// ---- resident encode of a bucket -------------------------------------------------
// The same idea for a call with several tensors whose sum fits the chip: ONE launch
// reads every tensor once.  The unit of work is a piece: `rows` rows of 64 units of
// one tensor, held by one wave (register rows first, LDS rows after them), so the
// tensor, its extremes and its seed are wave-uniform and the inner loops are those
// of the single-tensor kernel.  Piece p belongs to wave p / G of workgroup p % G (G workgroups):
// consecutive pieces go to consecutive workgroups, so every CU gets the same mix of whole pieces
// and tensor ends (with piece p on wave p % 16 of workgroup p / 16 the workgroups that
// held sixteen whole pieces of a large tensor set the pace of both passes);
// the host picks the smallest `rows` for which all pieces fit (every tensor that is not tiny has at
// least one piece; the piece that ends a tensor also takes the 1..UNIT-1 elements
// behind its last whole unit).
//
// Tiny tensors (at most 2048 elements: the biases and normalisation parameters that make up two thirds of a
// convolutional network's tensor list) get no piece - each would cost a wave that could hold `rows` rows.  They are
// dealt out to the waves that are left without a piece, two to a wave, which request them at the start and encode
// them start to finish on their own behind the barrier, while the others quantise (a wave's reduction gives a
// tensor's extremes: no slots).
//
// The extremes travel through the epoch-tagged slots of the tiled kernels: a wave
// folds its piece into way (piece index % kSlotWays) of its tensor's three slots with
// atomic max operations whose results it waits for, the grid meets at the barrier of
// grid_exchange (its payload unused), and every wave then folds the ways of its
// tensor.

// A tensor of at most this many rows of 64 units is "tiny": 2048 elements at every width.
constexpr int tiny_rows(int bits) { return bits == 1 ? 4 : 8; }
constexpr int kTinyPerWave = 2;  // tiny tensors a left-over wave takes at a time
struct ResMultiArgs {
  int32_t nseg;
  int32_t piece_start[kCapLarge + 1];  // (a tiny tensor's entry equals the next one's)
  EncSeg seg[kCapLarge];
  uint64_t* slots;
  uint32_t epoch;
  uint32_t rows;       // rows of 64 units per piece
  uint32_t lds_rows;   // rows beyond the register rows, kept in LDS
  uint32_t gen;
  uint64_t* bar;
  uint32_t* host_flag;
  uint64_t spin_limit;
  uint64_t* stamps;    // measurement aid, normally null (phase_stamp)
  uint32_t* done;      // pinned host words, one per workgroup: set to `gen` by a workgroup that got through the barrier
  int32_t ntiny;       // tensors without a piece: the waves without a piece encode them on their own
  int16_t tiny[kCapLarge];  // their indices
};
static_assert(sizeof(ResMultiArgs) <= 9600, "kernel-argument budget");

// One wave encodes kTinyPerWave whole tensors of at most tiny_rows * 64 units each (plus the elements behind their
// last whole units), in two steps.  tiny_request asks for the tensors' rows, into the registers the wave would
// hold a piece in, when the kernel starts: the requests queue behind those of the fifteen waves beside it and
// land about when their pieces have (a CU serves its waves' requests in order).  tiny_finish does the rest behind
// the grid's barrier, when memory is idle and the other waves quantise: the tensors' extremes from the wave's own
// reduction, the header, the codes.
template <int B>
struct TinyShape {
  static constexpr int DPB = 8 / B;
  static constexpr int UNIT = DPB > 4 ? DPB : 4;
  static constexpr int H = UNIT / 4;
  static constexpr int BPU = UNIT / DPB;
  static constexpr int ROWS = tiny_rows(B);
};
template <int B, int KV>
__device__ __forceinline__ void tiny_request(const ResMultiArgs& a, int t0, int step, uint32_t lane, float4 (&v)[KV][TinyShape<B>::H]) {
  using S = TinyShape<B>;
  static_assert(kTinyPerWave * S::ROWS <= KV, "the tiny tensors' rows must fit the wave's register rows");
  const float qnan = __builtin_nanf("");
#pragma unroll
  for (int i = 0; i < kTinyPerWave; i++) {
    const bool have = t0 + i * step < a.ntiny;  // wave-uniform
    const EncSeg& sg = a.seg[a.tiny[have ? t0 + i * step : t0]];
    const uint32_t full_units = have ? static_cast<uint32_t>(sg.n) / S::UNIT : 0u;
#pragma unroll
    for (int k = 0; k < S::ROWS; k++) {
      const uint32_t u = k * kWave + lane;
#pragma unroll
      for (int h = 0; h < S::H; h++)
        v[i * S::ROWS + k][h] = u < full_units ? ld4_stream(sg.x + (u * S::UNIT + h * 4)) : make_float4(qnan, qnan, qnan, qnan);
    }
  }
}
template <int B, bool RANDOM, int KV>
__device__ __forceinline__ void tiny_finish(const ResMultiArgs& a, int t0, int step, uint32_t lane, const float4 (&v)[KV][TinyShape<B>::H]) {
  using S = TinyShape<B>;
  constexpr int DPB = S::DPB, UNIT = S::UNIT, H = S::H, BPU = S::BPU, ROWS = S::ROWS;
  constexpr uint32_t stride_bytes = uint32_t(kWave) * BPU;
#pragma unroll
  for (int i = 0; i < kTinyPerWave; i++) {
    if (t0 + i * step >= a.ntiny) break;  // wave-uniform
    const EncSeg& sg = a.seg[a.tiny[t0 + i * step]];
    const float* __restrict__ xp = sg.x;
    const uint32_t n = static_cast<uint32_t>(sg.n);
    const uint32_t full_units = n / UNIT;
    float mn = __builtin_inff(), mx = -__builtin_inff(), am = __builtin_inff();
#pragma unroll
    for (int k = 0; k < ROWS; k++)
#pragma unroll
      for (int h = 0; h < H; h++) acc3x4(v[i * ROWS + k][h], mn, mx, am);
    uint32_t fz = 0xFFFFFFFFu;
    if (am == 0.0f) {
      float d0 = 0.f, d1 = 0.f;
#pragma unroll
      for (int k = 0; k < ROWS; k++)
#pragma unroll
        for (int h = 0; h < H; h++) acc_zero4(v[i * ROWS + k][h], (k * kWave + lane) * UNIT + h * 4, d0, d1, fz);
    }
    if (lane == 0)
      for (uint32_t e = full_units * UNIT; e < n; e++) acc_zero(xp[e], e, mn, mx, fz);
    mn = wave_min(mn);
    mx = wave_max(mx);
    fz = wave_min_u32(fz);
    if ((mn == 0.0f || mx == 0.0f) && fz != 0xFFFFFFFFu) {  // a zero extreme carries the sign of the tensor's first zero
      const float zv = xp[fz];
      if (mn == 0.0f) mn = zv;
      if (mx == 0.0f) mx = zv;
    }
    const float gi = inverse_gap(mn, mx, B);
    if (lane == 0) write_header(sg.out, B, n, mn, mx);
    uint8_t* __restrict__ pay = sg.out + 10;
    uint32_t draw[UNIT];
    if (RANDOM) {
      const uint32_t x0 = sg.seed + lane * BPU;
#pragma unroll
      for (int q = 0; q < UNIT; q++) {
        const int jb = q / DPB, j = q % DPB;
        draw[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
      }
    }
#pragma unroll
    for (int k = 0; k < ROWS; k++) {
      if (uint32_t(k) * kWave >= full_units) break;  // wave-uniform: most tiny tensors are a row or two
      const uint32_t u = k * kWave + lane;
      const uint32_t packed = quant_unit<B, RANDOM>(v[i * ROWS + k], mn, gi, draw, stride_bytes);
      if (u < full_units) {
#pragma unroll
        for (int jb = 0; jb < BPU; jb++) pay[u * BPU + jb] = uint8_t(packed >> (8 * jb));
      }
    }
    if (lane == 0 && full_units * UNIT < n) {
      uint32_t d[UNIT];
#pragma unroll
      for (int q = 0; q < UNIT; q++) {
        const int jb = q / DPB, j = q % DPB;
        d[q] = lcg_mul(j + 2) * (sg.seed + full_units * BPU + jb) + lcg_add(j + 2);
      }
      quant_unit_ragged<B, RANDOM>(sg, mn, gi, full_units, d);
    }
  }
}

template <int B, bool RANDOM, int PRE>
__global__ __launch_bounds__(kResThreads) void terngrad_resident_multi_kernel(const ResMultiArgs a) {
  constexpr int DPB = 8 / B;
  constexpr int UNIT = DPB > 4 ? DPB : 4;
  constexpr int H = UNIT / 4;
  constexpr int BPU = UNIT / DPB;
  constexpr int KU = res_reg_groups(B, RANDOM) / H;  // unit rows held in registers
  constexpr int kWaves = kResThreads / kWave;
  constexpr uint32_t stride_bytes = uint32_t(kWave) * BPU;
  extern __shared__ float4 s_rows[];  // [wave][lds_rows][H][64], then the prepared draws [wave][PRE][H][64]
  __shared__ uint32_t s_ok[kBarWaves];

  // The wave index is the same in every lane: taken from the first lane, it and all that is derived from it
  // (piece, tensor, bounds) live in scalar registers.
  phase_stamp(a.stamps, 0);
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x & (kWave - 1);
  const int total = a.piece_start[a.nseg];
  const int my_piece = int(wave) * int(gridDim.x) + int(blockIdx.x);
  const bool active = my_piece < total;           // wave-uniform
  const int piece = active ? my_piece : total - 1;  // an idle wave looks at the last piece and touches nothing
  const int s = __builtin_amdgcn_readfirstlane(find_segment<kCapLarge>(a.piece_start, a.nseg, piece));
  const EncSeg& sg = a.seg[s];
  const float* __restrict__ xp = sg.x;
  const uint32_t n = static_cast<uint32_t>(sg.n);
  const uint32_t full_units = n / UNIT;
  const uint32_t pl = uint32_t(piece - a.piece_start[s]);
  const uint32_t npieces = uint32_t(a.piece_start[s + 1] - a.piece_start[s]);
  const uint32_t u_beg = pl * a.rows * kWave;
  const uint32_t u_lim = u_beg + a.rows * kWave;
  const uint32_t u_end = !active ? 0u : (u_lim < full_units ? u_lim : full_units);
  const bool ends_tensor = active && pl == npieces - 1;
  const uint32_t u0 = u_beg + lane;
  const float qnan = __builtin_nanf("");  // compares false both ways: ignored by min and max
  float4* s_mine = s_rows + size_t(wave) * a.lds_rows * H * kWave;
  float4* s_pre = s_rows + size_t(kWaves) * a.lds_rows * H * kWave + size_t(wave) * PRE * H * kWave;

  // ---- pass 1: load the piece, reduce ---------------------------------------------
  // As in the single-tensor kernel: all loads at once (the LDS rows, straight into LDS, ahead of the register rows), the
  // random addends of the first PRE rows while they are in flight, then every row reduced as it arrives,
  // one straight block per case.
  constexpr int KV = kTinyPerWave * tiny_rows(B) > KU ? kTinyPerWave * tiny_rows(B) : KU;
  float4 v[KV][H];
  float mn = __builtin_inff(), mx = -__builtin_inff(), am = __builtin_inff();
  const bool whole_rows = u_beg + uint32_t(KU * kWave) <= u_end;
  // A wave without a piece may have tiny tensors to encode (the host leaves at least ntiny / kTinyPerWave such
  // waves: wave total + t takes tensors t and t + nidle of the list).
  const int nidle = int(gridDim.x) * kWaves - total;
  const bool has_tiny = !active && my_piece - total < a.ntiny;
  const uint32_t ul0 = u0 + uint32_t(KU) * kWave;  // this lane's unit in the first LDS row
  for (uint32_t r = 0; r < a.lds_rows; r++) {
    const uint32_t u = ul0 + r * kWave;
    if (u < u_end) {
#pragma unroll
      for (int h = 0; h < H; h++) ld4_stream_to_lds(xp + size_t(u) * UNIT + h * 4, s_mine + (r * H + h) * kWave);
    }
  }
  auto pass1 = [&](auto whole) {
#pragma unroll
    for (int k = 0; k < KU; k++) {
      const uint32_t u = u0 + k * kWave;
#pragma unroll
      for (int h = 0; h < H; h++)
        v[k][h] = (decltype(whole)::value || u < u_end) ? ld4_stream(xp + size_t(u) * UNIT + h * 4)
                                                        : make_float4(qnan, qnan, qnan, qnan);
    }
    __builtin_amdgcn_sched_barrier(0);  // every load is requested before any other work: nothing moves across this line
    if (RANDOM && PRE > 0) {
      uint32_t d[UNIT];
      const uint32_t x0 = sg.seed + u0 * BPU;
#pragma unroll
      for (int q = 0; q < UNIT; q++) {
        const int jb = q / DPB, j = q % DPB;
        d[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
      }
      for (uint32_t k = 0; k < uint32_t(PRE); k++) {
#pragma unroll
        for (int h = 0; h < H; h++)
          s_pre[(k * H + h) * kWave + lane] =
              make_float4(u01_scaled(d[4 * h]), u01_scaled(d[4 * h + 1]), u01_scaled(d[4 * h + 2]), u01_scaled(d[4 * h + 3]));
#pragma unroll
        for (int q = 0; q < UNIT; q++) d[q] += lcg_mul(q % DPB + 2) * stride_bytes;
      }
    }
#pragma unroll
    for (int k = 0; k < KU; k++)
#pragma unroll
      for (int h = 0; h < H; h++) acc3x4(v[k][h], mn, mx, am);
  };
  if (whole_rows) pass1(std::true_type{});
  else if (!has_tiny) pass1(std::false_type{});
  else tiny_request<B>(a, my_piece - total, nidle, lane, v);
  if (a.lds_rows > 0) wait_vector_loads();
  for (uint32_t r = 0; r < a.lds_rows; r++) {
    if (ul0 + r * kWave < u_end) {
#pragma unroll
      for (int h = 0; h < H; h++) acc3x4(s_mine[(r * H + h) * kWave + lane], mn, mx, am);
    }
  }
  uint32_t fz = 0xFFFFFFFFu;
  if (am == 0.0f) {
    float d0 = 0.f, d1 = 0.f;
#pragma unroll
    for (int k = 0; k < KU; k++)
#pragma unroll
      for (int h = 0; h < H; h++) acc_zero4(v[k][h], (u0 + k * kWave) * UNIT + h * 4, d0, d1, fz);
    for (uint32_t r = 0; r < a.lds_rows; r++) {  // this lane's own LDS rows
      if (ul0 + r * kWave < u_end) {
#pragma unroll
        for (int h = 0; h < H; h++)
          acc_zero4(s_mine[(r * H + h) * kWave + lane], (ul0 + r * kWave) * UNIT + h * 4, d0, d1, fz);
      }
    }
  }
  if (ends_tensor && lane == 0)
    for (uint32_t e = full_units * UNIT; e < n; e++) acc_zero(xp[e], e, mn, mx, fz);
  mn = wave_min(mn);
  mx = wave_max(mx);
  fz = wave_min_u32(fz);
  const uint32_t ways = npieces < uint32_t(kSlotWays) ? npieces : uint32_t(kSlotWays);
  unsigned long long* sl = reinterpret_cast<unsigned long long*>(a.slots) + size_t(s) * kSlotsPerTensor;
  if (active && lane < 3) {
    // lane 0: key of the maximum; lane 1: complemented key of the minimum; lane 2: complemented index
    // of the first zero, 0 for none.  An active piece is never empty.
    const uint32_t key = lane == 0 ? okey(mx) : lane == 1 ? ~okey(mn) : (fz != 0xFFFFFFFFu ? 0xFFFFFFFEu - fz : 0u);
    const unsigned long long word = (static_cast<unsigned long long>(a.epoch) << 32) | key;
    const unsigned long long old =
        __hip_atomic_fetch_max(sl + lane * kSlotWays + (pl % kSlotWays), word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The barrier below must not be entered before the slot holds this piece: wait for the result.
    __asm__ volatile("" ::"v"(old));
  }
  __syncthreads();
  phase_stamp(a.stamps, 1);
  if (wave < uint32_t(kBarWaves)) {
    uint32_t k0 = 0u, k1 = 0u, k2 = 0u;  // the exchange only serves as the barrier here
    const bool ok = grid_exchange(a.bar, a.gen, a.spin_limit, wave, k0, k1, k2);
    if (lane == 0) {
      if (!ok) __hip_atomic_store(a.host_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      s_ok[wave] = ok ? 1u : 0u;
    }
  }
  __syncthreads();
  uint32_t oks = 1u;
#pragma unroll
  for (int q = 0; q < kBarWaves; q++) oks &= s_ok[q];
  if (oks == 0u) return;
  if (threadIdx.x == 0) __hip_atomic_store(a.done + blockIdx.x, a.gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  if (!active) {
    if (has_tiny) {
      tiny_finish<B, RANDOM>(a, my_piece - total, nidle, lane, v);
      if (a.stamps && lane == 0)
        __hip_atomic_fetch_max(reinterpret_cast<unsigned long long*>(a.stamps) + size_t(blockIdx.x) * 4 + 3,
                               static_cast<unsigned long long>(wall_clock64()), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
  }
  phase_stamp(a.stamps, 2);

  // ---- pass 2: the tensor's extremes, then quantise from registers ----------------
  {
    // All loads of a lane are in flight together (a lane reads a way that is not in use again from way 0:
    // a fold of maxima does not mind): one memory latency for the fold, not one per 64 ways.
    static_assert(kSlotWays == 2 * kWave, "two ways per lane");
    uint32_t kx = 0u, kn = 0u, kz = 0u;
    {
      const uint32_t w0 = lane < ways ? lane : 0u, w1 = lane + kWave < ways ? lane + kWave : 0u;
      unsigned long long v[6];
      v[0] = __hip_atomic_load(sl + w0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v[1] = __hip_atomic_load(sl + kSlotWays + w0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v[2] = __hip_atomic_load(sl + 2 * kSlotWays + w0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v[3] = __hip_atomic_load(sl + w1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v[4] = __hip_atomic_load(sl + kSlotWays + w1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      v[5] = __hip_atomic_load(sl + 2 * kSlotWays + w1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      uint32_t k[6];
#pragma unroll
      for (int i = 0; i < 6; i++) k[i] = (uint32_t(v[i] >> 32) == a.epoch) ? uint32_t(v[i]) : 0u;
      kx = k[0] > k[3] ? k[0] : k[3];
      kn = k[1] > k[4] ? k[1] : k[4];
      kz = k[2] > k[5] ? k[2] : k[5];
    }
    kx = wave_max_u32(kx);
    kn = wave_max_u32(kn);
    kz = wave_max_u32(kz);
    mx = from_okey(kx);
    mn = from_okey(~kn);
    if ((mn == 0.0f || mx == 0.0f) && kz != 0u) {
      // thrust::minmax_element returns the first extreme: a zero extreme carries the
      // sign of the first zero of the tensor.
      const float zv = xp[0xFFFFFFFEu - kz];
      if (mn == 0.0f) mn = zv;
      if (mx == 0.0f) mx = zv;
    }
  }
  const float gi = inverse_gap(mn, mx, B);
  if (pl == 0 && lane == 0) write_header(sg.out, B, n, mn, mx);

  uint8_t* __restrict__ pay = sg.out + 10;
  uint32_t draw[UNIT];
  if (RANDOM) {
    const uint32_t x0 = sg.seed + u0 * BPU + uint32_t(PRE) * stride_bytes;  // first row that draws for itself
#pragma unroll
    for (int q = 0; q < UNIT; q++) {
      const int jb = q / DPB, j = q % DPB;
      draw[q] = lcg_mul(j + 2) * (x0 + jb) + lcg_add(j + 2);
    }
  }
  auto register_rows = [&](auto whole) {
#pragma unroll
    for (int k = 0; k < KU; k++) {
      const uint32_t u = u0 + k * kWave;
      uint32_t packed;
      if (RANDOM && k < PRE) {
        float4 sc[H];
#pragma unroll
        for (int h = 0; h < H; h++) sc[h] = s_pre[(k * H + h) * kWave + lane];
        packed = quant_unit_prepared<B>(v[k], sc, mn, gi);
      } else {
        packed = quant_unit<B, RANDOM>(v[k], mn, gi, draw, stride_bytes);
      }
      if (decltype(whole)::value || u < u_end) {
#pragma unroll
        for (int jb = 0; jb < BPU; jb++) pay[size_t(u) * BPU + jb] = uint8_t(packed >> (8 * jb));
      }
    }
  };
  if (whole_rows) register_rows(std::true_type{}); else register_rows(std::false_type{});
  // The LDS rows follow the register rows of the same wave, so the draws simply go on.
  for (uint32_t r = 0; r < a.lds_rows; r++) {
    const uint32_t u = u0 + (uint32_t(KU) + r) * kWave;
    float4 f[H];
#pragma unroll
    for (int h = 0; h < H; h++) f[h] = s_mine[(r * H + h) * kWave + lane];
    const uint32_t packed = quant_unit<B, RANDOM>(f, mn, gi, draw, stride_bytes);
    if (u < u_end) {
#pragma unroll
      for (int jb = 0; jb < BPU; jb++) pay[size_t(u) * BPU + jb] = uint8_t(packed >> (8 * jb));
    }
  }
  // The unit that holds the end of the tensor, if its length is not a whole number of units.
  if (ends_tensor && lane == 0 && full_units * UNIT < n) {
    uint32_t d[UNIT];
#pragma unroll
    for (int q = 0; q < UNIT; q++) {
      const int jb = q / DPB, j = q % DPB;
      d[q] = lcg_mul(j + 2) * (sg.seed + full_units * BPU + jb) + lcg_add(j + 2);
    }
    quant_unit_ragged<B, RANDOM>(sg, mn, gi, full_units, d);
  }
  // the last of the workgroup's waves to get here leaves the reading (the waves hold pieces of different tensors
  // and lengths and no barrier joins them again)
  if (a.stamps && lane == 0)
    __hip_atomic_fetch_max(reinterpret_cast<unsigned long long*>(a.stamps) + size_t(blockIdx.x) * 4 + 3,
                           static_cast<unsigned long long>(wall_clock64()), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The 4*B bits holding the codes of the 4-element group that starts at element e.
template <int B>
__device__ __forceinline__ uint32_t group_bits(const uint8_t* __restrict__ pay, size_t e) {
  if (B == 1) return (uint32_t(pay[e >> 3]) >> (e & 4)) & 0xFu;
  if (B == 2) return pay[e >> 2];
  if (B == 4) return uint32_t(pay[e >> 1]) | (uint32_t(pay[(e >> 1) + 1]) << 8);
  return uint32_t(pay[e]) | (uint32_t(pay[e + 1]) << 8) | (uint32_t(pay[e + 2]) << 16) | (uint32_t(pay[e + 3]) << 24);
}

template <int B>
__device__ __forceinline__ float4 group_values(uint32_t bits, float gap, float mn) {
  constexpr uint32_t MASK = (1u << B) - 1u;
  // static_cast<float>(qval*gap + min_f), terngrad_body.h:127
  return make_float4(float(int((bits >> (0 * B)) & MASK)) * gap + mn, float(int((bits >> (1 * B)) & MASK)) * gap + mn,
                     float(int((bits >> (2 * B)) & MASK)) * gap + mn, float(int((bits >> (3 * B)) & MASK)) * gap + mn);
}

// STREAM selects the streaming store for the write-only case (the in-place add
// always streams).
template <int B, bool ADD, bool STREAM>
__device__ __forceinline__ void decode_tile(const DecSeg& sg, float mn, float gap, uint32_t cnt, uint32_t tile_in_seg) {
  constexpr int DPB = 8 / B;
  constexpr uint32_t MASK = (1u << B) - 1u;
  float* __restrict__ op = sg.out;
  const uint8_t* __restrict__ pay = sg.in + 10;
  const uint32_t g0 = tile_in_seg * uint32_t(kThreads * kDIters) + threadIdx.x;  // groups of 4 elements
  if (uint64_t(g0 - threadIdx.x + kThreads * kDIters) * 4 <= cnt) {
    // Whole tile inside the tensor.  All code loads of the lane are requested first (one after the other,
    // each behind the store before it, a workgroup lived through four memory latencies and the grid was
    // close to waiting for loads rather than for its stores); the stores then follow one per step, kept
    // apart by the barrier (streaming stores issued back to back run about 35 % slower here).
    uint32_t q[kDIters];
#pragma unroll
    for (int k = 0; k < kDIters; k++) q[k] = group_bits<B>(pay, size_t(g0 + k * kThreads) * 4);
    float4 o[kDIters];
    if (ADD) {
#pragma unroll
      for (int k = 0; k < kDIters; k++) o[k] = ld4_stream(op + size_t(g0 + k * kThreads) * 4);
    }
#pragma unroll
    for (int k = 0; k < kDIters; k++) {
      const size_t e = size_t(g0 + k * kThreads) * 4;
      float4 v = group_values<B>(q[k], gap, mn);
      if (ADD) { v.x += o[k].x; v.y += o[k].y; v.z += o[k].z; v.w += o[k].w; }
      if (ADD || STREAM) st4_stream(op + e, v); else st4(op + e, v);
      __asm__ volatile("" ::: "memory");
    }
    return;
  }
  for (int k = 0; k < kDIters; k++) {
    const size_t e = size_t(g0 + k * kThreads) * 4;
    if (e + 4 <= cnt) {
      float4 v = group_values<B>(group_bits<B>(pay, e), gap, mn);
      if (ADD) {
        const float4 o = ld4(op + e);
        v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
      }
      st4(op + e, v);
    } else {
      for (size_t i = e; i < cnt && i < e + 4; i++) {
        const uint32_t q = (pay[i / DPB] >> ((i % DPB) * B)) & MASK;
        const float v = float(int(q)) * gap + mn;
        op[i] = ADD ? v + op[i] : v;
      }
    }
  }
}

template <int B>
__device__ __forceinline__ void decode_dispatch(const DecSeg& sg, float mn, float gap, uint32_t cnt, uint32_t t, bool ss) {
  if (sg.add) decode_tile<B, true, true>(sg, mn, gap, cnt, t);
  else if (ss) decode_tile<B, false, true>(sg, mn, gap, cnt, t);
  else decode_tile<B, false, false>(sg, mn, gap, cnt, t);
}

template <int CAP>
__global__ __launch_bounds__(kThreads) void terngrad_decode_kernel(const DecArgs<CAP> a) {
  const int tile = blockIdx.x;
  const int s = find_segment<CAP>(a.tile_start, a.nseg, tile);
  const uint8_t* __restrict__ in = a.seg[s].in;
  const uint32_t bits = in[0];
  const uint32_t tail = in[1];
  uint32_t mb = 0, xb = 0;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    mb |= uint32_t(in[2 + i]) << (8 * i);
    xb |= uint32_t(in[6 + i]) << (8 * i);
  }
  if (bits != 1 && bits != 2 && bits != 4 && bits != 8) {
    if (threadIdx.x == 0 && tile == a.tile_start[s]) atomicOr(a.status, 1u);
    return;
  }
  const float mn = __uint_as_float(mb), mx = __uint_as_float(xb);
  const float gap = (mx - mn) / (float(1 << bits) - 1.0f);
  // ((in_size-10) << lg2(dpb)) - tail, terngrad_body.h:373; clamped to the output.
  int64_t c = int64_t(a.seg[s].in_size - 10) * int64_t(8 / bits) - int64_t(tail);
  if (c > a.seg[s].out_size) c = a.seg[s].out_size;
  if (c <= 0) return;
  const uint32_t cnt = static_cast<uint32_t>(c);
  const uint32_t t = static_cast<uint32_t>(tile - a.tile_start[s]);
  switch (bits) {
    case 1: decode_dispatch<1>(a.seg[s], mn, gap, cnt, t, a.stream_store != 0); break;
    case 2: decode_dispatch<2>(a.seg[s], mn, gap, cnt, t, a.stream_store != 0); break;
    case 4: decode_dispatch<4>(a.seg[s], mn, gap, cnt, t, a.stream_store != 0); break;
    default: decode_dispatch<8>(a.seg[s], mn, gap, cnt, t, a.stream_store != 0); break;
  }
}

// ---- several messages into one tensor ---------------------------------------
// The reference's root path hands terngrad_r_body the same output tensor once per
// gathered message (hp_cuda.cpp:421-439) and applies them one after the other.
// Here a tensor's messages are applied in one pass in call order: same sequence
// of fp32 operations per element, one read and one write of the tensor.
constexpr int kMultiSegs = 64;
constexpr int kMultiSlots = 448;
constexpr int kMultiSlotsPerSeg = 32;  // header fields of one tensor's messages are staged in LDS
constexpr int kMultiRep = 4;            // sub-tiles of kDecTile elements per workgroup of the multi-message decode
struct MSeg {
  float* out;
  int32_t out_size;
  int32_t first_slot;
  int32_t nslots;
  int32_t pad;
};
struct MSlot {
  const uint8_t* in;
  int32_t in_size;
  int32_t add;
};
struct MArgs {
  int32_t nseg;
  int32_t tile_start[kMultiSegs + 1];
  MSeg seg[kMultiSegs];
  MSlot slot[kMultiSlots];
  uint32_t* status;
};
static_assert(sizeof(MArgs) <= 9600, "kernel-argument budget");
// The same for tensors whose messages lie at a fixed distance from each other, have one size and are all added
// (the first one may also overwrite): the gathered slots of the reference's communication buffer
// (hp_cuda.cpp:421-439), of which the root leaves out its own - one gap of twice the distance is part of the form.  A tensor then takes 40 bytes of table whatever its number of messages, and ResNet-50's
// 161 tensors with 7 messages each are ONE launch instead of three.
constexpr int kStrideSegs = 208;
struct SSeg {
  float* out;
  const uint8_t* in0;  // the first message
  int64_t stride;      // bytes from one message to the next
  int32_t out_size;
  int32_t in_size;
  int16_t nslots;
  int16_t add0;        // the first message is added to what the tensor holds
  int16_t skip;        // messages from this one on lie one distance further (the root's own slot is left out); -1: none
  int16_t pad;
};
struct SArgs {
  int32_t nseg;
  int32_t tile_start[kStrideSegs + 1];
  SSeg seg[kStrideSegs];
  uint32_t* status;
};
static_assert(sizeof(SSeg) == 40 && sizeof(SArgs) <= 9600, "kernel-argument budget");
// What the kernel asks of either table: the tensor of a tile, its number of messages, and message j of it.
struct MultiMsg {
  const uint8_t* in;
  int32_t in_size;
  int32_t add;
};
__device__ __forceinline__ int multi_segment(const MArgs& a, int tile) { return find_segment<kMultiSegs>(a.tile_start, a.nseg, tile); }
__device__ __forceinline__ int multi_segment(const SArgs& a, int tile) { return find_segment<kStrideSegs>(a.tile_start, a.nseg, tile); }
__device__ __forceinline__ MultiMsg multi_message(const MArgs& a, int s, int j) {
  const MSlot& m = a.slot[a.seg[s].first_slot + j];
  return MultiMsg{m.in, m.in_size, m.add};
}
__device__ __forceinline__ MultiMsg multi_message(const SArgs& a, int s, int j) {
  const int skip = a.seg[s].skip;
  return MultiMsg{a.seg[s].in0 + int64_t(j + ((skip >= 0 && j >= skip) ? 1 : 0)) * a.seg[s].stride, a.seg[s].in_size,
                  j == 0 ? int32_t(a.seg[s].add0) : 1};
}

__device__ __forceinline__ uint32_t code_at(const uint8_t* __restrict__ pay, size_t i, uint32_t bits) {
  const uint32_t dpb = 8u / bits;
  return (uint32_t(pay[i / dpb]) >> ((i % dpb) * bits)) & ((1u << bits) - 1u);
}

// The common case of the multi-message decoder (NS complete 2-bit messages, 2 <= NS <= 8), for the sub-tiles of
// the workgroup that lie wholly inside the tensor; returns how many of its kMultiRep sub-tiles it has done.
// A wave owns kDIters * 64 consecutive groups, i.e. that many consecutive payload bytes of every message: each
// message costs the wave ONE load (a dword per lane) and the lanes pick their bytes out of it with cross-lane
// reads.  NS is a compile-time constant and the loads are unconditional: under per-message branches the
// compiler made every load wait for the one before, and each message then cost every sub-tile one more memory
// latency (7 messages into 25.5 M elements: 75 us; now 65, of which about 30 are the 22 operations per group
// and message).
template <int NS>
__device__ __forceinline__ uint32_t decode_two_bit_whole(float* __restrict__ op, uint32_t n, bool need_old, uint32_t sub0,
                                                             const uint8_t* const* s_pay, const float* s_gap,
                                                             const float* s_mn, const int32_t* s_add) {
  static_assert(kDIters * 4 <= kWave, "a wave's bytes of one message must fit one dword per lane");
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t whole = n / uint32_t(kThreads * kDIters * 4);  // sub-tiles wholly inside the tensor
  const uint32_t nfull = whole > sub0 ? (whole - sub0 < uint32_t(kMultiRep) ? whole - sub0 : uint32_t(kMultiRep)) : 0u;
  // per-message constants as wave-uniform values in scalar registers
  const uint8_t* pay[NS];
  float gap[NS], mn[NS];
  uint32_t addm = 0;
#pragma unroll
  for (int j = 0; j < NS; j++) {
    const uint64_t pj = reinterpret_cast<uint64_t>(s_pay[j]);
    // (the builtin returns a signed int: without the cast to uint32_t a low half with its top bit set would
    // be sign-extended over the high half)
    const uint32_t plo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(uint32_t(pj))));
    const uint32_t phi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(uint32_t(pj >> 32))));
    pay[j] = reinterpret_cast<const uint8_t*>(uint64_t(plo) | (uint64_t(phi) << 32));
    gap[j] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(s_gap[j])));
    mn[j] = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(s_mn[j])));
    addm |= (__builtin_amdgcn_readfirstlane(s_add[j]) != 0 ? 1u : 0u) << j;
  }
  const bool all_add = addm == (1u << NS) - 1u;  // the root's gather-decode: no select per value then
  const uint32_t pick = (lane / 4) * 4, shift = 8 * (lane & 3);
  auto first_group = [&](uint32_t rep) {  // the wave's first group of sub-tile rep
    return (sub0 + rep) * uint32_t(kThreads * kDIters) + (threadIdx.x / kWave) * uint32_t(kDIters * kWave);
  };
  auto request = [&](uint32_t rep, float4 (&acc)[kDIters], uint32_t (&dw)[NS]) {
    const uint32_t gw = first_group(rep);
    if (need_old) {
#pragma unroll
      for (int k = 0; k < kDIters; k++) acc[k] = ld4_stream(op + size_t(gw + k * kWave + lane) * 4);
    } else {
#pragma unroll
      for (int k = 0; k < kDIters; k++) acc[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int j = 0; j < NS; j++) dw[j] = as_global(reinterpret_cast<const u32u*>(pay[j] + gw + lane * 4))->v;  // the payload starts at byte 10
  };
  auto fold_store = [&](uint32_t rep, float4 (&acc)[kDIters], const uint32_t (&dw)[NS]) {
    const uint32_t gw = first_group(rep);
    if (all_add) {
#pragma unroll
      for (int j = 0; j < NS; j++)
#pragma unroll
        for (int k = 0; k < kDIters; k++) {
          const uint32_t byte = (__builtin_amdgcn_ds_bpermute(int(k * kWave + pick), int(dw[j])) >> shift) & 0xFFu;
          const float4 v = group_values<2>(byte, gap[j], mn[j]);
          acc[k].x = v.x + acc[k].x; acc[k].y = v.y + acc[k].y; acc[k].z = v.z + acc[k].z; acc[k].w = v.w + acc[k].w;
        }
    } else {
#pragma unroll
      for (int j = 0; j < NS; j++) {
        const bool add = (addm >> j) & 1u;
#pragma unroll
        for (int k = 0; k < kDIters; k++) {
          const uint32_t byte = (__builtin_amdgcn_ds_bpermute(int(k * kWave + pick), int(dw[j])) >> shift) & 0xFFu;
          const float4 v = group_values<2>(byte, gap[j], mn[j]);
          acc[k].x = add ? v.x + acc[k].x : v.x; acc[k].y = add ? v.y + acc[k].y : v.y;
          acc[k].z = add ? v.z + acc[k].z : v.z; acc[k].w = add ? v.w + acc[k].w : v.w;
        }
      }
    }
#pragma unroll
    for (int k = 0; k < kDIters; k++) {
      st4_stream(op + size_t(gw + k * kWave + lane) * 4, acc[k]);
      __asm__ volatile("" ::: "memory");
    }
  };
  float4 acc0[kDIters];
  uint32_t dw0[NS];
  for (uint32_t rep = 0; rep < nfull; rep++) {
    request(rep, acc0, dw0);
    fold_store(rep, acc0, dw0);
  }
  return nfull;
}

template <typename Args>
__global__ __launch_bounds__(kThreads) void terngrad_decode_multi_kernel(const Args a) {
  __shared__ float s_mn[kMultiSlotsPerSeg], s_gap[kMultiSlotsPerSeg];
  __shared__ uint32_t s_cnt[kMultiSlotsPerSeg], s_bits[kMultiSlotsPerSeg];
  __shared__ int32_t s_add[kMultiSlotsPerSeg];
  __shared__ const uint8_t* s_pay[kMultiSlotsPerSeg];
  const int tile = blockIdx.x;
  const int s = multi_segment(a, tile);
  float* __restrict__ op = a.seg[s].out;
  const int ns = a.seg[s].nslots;
  if (int(threadIdx.x) < ns) {
    const int j = threadIdx.x;
    const MultiMsg msg = multi_message(a, s, j);
    const uint8_t* in = msg.in;
    const uint32_t bits = in[0], tail = in[1];
    uint32_t mb = 0, xb = 0;
    for (int i = 0; i < 4; i++) {
      mb |= uint32_t(in[2 + i]) << (8 * i);
      xb |= uint32_t(in[6 + i]) << (8 * i);
    }
    uint32_t cnt = 0;
    float gap = 0.f;
    if (bits == 1 || bits == 2 || bits == 4 || bits == 8) {
      gap = (__uint_as_float(xb) - __uint_as_float(mb)) / (float(1 << bits) - 1.0f);
      int64_t c = int64_t(msg.in_size - 10) * int64_t(8 / bits) - int64_t(tail);
      if (c > a.seg[s].out_size) c = a.seg[s].out_size;
      cnt = c > 0 ? uint32_t(c) : 0u;
    } else if (tile == a.tile_start[s]) {
      atomicOr(a.status, 1u);
    }
    s_mn[j] = __uint_as_float(mb);
    s_gap[j] = gap;
    s_cnt[j] = cnt;
    s_bits[j] = cnt ? bits : 8u;
    s_add[j] = msg.add;
    s_pay[j] = in + 10;
  }
  __syncthreads();
  const uint32_t n = static_cast<uint32_t>(a.seg[s].out_size);
  const bool need_old = s_add[0] != 0;
  bool all_cover = true;  // every message covers the whole tensor (the normal case)
  for (int j = 0; j < ns; j++) all_cover = all_cover && s_cnt[j] == n;
  bool all_two_bit = true;  // ... and is a 2-bit message (the configuration the reference ships with)
  for (int j = 0; j < ns; j++) all_two_bit = all_two_bit && s_bits[j] == 2u;
  // The headers are parsed once per workgroup and serve kMultiRep consecutive sub-tiles.
  uint32_t rep_begin = 0;
  if (all_cover && all_two_bit && ns <= 8) {
    const uint32_t sub0 = static_cast<uint32_t>(tile - a.tile_start[s]) * kMultiRep;
    switch (ns) {  // the number of messages as a compile-time constant: straight-line code, all loads of a sub-tile in flight together
      case 2: rep_begin = decode_two_bit_whole<2>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      case 3: rep_begin = decode_two_bit_whole<3>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      case 4: rep_begin = decode_two_bit_whole<4>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      case 5: rep_begin = decode_two_bit_whole<5>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      case 6: rep_begin = decode_two_bit_whole<6>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      case 7: rep_begin = decode_two_bit_whole<7>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      case 8: rep_begin = decode_two_bit_whole<8>(op, n, need_old, sub0, s_pay, s_gap, s_mn, s_add); break;
      default: break;
    }
  }
  for (uint32_t rep = rep_begin; rep < uint32_t(kMultiRep); rep++) {
  const uint32_t g0 = (static_cast<uint32_t>(tile - a.tile_start[s]) * kMultiRep + rep) * uint32_t(kThreads * kDIters) + threadIdx.x;
  if (uint64_t(g0 - threadIdx.x) * 4 >= n) break;
  if (all_cover && all_two_bit && uint64_t(g0 - threadIdx.x + kThreads * kDIters) * 4 <= n) {
    // Whole tile of complete 2-bit messages.  A wave owns kDIters * 64 consecutive groups, i.e. that many
    // consecutive payload bytes of every message: each message costs the wave ONE load (a dword per lane)
    // and the lanes pick their bytes out of it with cross-lane reads, instead of one byte load per group
    // and message (28 loads per lane for 7 messages: the address pipeline, not memory, was the limit).
    static_assert(kDIters * 4 <= kWave, "a wave's bytes of one message must fit one dword per lane");
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t gw = g0 - threadIdx.x + (threadIdx.x / kWave) * uint32_t(kDIters * kWave);  // the wave's first group
    float4 acc[kDIters];
#pragma unroll
    for (int k = 0; k < kDIters; k++)
      acc[k] = need_old ? ld4_stream(op + size_t(gw + k * kWave + lane) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j0 = 0; j0 < ns; j0 += 8) {
      uint32_t dw[8];
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        dw[jj] = 0u;
        if (j0 + jj < ns && lane < uint32_t(kDIters * kWave / 4))
          dw[jj] = as_global(reinterpret_cast<const u32u*>(s_pay[j0 + jj] + gw + lane * 4))->v;  // the payload starts at byte 10
      }
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        if (j0 + jj < ns) {
          const float gap = s_gap[j0 + jj], mn = s_mn[j0 + jj];
          const bool add = s_add[j0 + jj] != 0;
#pragma unroll
          for (int k = 0; k < kDIters; k++) {
            const uint32_t byte = (__shfl(dw[jj], k * (kWave / 4) + lane / 4, kWave) >> (8 * (lane & 3))) & 0xFFu;
            const float4 v = group_values<2>(byte, gap, mn);
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
    for (int k = 0; k < kDIters; k++) {
      st4_stream(op + size_t(gw + k * kWave + lane) * 4, acc[k]);
      __asm__ volatile("" ::: "memory");
    }
    continue;
  }
  if (all_cover && uint64_t(g0 - threadIdx.x + kThreads * kDIters) * 4 <= n) {
    // Whole tile, every message complete, other widths: old values and the code bytes of up to 4 messages x 4
    // groups are requested together, then folded in message order.
    float4 acc[kDIters];
#pragma unroll
    for (int k = 0; k < kDIters; k++)
      acc[k] = need_old ? ld4_stream(op + size_t(g0 + k * kThreads) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j0 = 0; j0 < ns; j0 += 4) {
      uint32_t raw[4][kDIters];
#pragma unroll
      for (int jj = 0; jj < 4; jj++)
#pragma unroll
        for (int k = 0; k < kDIters; k++) {
          raw[jj][k] = 0;
          if (j0 + jj < ns) {
            const size_t e = size_t(g0 + k * kThreads) * 4;
            const uint32_t bits = s_bits[j0 + jj];
            const uint8_t* __restrict__ pay = s_pay[j0 + jj];
            if (bits == 1) raw[jj][k] = (uint32_t(pay[e >> 3]) >> (e & 4)) & 0xFu;
            else if (bits == 2) raw[jj][k] = pay[e >> 2];
            else if (bits == 4) raw[jj][k] = group_bits<4>(pay, e);
            else raw[jj][k] = group_bits<8>(pay, e);
          }
        }
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        if (j0 + jj < ns) {
          const uint32_t bits = s_bits[j0 + jj];
          const float gap = s_gap[j0 + jj], mn = s_mn[j0 + jj];
          const bool add = s_add[j0 + jj] != 0;
#pragma unroll
          for (int k = 0; k < kDIters; k++) {
            float4 v;
            if (bits == 1) v = group_values<1>(raw[jj][k], gap, mn);
            else if (bits == 2) v = group_values<2>(raw[jj][k], gap, mn);
            else if (bits == 4) v = group_values<4>(raw[jj][k], gap, mn);
            else v = group_values<8>(raw[jj][k], gap, mn);
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
    for (int k = 0; k < kDIters; k++) {
      st4_stream(op + size_t(g0 + k * kThreads) * 4, acc[k]);
      __asm__ volatile("" ::: "memory");
    }
    continue;
  }
  if (all_cover) {
    // The sub-tile that holds the end of the tensor, every message complete.  Its whole groups are handled like
    // the ones above, with the loads of all of a lane's groups and of up to 8 messages in flight together; only
    // the tensor's last, partial group goes element by element.  (Done element by element for the whole
    // sub-tile, each element waited for its own loads, message after message: up to 16 x (1 + messages)
    // memory latencies in a row in ONE workgroup.  Depending on n mod 4096 that tail alone took up to 35 us and
    // made the time of a 7-message decode jump up and down with the size of the tensor.)
    float4 acc[kDIters];
    bool live[kDIters];
#pragma unroll
    for (int k = 0; k < kDIters; k++) {
      const size_t e = size_t(g0 + k * kThreads) * 4;
      live[k] = e + 4 <= n;
      acc[k] = (live[k] && need_old) ? ld4(op + e) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int j0 = 0; j0 < ns; j0 += 8) {
      uint32_t raw[8][kDIters];
#pragma unroll
      for (int jj = 0; jj < 8; jj++)
#pragma unroll
        for (int k = 0; k < kDIters; k++) {
          raw[jj][k] = 0;
          if (j0 + jj < ns && live[k]) {
            const size_t e = size_t(g0 + k * kThreads) * 4;
            const uint32_t bits = s_bits[j0 + jj];
            global_ptr<uint8_t> pay = as_global(s_pay[j0 + jj]);
            if (bits == 1) raw[jj][k] = (uint32_t(pay[e >> 3]) >> (e & 4)) & 0xFu;
            else if (bits == 2) raw[jj][k] = pay[e >> 2];
            else if (bits == 4) raw[jj][k] = uint32_t(pay[e >> 1]) | (uint32_t(pay[(e >> 1) + 1]) << 8);
            else raw[jj][k] = uint32_t(pay[e]) | (uint32_t(pay[e + 1]) << 8) | (uint32_t(pay[e + 2]) << 16) | (uint32_t(pay[e + 3]) << 24);
          }
        }
#pragma unroll
      for (int jj = 0; jj < 8; jj++) {
        if (j0 + jj < ns) {
          const uint32_t bits = s_bits[j0 + jj];
          const float gap = s_gap[j0 + jj], mn = s_mn[j0 + jj];
          const bool add = s_add[j0 + jj] != 0;
#pragma unroll
          for (int k = 0; k < kDIters; k++) {
            float4 v;
            if (bits == 1) v = group_values<1>(raw[jj][k], gap, mn);
            else if (bits == 2) v = group_values<2>(raw[jj][k], gap, mn);
            else if (bits == 4) v = group_values<4>(raw[jj][k], gap, mn);
            else v = group_values<8>(raw[jj][k], gap, mn);
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
    for (int k = 0; k < kDIters; k++)
      if (live[k]) st4(op + size_t(g0 + k * kThreads) * 4, acc[k]);
    // the tensor's last 1..3 elements, if this lane owns them
#pragma unroll
    for (int k = 0; k < kDIters; k++) {
      const size_t e = size_t(g0 + k * kThreads) * 4;
      if (e < n && !live[k]) {
        float tail[3];
        const int lim = int(n - e);
        for (int i = 0; i < lim; i++) tail[i] = need_old ? op[e + i] : 0.f;
        for (int j = 0; j < ns; j++) {
          const float gap = s_gap[j], mn = s_mn[j];
          const bool add = s_add[j] != 0;
          for (int i = 0; i < lim; i++) {
            const float v = float(int(code_at(s_pay[j], e + i, s_bits[j]))) * gap + mn;  // terngrad_body.h:127, :158
            tail[i] = add ? v + tail[i] : v;
          }
        }
        for (int i = 0; i < lim; i++) op[e + i] = tail[i];
      }
    }
    continue;
  }
  // Messages that cover different numbers of elements (a clamped or malformed header): element by element.
  for (int k = 0; k < kDIters; k++) {
    const size_t e = size_t(g0 + k * kThreads) * 4;
    if (e >= n) break;
    const int lim = (n - e >= 4) ? 4 : int(n - e);
    for (int i = 0; i < lim; i++) {
      float acc = need_old ? op[e + i] : 0.f;
      bool touched = need_old;
      for (int j = 0; j < ns; j++) {
        if (e + i < s_cnt[j]) {
          const float v = float(int(code_at(s_pay[j], e + i, s_bits[j]))) * s_gap[j] + s_mn[j];  // terngrad_body.h:127, :158
          acc = s_add[j] ? v + acc : v;
          touched = true;
        }
      }
      if (touched) op[e + i] = acc;
    }
  }
  }
}

inline int32_t ceil_div(int64_t a, int64_t b) { return static_cast<int32_t>((a + b - 1) / b); }

uint64_t resident_spin_limit() {
  const int64_t ms = hpx::option(hpx::kOptTerngradBarrierMs);
  return uint64_t(ms < 0 ? 0 : ms) * 100000ull;  // wall_clock64 ticks at 100 MHz
}

// Workgroups of a resident launch: one per CU, or fewer when the option says so (a process that has been
// given only some of the CUs must say so: the workgroups of such a launch wait for each other, so all of them
// have to run at the same time).
int resident_grid(const hpx::Workspace* ws) {
  const int64_t cap = hpx::option(hpx::kOptTerngradResidentWorkgroups);
  return (cap > 0 && cap < ws->num_cus) ? int(cap) : ws->num_cus;
}

// Fills chunk_units / lds_rows when tensor (n, bits) fits the chip, and the streamed part as well when it is
// larger (the single launch then keeps the tensor's head on chip and streams the rest twice; measured against the
// two launches of small workgroups it stays ahead at every size: 160 M elements 205 against 228 us, 260 M 342
// against 369); false when the single launch is not to be used.
bool resident_plan(int32_t n, int bits, bool random, const hpx::Workspace* ws, ResArgs& ra) {
  const int64_t min_elems = hpx::option(hpx::kOptTerngradResidentMin);
  if (min_elems < 0 || n < min_elems || resident_grid(ws) <= 0 || resident_grid(ws) > kBarMaxWorkgroups) return false;
  const int unit = (8 / bits) > 4 ? (8 / bits) : 4;
  const int h = unit / 4;
  const int64_t full_units = n / unit;
  const int64_t grid = resident_grid(ws);
  const int64_t per_wg = (full_units + grid - 1) / grid;
  int64_t rows = (per_wg + kResThreads - 1) / kResThreads;
  if (rows < 1) rows = 1;
  const int reg_rows = res_reg_groups(bits, random) / h, lds_rows_max = kResLdsGroups / h;
  ra.stream_u0 = 0u;
  ra.stream_units = 0u;
  if (rows > reg_rows + lds_rows_max) {
    // Larger than the chip: every workgroup keeps a full share, the rest is streamed.
    const int64_t share = int64_t(reg_rows + lds_rows_max) * kResThreads;
    if (hpx::option(hpx::kOptTerngradResidentStreamed) == 0) return false;
    const int64_t rest = full_units - share * grid;
    ra.chunk_units = static_cast<uint32_t>(share);
    ra.reg_rows = static_cast<uint32_t>(reg_rows);
    ra.lds_rows = static_cast<uint32_t>(lds_rows_max);
    ra.pre_rows = 0u;
    ra.stream_u0 = static_cast<uint32_t>(share * grid);
    ra.stream_units = static_cast<uint32_t>(((rest + grid - 1) / grid + kWave - 1) / kWave * kWave);
    return true;
  }
  // The share itself is only rounded up to whole waves' worth of units, so that every CU has one (rounded to
  // whole rows, the headline tensor's 24.4 rows per workgroup became 25 rows for 250 workgroups and none for six).
  ra.chunk_units = static_cast<uint32_t>((per_wg + kWave - 1) / kWave * kWave);
  ra.reg_rows = static_cast<uint32_t>(rows < reg_rows ? rows : reg_rows);
  ra.lds_rows = rows > reg_rows ? static_cast<uint32_t>(rows - reg_rows) : 0u;
  const int spare_rows = (kResLdsTotalGroups - int(ra.lds_rows) * h) / h;
  ra.pre_rows = (random && spare_rows >= res_pre_rows(bits)) ? static_cast<uint32_t>(res_pre_rows(bits)) : 0u;
  return true;
}

template <int B, bool RANDOM, int PRE, bool STREAMED = false>
int launch_resident_as(const ResArgs& ra, int num_cus, hipStream_t st) {
  constexpr int H = ((8 / B) > 4 ? (8 / B) : 4) / 4;
  // The dynamic-LDS limit is a property of the function on one device: raise it once per device.
  static std::mutex attr_mu;
  static uint64_t attr_done = 0;  // bit d: done on device d (devices beyond 63 set it on every launch)
  {
    int dev = 0;
    HPX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(attr_mu);
    if (dev >= 64 || !(attr_done >> dev & 1)) {
      HPX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&terngrad_resident_kernel<B, RANDOM, PRE, STREAMED>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                  kResLdsTotalGroups * kResThreads * int(sizeof(float4))));
      if (dev < 64) attr_done |= uint64_t(1) << dev;
    }
  }
  const size_t lds = size_t(ra.lds_rows + PRE) * H * kResThreads * sizeof(float4);
  HPX_LAUNCH_LDS(STREAMED ? "terngrad_resident_streamed_kernel" : "terngrad_resident_kernel", hpx::g_prof_on,
                 (terngrad_resident_kernel<B, RANDOM, PRE, STREAMED>), dim3(num_cus), dim3(kResThreads), lds, st, ra);
  HPX_HIP(hipGetLastError());
  return HPX_OK;
}

template <int B>
int launch_resident_bits(const ResArgs& ra, int num_cus, hipStream_t st) {
  if (ra.stream_units)
    return ra.seg.random ? launch_resident_as<B, true, 0, true>(ra, num_cus, st) : launch_resident_as<B, false, 0, true>(ra, num_cus, st);
  if (!ra.seg.random) return launch_resident_as<B, false, 0>(ra, num_cus, st);
  if (ra.pre_rows) return launch_resident_as<B, true, res_pre_rows(B)>(ra, num_cus, st);
  return launch_resident_as<B, true, 0>(ra, num_cus, st);
}

// The tag of the next launch that uses the reduction slots / the exchange memory.
int next_slot_epoch(hpx::Workspace* ws, hipStream_t st) {
  if (++ws->epoch == 0) {
    // The 32-bit tag wrapped: start over from cleared slots.
    HPX_HIP(hipStreamSynchronize(st));
    HPX_HIP(hipMemset(ws->slots, 0, ws->slot_words * sizeof(uint64_t)));
    ws->epoch = 1;
  }
  return HPX_OK;
}
int next_barrier_generation(hpx::Workspace* ws, hipStream_t st) {
  if (++ws->bar_gen == 0) {
    // The 32-bit generation wrapped: start over from cleared exchange memory.
    HPX_HIP(hipStreamSynchronize(st));
    HPX_HIP(hipMemset(ws->bar, 0, hpx::kBarWords * sizeof(uint32_t)));
    // the stream is idle: whatever the log still held has finished, and the workgroups' words start over too
    if (!hpx::barrier_expired(ws)) ws->resident_log.clear([](hpx::Workspace::ResidentMark) {});
    for (int w = 0; w < hpx::kBarMaxWorkgroups; w++) ws->done[w] = 0;
    ws->bar_gen = 1;
  }
  return HPX_OK;
}

// How many of the first tensors of a list can share one resident launch: they have the width and rounding
// mode of the first, are at most kCapLarge, and their pieces at the largest row count fit the chip.
int resident_multi_extent(int count, const int32_t* in_sizes, const uint8_t* bitwidths, const int32_t* enable_randoms,
                          const hpx::Workspace* ws) {
  if (resident_grid(ws) <= 0 || resident_grid(ws) > kBarMaxWorkgroups) return 0;
  const int bits = bitwidths[0];
  const bool random = enable_randoms[0] != 0;
  const int unit = (8 / bits) > 4 ? (8 / bits) : 4;
  const int h = unit / 4;
  const int64_t rows_max = res_reg_groups(bits, random) / h + kResLdsGroups / h;
  const int64_t waves = int64_t(resident_grid(ws)) * (kResThreads / kWave);
  int64_t pieces = 0;
  int k = 0;
  for (; k < count && k < kCapLarge; k++) {
    if (bitwidths[k] != bits || (enable_randoms[k] != 0) != random) break;
    const int64_t p = (in_sizes[k] / unit + rows_max * kWave - 1) / (rows_max * kWave);
    pieces += p < 1 ? 1 : p;
    if (pieces > waves) break;
  }
  return k;
}

// Rows per piece for a call with several tensors, or false when the call does not qualify: one bit
// width and rounding mode, a total of at least the resident threshold, and all pieces on the chip at once.
bool resident_multi_plan(int count, const int32_t* in_sizes, const uint8_t* bitwidths, const int32_t* enable_randoms,
                         const hpx::Workspace* ws, ResMultiArgs& ma, uint32_t& pre_rows) {
  const int64_t min_elems = hpx::option(hpx::kOptTerngradResidentMin);
  if (min_elems < 0 || hpx::option(hpx::kOptTerngradResidentBucket) == 0) return false;
  if (count < 2 || count > kCapLarge || resident_grid(ws) <= 0 || resident_grid(ws) > kBarMaxWorkgroups) return false;
  const int bits = bitwidths[0];
  const bool random = enable_randoms[0] != 0;
  int64_t total = 0;
  for (int i = 0; i < count; i++) {
    if (bitwidths[i] != bits || (enable_randoms[i] != 0) != random) return false;
    total += in_sizes[i];
  }
  if (total < min_elems) return false;
  const int unit = (8 / bits) > 4 ? (8 / bits) : 4;
  const int h = unit / 4;
  const int reg_rows = res_reg_groups(bits, random) / h, lds_rows_max = kResLdsGroups / h;
  const int64_t waves = int64_t(resident_grid(ws)) * (kResThreads / kWave);
  int64_t total_units = 0;
  for (int i = 0; i < count; i++) total_units += in_sizes[i] / unit;
  // Tiny tensors take no piece; kTinyPerWave of them share a wave that has none.  (With nothing but tiny tensors
  // there would be no piece at all: then they are tensors like any other.)
  int ntiny = 0;
  for (int i = 0; i < count; i++) ntiny += in_sizes[i] / unit <= tiny_rows(bits) * kWave ? 1 : 0;
  if (ntiny == count) ntiny = 0;
  const bool riders = ntiny > 0;
  auto is_tiny = [&](int i) { return riders && in_sizes[i] / unit <= tiny_rows(bits) * kWave; };
  const int64_t tiny_waves = (ntiny + kTinyPerWave - 1) / kTinyPerWave;
  int64_t rows = (total_units + waves * kWave - 1) / (waves * kWave);
  if (rows < 1) rows = 1;
  for (; rows <= reg_rows + lds_rows_max; rows++) {
    int64_t pieces = 0;
    for (int i = 0; i < count; i++) {
      const int64_t p = (in_sizes[i] / unit + rows * kWave - 1) / (rows * kWave);
      pieces += is_tiny(i) ? 0 : (p < 1 ? 1 : p);
    }
    if (pieces + tiny_waves <= waves) break;
  }
  if (rows > reg_rows + lds_rows_max) return false;
  ma.rows = static_cast<uint32_t>(rows);
  ma.lds_rows = rows > reg_rows ? static_cast<uint32_t>(rows - reg_rows) : 0u;
  // prepared rows: the full set, or three quarters or half of it when the tensors' LDS rows leave no room for more
  const int spare_rows = (kResLdsTotalGroups - int(ma.lds_rows) * h) / h;
  pre_rows = 0u;
  if (random && spare_rows >= res_pre_rows(bits)) pre_rows = static_cast<uint32_t>(res_pre_rows(bits));
  else if (random && spare_rows >= res_pre_rows(bits) * 3 / 4) pre_rows = static_cast<uint32_t>(res_pre_rows(bits) * 3 / 4);
  else if (random && spare_rows >= res_pre_rows(bits) / 2) pre_rows = static_cast<uint32_t>(res_pre_rows(bits) / 2);
  ma.nseg = count;
  ma.ntiny = 0;
  ma.piece_start[0] = 0;
  for (int i = 0; i < count; i++) {
    const int64_t p = (in_sizes[i] / unit + rows * kWave - 1) / (rows * kWave);
    ma.piece_start[i + 1] = ma.piece_start[i] + (is_tiny(i) ? 0 : static_cast<int32_t>(p < 1 ? 1 : p));
    if (is_tiny(i)) ma.tiny[ma.ntiny++] = static_cast<int16_t>(i);
  }
  return true;
}

template <int B, bool RANDOM, int PRE>
int launch_resident_multi_as(const ResMultiArgs& ma, int num_cus, hipStream_t st) {
  constexpr int H = ((8 / B) > 4 ? (8 / B) : 4) / 4;
  static std::mutex attr_mu;
  static uint64_t attr_done = 0;  // bit d: done on device d (devices beyond 63 set it on every launch)
  {
    int dev = 0;
    HPX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> g(attr_mu);
    if (dev >= 64 || !(attr_done >> dev & 1)) {
      HPX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&terngrad_resident_multi_kernel<B, RANDOM, PRE>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                  kResLdsTotalGroups * kResThreads * int(sizeof(float4))));
      if (dev < 64) attr_done |= uint64_t(1) << dev;
    }
  }
  const size_t lds = size_t(ma.lds_rows + PRE) * H * kResThreads * sizeof(float4);
  HPX_LAUNCH_LDS("terngrad_resident_multi_kernel", hpx::g_prof_on, (terngrad_resident_multi_kernel<B, RANDOM, PRE>),
                 dim3(num_cus), dim3(kResThreads), lds, st, ma);
  HPX_HIP(hipGetLastError());
  return HPX_OK;
}

template <int B>
int launch_resident_multi_bits(const ResMultiArgs& ma, bool random, uint32_t pre_rows, int num_cus, hipStream_t st) {
  if (!random) return launch_resident_multi_as<B, false, 0>(ma, num_cus, st);
  if (pre_rows == uint32_t(res_pre_rows(B))) return launch_resident_multi_as<B, true, res_pre_rows(B)>(ma, num_cus, st);
  if (pre_rows == uint32_t(res_pre_rows(B) * 3 / 4)) return launch_resident_multi_as<B, true, res_pre_rows(B) * 3 / 4>(ma, num_cus, st);
  if (pre_rows == uint32_t(res_pre_rows(B) / 2)) return launch_resident_multi_as<B, true, res_pre_rows(B) / 2>(ma, num_cus, st);
  return launch_resident_multi_as<B, true, 0>(ma, num_cus, st);
}

int launch_resident_multi(const ResMultiArgs& ma, int bits, bool random, uint32_t pre_rows, int num_cus, hipStream_t st) {
  switch (bits) {
    case 1: return launch_resident_multi_bits<1>(ma, random, pre_rows, num_cus, st);
    case 2: return launch_resident_multi_bits<2>(ma, random, pre_rows, num_cus, st);
    case 4: return launch_resident_multi_bits<4>(ma, random, pre_rows, num_cus, st);
    default: return launch_resident_multi_bits<8>(ma, random, pre_rows, num_cus, st);
  }
}

int launch_resident(const ResArgs& ra, int num_cus, hipStream_t st) {
  switch (ra.seg.bits) {
    case 1: return launch_resident_bits<1>(ra, num_cus, st);
    case 2: return launch_resident_bits<2>(ra, num_cus, st);
    case 4: return launch_resident_bits<4>(ra, num_cus, st);
    default: return launch_resident_bits<8>(ra, num_cus, st);
  }
}

template <int CAP>
int launch_encode(int count, const float* const* ins, const int32_t* in_sizes, uint8_t* const* outs,
                  const int32_t* out_sizes, const uint8_t* bitwidths, const int32_t* enable_randoms,
                  const uint64_t* seeds, uint64_t* slot_base, uint32_t epoch, hipStream_t st, bool timed = true) {
  // timed = false: the launches are never bracketed by profiling events (creating an event allocates)
  const bool prof = timed && hpx::g_prof_on;
  EncArgs<CAP> a;
  int i = 0;
  while (i < count) {
    const int first = i;
    a.nseg = 0;
    a.tile_start[0] = 0;
    a.slots = slot_base + size_t(first) * kSlotsPerTensor;
    a.epoch = epoch;
    int32_t qstart[CAP + 1];
    qstart[0] = 0;
    while (i < count && a.nseg < CAP) {
      const int32_t n = in_sizes[i];
      const int b = bitwidths[i];
      const int unit = (8 / b) > 4 ? (8 / b) : 4;
      const int32_t rt = ceil_div(n, kRedTile);
      const int32_t qt = ceil_div(ceil_div(n, unit), kThreads * kQIters);
      if (int64_t(a.tile_start[a.nseg]) + rt > INT32_MAX || int64_t(qstart[a.nseg]) + qt > INT32_MAX) break;
      const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
      a.seg[a.nseg] = EncSeg{ins[i], outs[i], n, out_sizes[i], static_cast<uint32_t>(seed),
                             static_cast<uint8_t>(b), static_cast<uint8_t>(enable_randoms[i] != 0), 0};
      a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + rt;
      qstart[a.nseg + 1] = qstart[a.nseg] + qt;
      a.nseg++;
      i++;
    }
    HPX_LAUNCH_LDS("terngrad_minmax_kernel", prof, terngrad_minmax_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), 0, st, a);
    HPX_HIP(hipGetLastError());
    for (int k = 0; k <= a.nseg; k++) a.tile_start[k] = qstart[k];
    HPX_LAUNCH_LDS("terngrad_quant_kernel", prof, terngrad_quant_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), 0, st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

template <int CAP>
int launch_decode(int count, float* const* outs, const int32_t* out_sizes, const uint8_t* const* ins,
                  const int32_t* in_sizes, const int32_t* is_add_tos, uint32_t* status, hipStream_t st) {
  DecArgs<CAP> a;
  a.status = status;
  size_t out_bytes = 0;
  for (int k = 0; k < count; k++) out_bytes += out_sizes[k] > 0 ? size_t(out_sizes[k]) * 4 : 0;
  a.stream_store = out_bytes <= hpx::stream_store_max_bytes();
  int i = 0;
  while (i < count) {
    a.nseg = 0;
    a.tile_start[0] = 0;
    bool any_add = false;
    while (i < count && a.nseg < CAP) {
      HPX_ARG(out_sizes[i] >= 0 && in_sizes[i] >= 10, "hpx_terngrad_decode: message %d: out_size %d, in_size %d", i,
              out_sizes[i], in_sizes[i]);
      if (out_sizes[i] > 0) {
        HPX_ARG(outs[i] && ins[i], "hpx_terngrad_decode: message %d has a null pointer", i);
        const int32_t t = ceil_div(out_sizes[i], kDecTile);
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;
        a.seg[a.nseg] = DecSeg{outs[i], ins[i], out_sizes[i], in_sizes[i], is_add_tos[i] != 0, 0};
        any_add = any_add || is_add_tos[i] != 0;
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
      }
      i++;
    }
    if (a.nseg == 0) continue;
    // write mode throughout: a pure write stream, held to four workgroups per CU (hpx_common.h)
    const int pad = (a.stream_store && !any_add) ? hpx::kWriteStreamPadLds4 : 0;
    HPX_LAUNCH_LDS("terngrad_decode_kernel", hpx::g_prof_on, terngrad_decode_kernel<CAP>, dim3(a.tile_start[a.nseg]), dim3(kThreads), pad, st, a);
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

int launch_decode_multi(int count, float* const* outs, const int32_t* out_sizes, const uint8_t* const* ins,
                        const int32_t* in_sizes, const int32_t* is_add_tos, uint32_t* status, hipStream_t st) {
  std::vector<char> done(count, 0);
  int left = 0;
  for (int j = 0; j < count; j++) {
    HPX_ARG(out_sizes[j] >= 0 && in_sizes[j] >= 10, "hpx_terngrad_decode: message %d: out_size %d, in_size %d", j,
            out_sizes[j], in_sizes[j]);
    if (out_sizes[j] == 0) { done[j] = 1; continue; }
    HPX_ARG(outs[j] && ins[j], "hpx_terngrad_decode: message %d has a null pointer", j);
    left++;
  }
  if (left == 0) return HPX_OK;
  auto tiles_of = [](int32_t n) { return ceil_div(n, kDecTile * kMultiRep); };
  {
    // The fixed-distance form when the whole call fits it: at most kStrideSegs tensors, every tensor's messages (in
    // call order) at one distance from each other, of one size, and all but the first added.
    SArgs sa;
    sa.status = status;
    sa.nseg = 0;
    std::unordered_map<float*, int> index;
    std::vector<const uint8_t*> last(kStrideSegs, nullptr);
    bool fits = true;
    for (int j = 0; j < count && fits; j++) {
      if (out_sizes[j] == 0) continue;
      auto it = index.find(outs[j]);
      if (it == index.end()) {
        if (sa.nseg == kStrideSegs) { fits = false; break; }
        index[outs[j]] = sa.nseg;
        sa.seg[sa.nseg] = SSeg{outs[j], ins[j], 0, out_sizes[j], in_sizes[j], 1, int16_t(is_add_tos[j] != 0), -1, 0};
        last[sa.nseg] = ins[j];
        sa.nseg++;
        continue;
      }
      SSeg& g = sa.seg[it->second];
      const int64_t step = static_cast<int64_t>(reinterpret_cast<intptr_t>(ins[j]) - reinterpret_cast<intptr_t>(last[it->second]));  // addresses, not elements of one array
      if (g.nslots == kMultiSlotsPerSeg || is_add_tos[j] == 0 || in_sizes[j] != g.in_size || out_sizes[j] != g.out_size) fits = false;
      else if (g.nslots == 1) g.stride = step;
      else if (step == g.stride) {}
      else if (g.skip < 0 && step == 2 * g.stride) g.skip = g.nslots;                                   // the gap
      else if (g.skip < 0 && g.nslots == 2 && 2 * step == g.stride) { g.stride = step; g.skip = 1; }    // the gap came first
      else fits = false;
      last[it->second] = ins[j];
      g.nslots++;
    }
    int64_t tiles = 0;
    sa.tile_start[0] = 0;
    for (int k = 0; k < sa.nseg && fits; k++) {
      tiles += tiles_of(sa.seg[k].out_size);
      if (tiles > INT32_MAX) fits = false;
      sa.tile_start[k + 1] = int32_t(tiles);
    }
    if (fits && sa.nseg > 0) {
      HPX_LAUNCH("terngrad_decode_multi_kernel", terngrad_decode_multi_kernel<SArgs>, dim3(sa.tile_start[sa.nseg]), dim3(kThreads), st, sa);
      HPX_HIP(hipGetLastError());
      return HPX_OK;
    }
  }
  MArgs a;
  a.status = status;
  while (left > 0) {
    const std::vector<MultiGroup> groups = plan_multi_launch(count, outs, out_sizes, done, tiles_of);
    a.nseg = 0;
    a.tile_start[0] = 0;
    int nslots = 0;
    for (const MultiGroup& g : groups) {
      a.seg[a.nseg] = MSeg{g.out, g.n, nslots, static_cast<int32_t>(g.msgs.size()), 0};
      for (int m : g.msgs) a.slot[nslots++] = MSlot{ins[m], in_sizes[m], is_add_tos[m] != 0};
      a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + tiles_of(g.n);
      a.nseg++;
    }
    if (nslots == 0) { hpx::set_error("hpx_terngrad_decode: could not place the remaining messages"); return HPX_ERR_ARG; }
    left -= nslots;
    HPX_LAUNCH("terngrad_decode_multi_kernel", terngrad_decode_multi_kernel<MArgs>, dim3(a.tile_start[a.nseg]), dim3(kThreads), st, a);
    HPX_HIP(hipGetLastError());
  }
  return HPX_OK;
}

// Encodes the listed tensors with the tiled pair of kernels (ws->mu held).  `seeds` may be null (wall clock).
int encode_tiled(hpx::Workspace* ws, hipStream_t st, int count, const float* const* ins, const int32_t* in_sizes,
                 uint8_t* const* outs, const int32_t* out_sizes, const uint8_t* bitwidths, const int32_t* enable_randoms,
                 const uint64_t* seeds) {
  int rc = hpx::ensure_slots(ws, size_t(count) * kSlotsPerTensor);
  if (rc != HPX_OK) return rc;
  rc = next_slot_epoch(ws, st);  // its own tag: the slots may hold words of an earlier launch of the same call
  if (rc != HPX_OK) return rc;
  if (count <= kCapSmall)
    return launch_encode<kCapSmall>(count, ins, in_sizes, outs, out_sizes, bitwidths, enable_randoms, seeds, ws->slots,
                                    ws->epoch, st);
  return launch_encode<kCapLarge>(count, ins, in_sizes, outs, out_sizes, bitwidths, enable_randoms, seeds, ws->slots,
                                  ws->epoch, st);
}

// A barrier kernel on this stream gave up waiting (ws->mu held): barrier kernels are switched off for the
// stream and every tensor they have encoded since the stream was last known to be good is queued again
// through the tiled kernels, with the seed it was given the first time, so the same message comes out.
inline auto recycle_into(hpx::Workspace*) {
  return [](hpx::Workspace::ResidentMark) {};  // marks own nothing
}

int repair_resident_log(hpx::Workspace* ws, hipStream_t st) {
  ws->barrier_broken = true;
  if (ws->resident_log.empty()) return HPX_OK;
  const int m = int(ws->resident_log.size());
  std::vector<const float*> t_in(m);
  std::vector<uint8_t*> t_out(m);
  std::vector<int32_t> t_isz(m), t_osz(m), t_rnd(m);
  std::vector<uint8_t> t_bits(m);
  std::vector<uint64_t> t_seed(m);
  for (int k = 0; k < m; k++) {
    const hpx::Workspace::ResidentRec& r = ws->resident_log.records()[k];
    t_in[k] = r.x; t_out[k] = r.out; t_isz[k] = r.n; t_osz[k] = r.out_size;
    t_rnd[k] = r.random; t_bits[k] = r.bits; t_seed[k] = r.seed;
  }
  ws->resident_log.clear(recycle_into(ws));
  ws->repaired += uint64_t(m);
  return encode_tiled(ws, st, m, t_in.data(), t_isz.data(), t_out.data(), t_osz.data(), t_bits.data(), t_rnd.data(),
                      t_seed.data());
}

// Drops the records of earlier launches whose workgroups have all come through their barrier, while the
// expiry flag is down: such a launch will never have to be repeated, its buffers are the caller's again and must
// not be named by a later repair (ws->mu held, barrier memory ensured).
void prune_resident_log(hpx::Workspace* ws) {
  if (!ws->done) return;
  const volatile uint32_t* done = ws->done;
  ws->resident_log.prune(
      [done](hpx::Workspace::ResidentMark m) {
        for (int w = 0; w < m.grid; w++)
          if (int32_t(done[w] - m.gen) < 0) return false;  // generations only grow (a wrap clears the words)
        return true;
      },
      [ws] { return !hpx::barrier_expired(ws); }, recycle_into(ws));
}

// Marks the log behind a barrier launch that has just been queued (ws->mu held).
void mark_resident_log(hpx::Workspace* ws, uint32_t gen, int grid) {
  ws->resident_log.mark(hpx::Workspace::ResidentMark{gen, grid}, recycle_into(ws));
}

// Waits for the stream and settles the log of barrier-kernel encodes: cleared if they all got through, encoded
// again if one gave up (ws->mu held).
int settle_resident_log(hpx::Workspace* ws, hipStream_t st) {
  HPX_HIP(hipStreamSynchronize(st));
  if (!hpx::barrier_expired(ws)) {
    ws->resident_log.clear(recycle_into(ws));
    return HPX_OK;
  }
  // every kernel of the stream has finished: nothing can raise the flag again behind this
  *reinterpret_cast<volatile uint32_t*>(ws->pinned + hpx::kPinnedFlagOffset) = 0;
  const int rc = repair_resident_log(ws, st);
  if (rc != HPX_OK) return rc;
  HPX_HIP(hipStreamSynchronize(st));
  return HPX_OK;
}

// ---- encode without allocation ------------------------------------------------------
constexpr int kNoAllocMaxTensors = kCapLarge;
constexpr uint32_t kNoAllocWords = uint32_t(kNoAllocMaxTensors) * kSlotsPerTensor;
static_assert(sizeof(scratch) == size_t(kNoAllocWords) * sizeof(unsigned long long), "scratch must hold the slots of one full table");

__global__ __launch_bounds__(kThreads) void terngrad_scratch_clear_kernel(unsigned long long* __restrict__ p, uint32_t words) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i < words) p[i] = 0ull;
}

// Device address of `scratch` on the current device (every GPU holds its own copy at its own address),
// looked up once per device.
constexpr int kNoAllocMaxDevices = 64;
int scratch_address(unsigned long long** out) {
  static std::mutex mu;
  static unsigned long long* ptr[kNoAllocMaxDevices] = {};
  int dev = 0;
  HPX_HIP(hipGetDevice(&dev));
  HPX_ARG(dev >= 0 && dev < kNoAllocMaxDevices, "hpx_terngrad_encode_noalloc: device %d (at most %d devices)", dev, kNoAllocMaxDevices);
  std::lock_guard<std::mutex> g(mu);
  if (!ptr[dev]) {
    unsigned long long* p = nullptr;
    HPX_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
    HPX_ARG(p != nullptr, "hpx_terngrad_encode_noalloc: no device address for the scratch array");
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return HPX_OK;
}

// Measurement aid: where resident launches leave their phase stamps (null: nowhere).
std::atomic<uint64_t*> g_phase_stamps{nullptr};
std::atomic<int32_t> g_phase_capacity{0};
uint64_t* phase_stamps_for(int grid) {
  uint64_t* p = g_phase_stamps.load(std::memory_order_relaxed);
  return p && grid <= g_phase_capacity.load(std::memory_order_relaxed) ? p : nullptr;
}

constexpr size_t kResidentLogMax = 4096;  // records kept before hpx_terngrad_encode settles the log itself

}  // namespace

HPX_API int hpx_terngrad_encode(int count, const float* const* ins, const int32_t* in_sizes,
                                uint8_t* const* outs, const int32_t* out_sizes,
                                const uint8_t* bitwidths, const int32_t* enable_randoms,
                                const uint64_t* seeds, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_terngrad_encode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(ins && in_sizes && outs && out_sizes && bitwidths && enable_randoms,
          "hpx_terngrad_encode: null argument array");
  for (int i = 0; i < count; i++) {
    const uint8_t b = bitwidths[i];
    if (!(b == 1 || b == 2 || b == 4 || b == 8)) {
      hpx::set_error("Invalid value of bitwidth, check value: bitwidth=%d", int(b));
      return HPX_ERR_BODY;
    }
    HPX_ARG(in_sizes[i] > 0, "hpx_terngrad_encode: tensor %d has size %d (must be positive)", i, in_sizes[i]);
    HPX_ARG(ins[i] && outs[i], "hpx_terngrad_encode: tensor %d has a null pointer", i);
    const int64_t need = 10 + (int64_t(in_sizes[i]) + 8 / b - 1) / (8 / b);
    HPX_ARG(out_sizes[i] >= need, "hpx_terngrad_encode: tensor %d needs %lld output bytes, got %d", i,
            static_cast<long long>(need), out_sizes[i]);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc = hpx::reject_capture(st, "hpx_terngrad_encode");
  if (rc != HPX_OK) return rc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  rc = hpx::ensure_workspace(ws, 0);
  if (rc != HPX_OK) return rc;
  rc = hpx::ensure_slots(ws, size_t(count) * kSlotsPerTensor);
  if (rc != HPX_OK) return rc;
  rc = hpx::ensure_barrier(ws);
  if (rc != HPX_OK) return rc;

  // A barrier kernel of an earlier call on this stream gave up waiting: its messages are queued again
  // through the tiled kernels before this call's work, and this call takes the tiled kernels too.  (The
  // flag stays up until hpx_terngrad_encode_status has waited for the stream: workgroups of that
  // kernel may still be on their way out.)
  prune_resident_log(ws);
  if (!ws->barrier_broken && hpx::barrier_expired(ws)) {
    rc = repair_resident_log(ws, st);
    if (rc != HPX_OK) return rc;
  }
  if (ws->resident_log.size() + size_t(count) > kResidentLogMax) {
    rc = settle_resident_log(ws, st);
    if (rc != HPX_OK) return rc;
  }
  uint32_t* expired = reinterpret_cast<uint32_t*>(ws->pinned + hpx::kPinnedFlagOffset);
  // Consecutive tensors of one width and rounding mode that fit the chip together and add up to the
  // resident threshold take one resident launch per such group; a remaining tensor that is large enough
  // takes the single-tensor resident kernel; the rest goes to the tiled pair of kernels.
  std::vector<int> tiled;
  tiled.reserve(count);
  const bool buckets = count >= 2 && hpx::option(hpx::kOptTerngradResidentBucket) != 0 &&
                       hpx::option(hpx::kOptTerngradResidentMin) >= 0;
  auto log_resident = [&](const EncSeg& sg, uint64_t seed) {
    ws->resident_log.add(hpx::Workspace::ResidentRec{sg.x, sg.out, sg.n, sg.out_size, seed, sg.bits, sg.random});
  };
  int i = 0;
  while (i < count) {
    int j = i;
    if (buckets && !ws->barrier_broken) j = i + resident_multi_extent(count - i, in_sizes + i, bitwidths + i, enable_randoms + i, ws);
    if (j - i >= 2) {
      ResMultiArgs ma;
      uint32_t pre_rows = 0;
      if (resident_multi_plan(j - i, in_sizes + i, bitwidths + i, enable_randoms + i, ws, ma, pre_rows) &&
          hpx::claim_barrier_kernels(ws)) {
        for (int k = i; k < j; k++) {
          const uint64_t seed = seeds ? seeds[k] : hpx::clock_seed();
          ma.seg[k - i] = EncSeg{ins[k], outs[k], in_sizes[k], out_sizes[k], static_cast<uint32_t>(seed), bitwidths[k],
                                 static_cast<uint8_t>(enable_randoms[k] != 0), 0};
          log_resident(ma.seg[k - i], seed);
        }
        rc = next_barrier_generation(ws, st);
        if (rc != HPX_OK) return rc;
        rc = next_slot_epoch(ws, st);
        if (rc != HPX_OK) return rc;
        ma.slots = ws->slots;
        ma.epoch = ws->epoch;
        ma.gen = ws->bar_gen;
        ma.bar = reinterpret_cast<uint64_t*>(ws->bar);
        ma.host_flag = expired;
        ma.spin_limit = resident_spin_limit();
        ma.stamps = phase_stamps_for(resident_grid(ws));
        ma.done = ws->done;
        rc = launch_resident_multi(ma, bitwidths[i], enable_randoms[i] != 0, pre_rows, resident_grid(ws), st);
        if (rc != HPX_OK) return rc;
        mark_resident_log(ws, ma.gen, resident_grid(ws));
        i = j;
        continue;
      }
    }
    // tensors i .. max(j, i + 1) - 1, each on its own
    const int stop = j > i ? j : i + 1;
    for (; i < stop; i++) {
      ResArgs ra;
      if (ws->barrier_broken || !resident_plan(in_sizes[i], bitwidths[i], enable_randoms[i] != 0, ws, ra) ||
          !hpx::claim_barrier_kernels(ws)) {
        tiled.push_back(i);
        continue;
      }
      const uint64_t seed = seeds ? seeds[i] : hpx::clock_seed();
      ra.seg = EncSeg{ins[i], outs[i], in_sizes[i], out_sizes[i], static_cast<uint32_t>(seed), bitwidths[i],
                      static_cast<uint8_t>(enable_randoms[i] != 0), 0};
      log_resident(ra.seg, seed);
      rc = next_barrier_generation(ws, st);
      if (rc != HPX_OK) return rc;
      ra.gen = ws->bar_gen;
      ra.bar = reinterpret_cast<uint64_t*>(ws->bar);
      ra.host_flag = expired;
      ra.spin_limit = resident_spin_limit();
      ra.stamps = phase_stamps_for(resident_grid(ws));
      ra.done = ws->done;
      rc = launch_resident(ra, resident_grid(ws), st);
      if (rc != HPX_OK) return rc;
      mark_resident_log(ws, ra.gen, resident_grid(ws));
    }
  }
  if (tiled.empty()) return HPX_OK;
  if (int(tiled.size()) == count)
    return encode_tiled(ws, st, count, ins, in_sizes, outs, out_sizes, bitwidths, enable_randoms, seeds);
  const int m = int(tiled.size());
  std::vector<const float*> t_in(m);
  std::vector<uint8_t*> t_out(m);
  std::vector<int32_t> t_isz(m), t_osz(m), t_rnd(m);
  std::vector<uint8_t> t_bits(m);
  std::vector<uint64_t> t_seed(m);
  for (int k = 0; k < m; k++) {
    const int i = tiled[k];
    t_in[k] = ins[i]; t_out[k] = outs[i]; t_isz[k] = in_sizes[i]; t_osz[k] = out_sizes[i];
    t_rnd[k] = enable_randoms[i]; t_bits[k] = bitwidths[i];
    t_seed[k] = seeds ? seeds[i] : hpx::clock_seed();
  }
  return encode_tiled(ws, st, m, t_in.data(), t_isz.data(), t_out.data(), t_osz.data(), t_bits.data(), t_rnd.data(),
                      t_seed.data());
}

HPX_API int hpx_terngrad_encode_noalloc(int count, const float* const* ins, const int32_t* in_sizes,
                                        uint8_t* const* outs, const int32_t* out_sizes,
                                        const uint8_t* bitwidths, const int32_t* enable_randoms,
                                        const uint64_t* seeds, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_terngrad_encode_noalloc: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(count <= kNoAllocMaxTensors, "hpx_terngrad_encode_noalloc: %d tensors in one call, at most %d (the fixed scratch array holds %d x %d slots)",
          count, kNoAllocMaxTensors, kNoAllocMaxTensors, kSlotsPerTensor);
  HPX_ARG(ins && in_sizes && outs && out_sizes && bitwidths && enable_randoms,
          "hpx_terngrad_encode_noalloc: null argument array");
  int64_t red_tiles = 0, quant_tiles = 0;
  for (int i = 0; i < count; i++) {
    const uint8_t b = bitwidths[i];
    if (!(b == 1 || b == 2 || b == 4 || b == 8)) {
      hpx::set_error("Invalid value of bitwidth, check value: bitwidth=%d", int(b));
      return HPX_ERR_BODY;
    }
    HPX_ARG(in_sizes[i] > 0, "hpx_terngrad_encode_noalloc: tensor %d has size %d (must be positive)", i, in_sizes[i]);
    HPX_ARG(ins[i] && outs[i], "hpx_terngrad_encode_noalloc: tensor %d has a null pointer", i);
    const int64_t need = 10 + (int64_t(in_sizes[i]) + 8 / b - 1) / (8 / b);
    HPX_ARG(out_sizes[i] >= need, "hpx_terngrad_encode_noalloc: tensor %d needs %lld output bytes, got %d", i,
            static_cast<long long>(need), out_sizes[i]);
    const int unit = (8 / b) > 4 ? (8 / b) : 4;
    red_tiles += ceil_div(in_sizes[i], kRedTile);
    quant_tiles += ceil_div(ceil_div(in_sizes[i], unit), kThreads * kQIters);
  }
  // one table, one pair of launches: the scratch array has room for exactly that
  HPX_ARG(red_tiles <= INT32_MAX && quant_tiles <= INT32_MAX, "hpx_terngrad_encode_noalloc: the tensors of one call add up to too many tiles (%lld)",
          static_cast<long long>(red_tiles));
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned long long* slots = nullptr;
  int rc = scratch_address(&slots);
  if (rc != HPX_OK) return rc;
  // The array keeps what the last call left: the slots this call uses start from zero again (a fill
  // kernel, not a memset node, so that the sequence can be recorded into a graph), and the epoch tag is
  // a constant.
  const uint32_t words = uint32_t(count) * kSlotsPerTensor;
  hipLaunchKernelGGL(terngrad_scratch_clear_kernel, dim3((words + kThreads - 1) / kThreads), dim3(kThreads), 0, st, slots, words);
  HPX_HIP(hipGetLastError());
  if (count <= kCapSmall)
    return launch_encode<kCapSmall>(count, ins, in_sizes, outs, out_sizes, bitwidths, enable_randoms, seeds,
                                    reinterpret_cast<uint64_t*>(slots), 1u, st, false);
  return launch_encode<kCapLarge>(count, ins, in_sizes, outs, out_sizes, bitwidths, enable_randoms, seeds,
                                  reinterpret_cast<uint64_t*>(slots), 1u, st, false);
}

HPX_API int hpx_terngrad_encode_status(hpx_stream_t stream) {
  hpx::clear_error();
  hipStream_t st = static_cast<hipStream_t>(stream);
  int rc = hpx::reject_capture(st, "hpx_terngrad_encode_status");
  if (rc != HPX_OK) return rc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  if (!ws->pinned) return HPX_OK;  // nothing has been encoded on this stream
  if (ws->resident_log.empty() && !hpx::barrier_expired(ws)) return HPX_OK;  // no barrier kernel is outstanding
  return settle_resident_log(ws, st);
}

HPX_API int hpx_terngrad_phase_stamps(uint64_t* device_words, int32_t workgroups) {
  hpx::clear_error();
  HPX_ARG(workgroups >= 0 && (device_words || workgroups == 0), "hpx_terngrad_phase_stamps: null buffer");
  g_phase_capacity.store(device_words ? workgroups : 0, std::memory_order_relaxed);
  g_phase_stamps.store(workgroups > 0 ? device_words : nullptr, std::memory_order_relaxed);
  return HPX_OK;
}

HPX_API int64_t hpx_terngrad_repaired(hpx_stream_t stream) {
  hpx::clear_error();
  hpx::Workspace* ws = hpx::workspace_record(static_cast<hipStream_t>(stream));
  if (!ws) return -1;
  std::lock_guard<std::mutex> lock(ws->mu);
  return int64_t(ws->repaired);
}

HPX_API int hpx_terngrad_decode(int count, float* const* outs, const int32_t* out_sizes,
                                const uint8_t* const* ins, const int32_t* in_sizes,
                                const int32_t* is_add_tos, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_terngrad_decode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(outs && out_sizes && ins && in_sizes && is_add_tos, "hpx_terngrad_decode: null argument array");
  hipStream_t st = static_cast<hipStream_t>(stream);
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int rc = hpx::ensure_workspace(ws, 0);
  if (rc != HPX_OK) return rc;
  uint32_t* status = ws->state + hpx::kStatusWord;
  switch (hpx::classify_outputs(count, outs, out_sizes)) {
    case 0: break;
    case 1:  // several messages accumulate into the same tensor(s): one pass per tensor
      return launch_decode_multi(count, outs, out_sizes, ins, in_sizes, is_add_tos, status, st);
    default: {  // partially overlapping outputs: keep the reference's one-message-at-a-time order
      for (int i = 0; i < count; i++) {
        const int rc1 = launch_decode<kCapSmall>(1, outs + i, out_sizes + i, ins + i, in_sizes + i, is_add_tos + i, status, st);
        if (rc1 != HPX_OK) return rc1;
      }
      return HPX_OK;
    }
  }
  if (count <= kCapSmall) return launch_decode<kCapSmall>(count, outs, out_sizes, ins, in_sizes, is_add_tos, status, st);
  return launch_decode<kCapLarge>(count, outs, out_sizes, ins, in_sizes, is_add_tos, status, st);
}

HPX_API int hpx_terngrad_decode_status(hpx_stream_t stream) {
  hpx::clear_error();
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const int rcc = hpx::reject_capture(st, "hpx_terngrad_decode_status")) return rcc;
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  int rc = hpx::ensure_workspace(ws, 0);
  if (rc != HPX_OK) return rc;
  uint32_t* flag = ws->state + hpx::kStatusWord;
  uint32_t* host = reinterpret_cast<uint32_t*>(ws->pinned);
  HPX_HIP(hipMemcpyAsync(host, flag, sizeof(uint32_t), hipMemcpyDeviceToHost, st));
  HPX_HIP(hipStreamSynchronize(st));
  if (*host & 1u) {
    HPX_HIP(hipMemsetAsync(flag, 0, sizeof(uint32_t), st));
    hpx::set_error("bitwidth is invalid");
    return HPX_ERR_BODY;
  }
  return HPX_OK;
}
