// PowerSGD rank-r phases over a batch of row-major fp32 matrices.
//
// Semantics are the ones the reference's comments state (powersgd_body.h:20-29,
// :41-50, :64-76); its literal copy_ calls have source and destination
// swapped:
//   encode1  M.flat[:N] = grad + residual ;  P = M Q        (n x m)(m x r)
//   encode2  P <- orthonormal columns     ;  Q = M^T P      (m x n)(n x r)
//   decode   M = P Q^T ; residual = grad - M.flat[:N] ; grad = M.flat[:N]
//
// Every phase is one streaming pass over the n x m data, so all three are bound
// by HBM; the rank-r contractions ride along on the matrix cores with
// v_mfma_f32_4x4x1_16b_f32: sixteen independent 4x4 outer-product blocks per
// instruction, so four columns of a rank-4 factor fill the N dimension exactly.
// Operand layout of that instruction: A[blk][i] in lane 4*blk+i, B[blk][j] in
// lane 4*blk+j, D[blk][i][j] in lane 4*blk+j, register i.
//
// Ranks up to 16 are handled as up to four column groups of four in one pass over the data.  Larger ranks
// (the reference takes any, powersgd_body.h:28,49,69) go sixteen columns at a time: every pass names a block
// of columns of P and Q by an offset pointer, the block's width `r` and the factors' row stride `ld`; encode1
// stores M in its first pass and reads it back in the others, decode builds M up over its passes and writes the
// residual and the gradient in the last.
#include "hpx_common.h"

namespace {
using namespace hpx;

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxSeg = 40;
constexpr int kMaxCG = 4;                 // column groups of 4 -> rank <= 16
constexpr int kStrip = 256;               // columns per wave step in encode2 / decode
constexpr int kE2RowsPerBlock = 128;      // rows folded into one partial of Q
// Decode is three write streams against one read stream; with 8 rows per wave instead of 32 the
// stores of a workgroup stay close together in time and address and the pass runs 10 % faster.
constexpr int kDecRowsPerBlock = 32;

struct Seg {
  const float* grad;   // encode1: in.  decode: in/out (as float*)
  const float* res;    // encode1: in.  decode: out
  const float* Q;
  float* M;
  float* P;
  float* Qout;         // encode2: Q to write;  partials live in the workspace
  int64_t numel;
  int32_t n, m, r;
  int32_t part_off;    // encode2: offset (in floats / 4) of this matrix's partials
  int32_t ld;          // row stride of P and Q (the full rank; r is the width of the block of columns at hand)
  int32_t mode;        // kFromM | kOntoM | kKeepGrad, for the passes of a rank above 16
};
constexpr int32_t kFromM = 1;    // encode1: M has been stored by an earlier pass: read it instead of grad + residual
constexpr int32_t kOntoM = 2;    // decode: add this block's P Q^T to what M holds instead of starting from zero
constexpr int32_t kKeepGrad = 4; // decode: more blocks follow: write M only, leave residual and gradient alone
struct Args {
  int32_t nseg;
  int32_t tile_start[kMaxSeg + 1];
  Seg seg[kMaxSeg];
  float* partials;
};
static_assert(sizeof(Args) <= 4096, "kernarg limit");

__device__ __forceinline__ f32x4 mfma4(float a, float b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 0, 0, 0);
}

// ---- encode1: M = G + R (flat prefix), P = M Q -------------------------------
// One workgroup per group of 4 rows; its 4 waves share out the columns and meet in
// LDS.  Lane 4b+i of a wave owns row i and the 4 columns k0+4b..k0+4b+3 of each
// 64-column step, which is one 128-bit load of G and of R and one store of M.
template <int CG>
__global__ __launch_bounds__(kThreads) void psgd_encode1_kernel(const Args a) {
  const int tile = blockIdx.x;
  const int s = find_segment<kMaxSeg>(a.tile_start, a.nseg, tile);
  const Seg& sg = a.seg[s];
  const float* __restrict__ G = sg.grad;
  const float* __restrict__ R = sg.res;
  const float* __restrict__ Q = sg.Q;
  float* __restrict__ M = sg.M;
  const int n = sg.n, m = sg.m, r = sg.r, ld = sg.ld;
  const bool from_m = (sg.mode & kFromM) != 0;
  const int64_t N = sg.numel;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int row0 = (tile - a.tile_start[s]) * 4;
  const int i = lane & 3, b = lane >> 2;
  const int row = row0 + i;
  // Columns: the workgroup walks the rows in chunks of kWaves * 256 columns, wave w taking the w-th 256 of each
  // chunk, so that at any time the four waves read neighbouring pieces of the same four rows (a contiguous
  // quarter of the row per wave ran 9 % slower); what is left past the last whole 256 goes round the waves in
  // 64-column steps.
  constexpr int kUnroll = 4;
  constexpr int kChunk = 64 * kUnroll;
  const int mfull = m / kChunk * kChunk;

  f32x4 acc[CG];
#pragma unroll
  for (int c = 0; c < CG; c++) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bool rows_full = (row0 + 3 < n) && (int64_t(row0 + 4) * m <= N);
  if (rows_full) {
    // Main loop: kUnroll 64-column steps at a time, every load issued before the first use.
    for (int k0 = wave * kChunk; k0 < mfull; k0 += kWaves * kChunk) {
      float4 g4[kUnroll], r4[kUnroll];
      float q[kUnroll][4][CG];
#pragma unroll
      for (int u = 0; u < kUnroll; u++) {
        const int64_t f = int64_t(row) * m + k0 + 64 * u + 4 * b;
        g4[u] = from_m ? ld4_stream(M + f) : ld4_stream(G + f);
        r4[u] = from_m ? make_float4(0.f, 0.f, 0.f, 0.f) : ld4_stream(R + f);
      }
#pragma unroll
      for (int u = 0; u < kUnroll; u++)
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int c = 0; c < CG; c++) {
            const int col = c * 4 + i;  // B operand: lane 4b+j holds Q[k][j]
            q[u][t][c] = col < r ? Q[int64_t(k0 + 64 * u + 4 * b + t) * ld + col] : 0.f;
          }
#pragma unroll
      for (int u = 0; u < kUnroll; u++) {
        const int64_t f = int64_t(row) * m + k0 + 64 * u + 4 * b;
        const float4 m4 = make_float4(g4[u].x + r4[u].x, g4[u].y + r4[u].y, g4[u].z + r4[u].z, g4[u].w + r4[u].w);
        if (!from_m) st4_stream(M + f, m4);  // the set of M matrices is far larger than the caches: do not allocate
        const float v[4] = {m4.x, m4.y, m4.z, m4.w};
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int c = 0; c < CG; c++) acc[c] = mfma4(v[t], q[u][t][c], acc[c]);
      }
    }
  }
  for (int k0 = (rows_full ? mfull : 0) + wave * 64; k0 < m; k0 += kWaves * 64) {
    const int kk = k0 + 4 * b;
    float v[4];
    if (rows_full && k0 + 64 <= m) {
      const int64_t f = int64_t(row) * m + kk;
      const float4 g4 = from_m ? ld4_stream(M + f) : ld4_stream(G + f);
      const float4 r4 = from_m ? make_float4(0.f, 0.f, 0.f, 0.f) : ld4_stream(R + f);
      const float4 m4 = make_float4(g4.x + r4.x, g4.y + r4.y, g4.z + r4.z, g4.w + r4.w);
      if (!from_m) st4(M + f, m4);
      v[0] = m4.x; v[1] = m4.y; v[2] = m4.z; v[3] = m4.w;
    } else {
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const int k = kk + t;
        float x = 0.f;
        if (row < n && k < m) {
          const int64_t f = int64_t(row) * m + k;
          if (f < N && !from_m) {
            x = G[f] + R[f];
            M[f] = x;
          } else {
            x = M[f];  // beyond the gradient: whatever the caller left in M takes part in P = M Q
          }
        }
        v[t] = x;
      }
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int k = kk + t;
#pragma unroll
      for (int c = 0; c < CG; c++) {
        const int col = c * 4 + i;  // B operand: lane 4b+j holds Q[k][j]
        const float q = (k < m && col < r) ? Q[int64_t(k) * ld + col] : 0.f;
        acc[c] = mfma4(v[t], q, acc[c]);
      }
    }
  }
  // acc[c][ii] in lane 4b+j is the part of P[row0+ii][4c+j] from this lane's columns: fold the 16 blocks
  __shared__ float s_p[kWaves][CG][4][4];
#pragma unroll
  for (int c = 0; c < CG; c++)
#pragma unroll
    for (int ii = 0; ii < 4; ii++) {
      float x = acc[c][ii];
#pragma unroll
      for (int o = 4; o < kWave; o <<= 1) x += __shfl_xor(x, o, kWave);
      if (lane < 4) s_p[wave][c][ii][lane] = x;
    }
  __syncthreads();
  if (threadIdx.x < CG * 16) {
    const int c = threadIdx.x / 16, ii = (threadIdx.x / 4) & 3, j = threadIdx.x & 3;
    const int col = c * 4 + j;
    if (row0 + ii < n && col < r) {
      float x = s_p[0][c][ii][j];
#pragma unroll
      for (int w = 1; w < kWaves; w++) x += s_p[w][c][ii][j];
      sg.P[int64_t(row0 + ii) * ld + col] = x;
    }
  }
}

// ---- encode2, step 1: orthonormalise the columns of P -------------------------
// Modified Gram-Schmidt, two sweeps (the second restores orthogonality lost to
// cancellation), reductions in fp64.  One workgroup per matrix; P is n x r <= 16.
constexpr int kOrthThreads = 1024;

__device__ __forceinline__ double block_sum(double v, double* s_red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  const int w = threadIdx.x / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) s_red[w] = v;
  __syncthreads();
  double t = 0;
#pragma unroll
  for (int k = 0; k < kOrthThreads / kWave; k++) t += s_red[k];
  return t;
}

// P[row][c] of the matrix being orthonormalised: either the caller's row-major
// array in global memory or a column-major copy in LDS (conflict-free for the
// row-strided sweeps below).
template <bool LDS>
struct PView {
  float* p;
  int n, r;
  __device__ __forceinline__ float& at(int row, int c) const { return LDS ? p[c * n + row] : p[int64_t(row) * r + c]; }
};

template <bool LDS>
__device__ __forceinline__ void gram_schmidt(const PView<LDS> P, double* s_red) {
  const int n = P.n, r = P.r;
  for (int sweep = 0; sweep < 2; sweep++) {
    for (int c = 0; c < r; c++) {
      double ss = 0;
      for (int row = threadIdx.x; row < n; row += kOrthThreads) {
        const double x = P.at(row, c);
        ss += x * x;
      }
      ss = block_sum(ss, s_red);
      const float inv = ss > 0 ? static_cast<float>(1.0 / sqrt(ss)) : 0.f;
      for (int row = threadIdx.x; row < n; row += kOrthThreads) P.at(row, c) *= inv;
      for (int c2 = c + 1; c2 < r; c2++) {
        double d = 0;
        for (int row = threadIdx.x; row < n; row += kOrthThreads) d += double(P.at(row, c)) * double(P.at(row, c2));
        d = block_sum(d, s_red);
        const float df = static_cast<float>(d);
        for (int row = threadIdx.x; row < n; row += kOrthThreads) P.at(row, c2) -= df * P.at(row, c);
      }
    }
  }
}

// Global-memory variant: any n x r.
__global__ __launch_bounds__(kOrthThreads) void psgd_orth_kernel(const Args a) {
  __shared__ double s_red[kOrthThreads / kWave];
  const Seg& sg = a.seg[blockIdx.x];
  gram_schmidt(PView<false>{sg.P, sg.n, sg.r}, s_red);
}

// LDS variant: the whole n x r factor (at most kOrthLdsFloats values) is staged in
// dynamic shared memory, orthonormalised there and written back.
constexpr int kOrthLdsFloats = 36 * 1024;  // 144 KiB of the 160 KiB LDS
__global__ __launch_bounds__(kOrthThreads) void psgd_orth_lds_kernel(const Args a) {
  __shared__ double s_red[kOrthThreads / kWave];
  extern __shared__ float s_p[];
  const Seg& sg = a.seg[blockIdx.x];
  float* __restrict__ Pg = sg.P;
  const int n = sg.n, r = sg.r;
  for (int e = threadIdx.x; e < n * r; e += kOrthThreads) s_p[(e % r) * n + e / r] = Pg[e];
  __syncthreads();
  gram_schmidt(PView<true>{s_p, n, r}, s_red);
  __syncthreads();
  for (int e = threadIdx.x; e < n * r; e += kOrthThreads) Pg[e] = s_p[(e % r) * n + e / r];
}

// ---- encode2, step 2: Q = M^T P ------------------------------------------------
// A workgroup takes a strip of 256 columns and 128 rows (32 per wave).  Per row a
// lane loads its 4 columns of M with one 128-bit load; register t of that load
// is the A operand of MFMA t, whose block b / row-of-block i' is column
// k0 + 16b + 4i' + t; the B operand is P[row][j] in every block.  The waves meet
// in LDS and the workgroup writes one partial of Q; a second kernel adds the
// partials in a fixed order.
template <int CG>
__global__ __launch_bounds__(kThreads) void psgd_mtp_kernel(const Args a) {
  const int tile = blockIdx.x;
  const int s = find_segment<kMaxSeg>(a.tile_start, a.nseg, tile);
  const Seg& sg = a.seg[s];
  const float* __restrict__ M = sg.M;
  const float* __restrict__ P = sg.P;
  const int n = sg.n, m = sg.m, r = sg.r, ld = sg.ld;
  const int strips = (m + kStrip - 1) / kStrip;
  const int t_in = tile - a.tile_start[s];
  const int strip = t_in % strips, rblk = t_in / strips;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int k0 = strip * kStrip;
  const int kk = k0 + 4 * lane;
  const int rbeg = rblk * kE2RowsPerBlock + wave * (kE2RowsPerBlock / kWaves);
  int rend = rbeg + kE2RowsPerBlock / kWaves;
  if (rend > n) rend = n;

  f32x4 acc[CG][4];
#pragma unroll
  for (int c = 0; c < CG; c++)
#pragma unroll
    for (int t = 0; t < 4; t++) acc[c][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bool cols_full = k0 + kStrip <= m;
  const int j = lane & 3;
  int row = rbeg;
  if (cols_full) {
    // Main loop: 8 rows at a time, every load issued before the first use.
    constexpr int kRows = 8;
    for (; row + kRows <= rend; row += kRows) {
      float4 m4[kRows];
      float p[kRows][CG];
#pragma unroll
      for (int u = 0; u < kRows; u++) m4[u] = ld4_stream(M + int64_t(row + u) * m + kk);
#pragma unroll
      for (int u = 0; u < kRows; u++)
#pragma unroll
        for (int c = 0; c < CG; c++) p[u][c] = (c * 4 + j) < r ? P[int64_t(row + u) * ld + c * 4 + j] : 0.f;
#pragma unroll
      for (int u = 0; u < kRows; u++) {
        const float v[4] = {m4[u].x, m4[u].y, m4[u].z, m4[u].w};
#pragma unroll
        for (int c = 0; c < CG; c++)
#pragma unroll
          for (int t = 0; t < 4; t++) acc[c][t] = mfma4(v[t], p[u][c], acc[c][t]);
      }
    }
  }
  for (; row < rend; row++) {
    float v[4];
    if (cols_full) {
      const float4 m4 = ld4_stream(M + int64_t(row) * m + kk);
      v[0] = m4.x; v[1] = m4.y; v[2] = m4.z; v[3] = m4.w;
    } else {
#pragma unroll
      for (int t = 0; t < 4; t++) v[t] = (kk + t < m) ? M[int64_t(row) * m + kk + t] : 0.f;
    }
#pragma unroll
    for (int c = 0; c < CG; c++) {
      const int col = c * 4 + j;
      const float p = col < r ? P[int64_t(row) * ld + col] : 0.f;
#pragma unroll
      for (int t = 0; t < 4; t++) acc[c][t] = mfma4(v[t], p, acc[c][t]);
    }
  }
  // acc[c][t][i'] in lane 4b+j  ->  Q[k0 + 16b + 4i' + t][4c + j]
  __shared__ float s_q[kWaves][CG][kStrip][4];
#pragma unroll
  for (int c = 0; c < CG; c++)
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int ii = 0; ii < 4; ii++) s_q[wave][c][16 * (lane >> 2) + 4 * ii + t][j] = acc[c][t][ii];
  __syncthreads();
  float* part = a.partials + (int64_t(sg.part_off) * 4) + int64_t(rblk) * m * r;
  for (int e = threadIdx.x; e < CG * kStrip * 4; e += kThreads) {
    const int c = e / (kStrip * 4), kl = (e / 4) % kStrip, jj = e & 3;
    const int k = k0 + kl, col = c * 4 + jj;
    if (k < m && col < r) {
      float x = s_q[0][c][kl][jj];
#pragma unroll
      for (int w = 1; w < kWaves; w++) x += s_q[w][c][kl][jj];
      part[int64_t(k) * r + col] = x;
    }
  }
}

__global__ __launch_bounds__(kThreads) void psgd_qreduce_kernel(const Args a) {
  const int tile = blockIdx.x;
  const int s = find_segment<kMaxSeg>(a.tile_start, a.nseg, tile);
  const Seg& sg = a.seg[s];
  const int64_t mr = int64_t(sg.m) * sg.r;
  const int nparts = (sg.n + kE2RowsPerBlock - 1) / kE2RowsPerBlock;
  const float* part = a.partials + int64_t(sg.part_off) * 4;
  const int64_t e = int64_t(tile - a.tile_start[s]) * kThreads + threadIdx.x;
  if (e < mr) {
    float x = 0.f;
    for (int p = 0; p < nparts; p++) x += part[int64_t(p) * mr + e];
    sg.Qout[(e / sg.r) * sg.ld + e % sg.r] = x;
  }
}

// ---- decode: M = P Q^T, residual = grad - M, grad = M ---------------------------
// A workgroup takes a strip of 256 columns and kDecRowsPerBlock rows (8 per wave).  MFMA
// (t, j) has A = P[row0+i'][j] and B = Q[k0+4*lane+t][j], so after the sum over
// j register i' of accumulator t is M[row0+i'][k0+4*lane+t]: the four
// accumulators give each lane 4 consecutive columns of 4 rows, i.e. 128-bit
// loads of grad and 128-bit stores of M, residual and grad.
template <int CG>
__global__ __launch_bounds__(kThreads) void psgd_decode_kernel(const Args a) {
  const int tile = blockIdx.x;
  const int s = find_segment<kMaxSeg>(a.tile_start, a.nseg, tile);
  const Seg& sg = a.seg[s];
  const float* __restrict__ P = sg.P;
  const float* __restrict__ Q = sg.Q;
  float* __restrict__ M = sg.M;
  float* __restrict__ G = const_cast<float*>(sg.grad);
  float* __restrict__ R = const_cast<float*>(sg.res);
  const int n = sg.n, m = sg.m, r = sg.r, ld = sg.ld;
  const bool onto_m = (sg.mode & kOntoM) != 0, keep_grad = (sg.mode & kKeepGrad) != 0;
  const int64_t N = sg.numel;
  const int strips = (m + kStrip - 1) / kStrip;
  const int t_in = tile - a.tile_start[s];
  const int strip = t_in % strips, rblk = t_in / strips;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int k0 = strip * kStrip;
  const int kk = k0 + 4 * lane;
  const int rbeg = rblk * kDecRowsPerBlock + wave * (kDecRowsPerBlock / kWaves);
  int rend = rbeg + kDecRowsPerBlock / kWaves;
  if (rend > n) rend = n;
  const int i = lane & 3;

  float q[4][CG * 4];  // Q[kk+t][col]
#pragma unroll
  for (int t = 0; t < 4; t++)
#pragma unroll
    for (int col = 0; col < CG * 4; col++) q[t][col] = (kk + t < m && col < r) ? Q[int64_t(kk + t) * ld + col] : 0.f;

  const bool cols_full = k0 + kStrip <= m;
  for (int row0 = rbeg; row0 < rend; row0 += 4) {
    const bool full4 = cols_full && row0 + 4 <= rend && int64_t(row0 + 3) * m + kk + 4 <= N;
    float4 g4[4];
    if (full4) {
#pragma unroll
      for (int ii = 0; ii < 4; ii++) g4[ii] = ld4_stream(G + int64_t(row0 + ii) * m + kk);
    }
    f32x4 acc[4];
#pragma unroll
    for (int t = 0; t < 4; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (onto_m) {  // a later block of columns of a rank above 16: go on from what the earlier blocks left in M
#pragma unroll
      for (int ii = 0; ii < 4; ii++)
#pragma unroll
        for (int t = 0; t < 4; t++)
          if (row0 + ii < rend && kk + t < m) acc[t][ii] = M[int64_t(row0 + ii) * m + kk + t];
    }
#pragma unroll
    for (int col = 0; col < CG * 4; col++) {
      const float p = (row0 + i < n && col < r) ? P[int64_t(row0 + i) * ld + col] : 0.f;
#pragma unroll
      for (int t = 0; t < 4; t++) acc[t] = mfma4(p, q[t][col], acc[t]);
    }
    if (full4) {
#pragma unroll
      for (int ii = 0; ii < 4; ii++) {
        const int64_t f = int64_t(row0 + ii) * m + kk;
        const float4 m4 = make_float4(acc[0][ii], acc[1][ii], acc[2][ii], acc[3][ii]);
        const float4 r4 = make_float4(g4[ii].x - m4.x, g4[ii].y - m4.y, g4[ii].z - m4.z, g4[ii].w - m4.w);
        if (!keep_grad) {
          st4_stream(R + f, r4);
          st4_stream(G + f, m4);  // in place over the line just read
        }
        st4(M + f, m4);  // plain: streaming this third store was measurably slower
      }
      continue;
    }
#pragma unroll
    for (int ii = 0; ii < 4; ii++) {
      const int row = row0 + ii;
      if (row >= rend) break;
      const int64_t f = int64_t(row) * m + kk;
      const float mv[4] = {acc[0][ii], acc[1][ii], acc[2][ii], acc[3][ii]};
#pragma unroll
      for (int t = 0; t < 4; t++) {
        if (kk + t < m) {
          if (f + t < N && !keep_grad) {
            R[f + t] = G[f + t] - mv[t];
            G[f + t] = mv[t];
          }
          M[f + t] = mv[t];
        }
      }
    }
  }
}

inline int32_t cdiv(int64_t x, int64_t y) { return static_cast<int32_t>((x + y - 1) / y); }

struct Batch {
  int count;
  const int32_t *ns, *ms, *rs;
};

constexpr int kPassCols = 4 * kMaxCG;  // columns of the factors one pass over the data handles

int check_dims(const char* who, const Batch& b, int* max_rank) {
  *max_rank = 1;
  for (int i = 0; i < b.count; i++) {
    HPX_ARG(b.ns[i] > 0 && b.ms[i] > 0 && b.rs[i] > 0, "%s: matrix %d has dims %d x %d rank %d", who, i, b.ns[i], b.ms[i],
            b.rs[i]);
    if (b.rs[i] > *max_rank) *max_rank = b.rs[i];
  }
  return HPX_OK;
}
// The block of columns [c0, c0 + kPassCols) of a rank-r factor: its width (0: the matrix has no such block) and
// the column groups of four it needs.
inline int block_cols(int r, int c0) { return r <= c0 ? 0 : (r - c0 < kPassCols ? r - c0 : kPassCols); }

#define PSGD_LAUNCH_CG_LDS(KERNEL, cg, grid, lds, st, args)                                                         \
  switch (cg) {                                                                                                     \
    case 1: HPX_LAUNCH_LDS(#KERNEL, hpx::g_prof_on, KERNEL<1>, dim3(grid), dim3(kThreads), lds, st, args); break;  \
    case 2: HPX_LAUNCH_LDS(#KERNEL, hpx::g_prof_on, KERNEL<2>, dim3(grid), dim3(kThreads), lds, st, args); break;  \
    case 3: HPX_LAUNCH_LDS(#KERNEL, hpx::g_prof_on, KERNEL<3>, dim3(grid), dim3(kThreads), lds, st, args); break;  \
    default: HPX_LAUNCH_LDS(#KERNEL, hpx::g_prof_on, KERNEL<4>, dim3(grid), dim3(kThreads), lds, st, args); break; \
  }
#define PSGD_LAUNCH_CG(KERNEL, cg, grid, st, args) PSGD_LAUNCH_CG_LDS(KERNEL, cg, grid, 0, st, args)

}  // namespace

HPX_API int hpx_powersgd_encode1(int count, const float* const* grads, const int64_t* numels,
                                 const float* const* residuals, const float* const* Qs, float* const* Ms,
                                 float* const* Ps, const int32_t* ns, const int32_t* ms, const int32_t* rs,
                                 hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_powersgd_encode1: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(grads && numels && residuals && Qs && Ms && Ps && ns && ms && rs, "hpx_powersgd_encode1: null argument array");
  int max_rank = 1;
  int rc = check_dims("hpx_powersgd_encode1", Batch{count, ns, ms, rs}, &max_rank);
  if (rc != HPX_OK) return rc;
  for (int i = 0; i < count; i++) {
    HPX_ARG(grads[i] && residuals[i] && Qs[i] && Ms[i] && Ps[i], "hpx_powersgd_encode1: matrix %d has a null pointer", i);
    HPX_ARG(numels[i] >= 0 && numels[i] <= int64_t(ns[i]) * ms[i], "hpx_powersgd_encode1: matrix %d: numel %lld exceeds n*m", i,
            static_cast<long long>(numels[i]));
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  Args a;
  a.partials = nullptr;
  for (int c0 = 0; c0 < max_rank; c0 += kPassCols) {
    int i = 0;
    while (i < count) {
      a.nseg = 0;
      a.tile_start[0] = 0;
      int cg = 1;
      while (i < count && a.nseg < kMaxSeg) {
        const int rb = block_cols(rs[i], c0);
        if (rb == 0) { i++; continue; }
        const int32_t t = cdiv(ns[i], 4);
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;
        a.seg[a.nseg] = Seg{grads[i], residuals[i], Qs[i] + c0, Ms[i], Ps[i] + c0, nullptr, numels[i], ns[i], ms[i], rb, 0,
                            rs[i], c0 ? kFromM : 0};
        if ((rb + 3) / 4 > cg) cg = (rb + 3) / 4;
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
        i++;
      }
      if (a.nseg == 0) continue;
      PSGD_LAUNCH_CG(psgd_encode1_kernel, cg, a.tile_start[a.nseg], st, a);
      HPX_HIP(hipGetLastError());
    }
  }
  return HPX_OK;
}

HPX_API int hpx_powersgd_encode2(int count, float* const* Ps, const float* const* Ms, float* const* Qs,
                                 const int32_t* ns, const int32_t* ms, const int32_t* rs, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_powersgd_encode2: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(Ps && Ms && Qs && ns && ms && rs, "hpx_powersgd_encode2: null argument array");
  int max_rank = 1;
  int rc = check_dims("hpx_powersgd_encode2", Batch{count, ns, ms, rs}, &max_rank);
  if (rc != HPX_OK) return rc;
  int64_t part_quads = 0;  // partial storage in units of 4 floats (one pass at a time uses it)
  for (int i = 0; i < count; i++) {
    HPX_ARG(Ps[i] && Ms[i] && Qs[i], "hpx_powersgd_encode2: matrix %d has a null pointer", i);
    part_quads += (int64_t(cdiv(ns[i], kE2RowsPerBlock)) * ms[i] * block_cols(rs[i], 0) + 3) / 4;
  }
  HPX_ARG(part_quads <= INT32_MAX, "hpx_powersgd_encode2: batch too large for one call");
  hipStream_t st = static_cast<hipStream_t>(stream);
  hpx::Workspace* ws = hpx::workspace_record(st);
  if (!ws) return HPX_ERR_HIP;
  std::lock_guard<std::mutex> lock(ws->mu);
  rc = hpx::ensure_workspace(ws, size_t(part_quads) * 16);
  if (rc != HPX_OK) return rc;
  Args a;
  a.partials = reinterpret_cast<float*>(ws->dev);
  // step 1: orthonormalise every P over all of its columns
  for (int i = 0; i < count;) {
    a.nseg = 0;
    int64_t max_nr = 0;
    for (; i < count && a.nseg < kMaxSeg; i++) {
      a.seg[a.nseg++] = Seg{nullptr, nullptr, nullptr, nullptr, Ps[i], nullptr, 0, ns[i], ms[i], rs[i], 0, rs[i], 0};
      if (int64_t(ns[i]) * rs[i] > max_nr) max_nr = int64_t(ns[i]) * rs[i];
    }
    if (max_nr <= kOrthLdsFloats) {
      const size_t lds = size_t(max_nr) * sizeof(float);
      HPX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(psgd_orth_lds_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)));
      HPX_LAUNCH_LDS("psgd_orth_kernel", hpx::g_prof_on, psgd_orth_lds_kernel, dim3(a.nseg), dim3(kOrthThreads), lds, st, a);
    } else {
      HPX_LAUNCH("psgd_orth_kernel", psgd_orth_kernel, dim3(a.nseg), dim3(kOrthThreads), st, a);
    }
    HPX_HIP(hipGetLastError());
  }
  // step 2: Q = M^T P, sixteen columns per pass over M
  for (int c0 = 0; c0 < max_rank; c0 += kPassCols) {
    int i = 0;
    int64_t poff = 0;
    while (i < count) {
      a.nseg = 0;
      a.tile_start[0] = 0;
      int32_t red_start[kMaxSeg + 1];
      red_start[0] = 0;
      int cg = 1;
      while (i < count && a.nseg < kMaxSeg) {
        const int rb = block_cols(rs[i], c0);
        if (rb == 0) { i++; continue; }
        const int32_t t = cdiv(ms[i], kStrip) * cdiv(ns[i], kE2RowsPerBlock);
        const int32_t tr = cdiv(int64_t(ms[i]) * rb, kThreads);
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX || int64_t(red_start[a.nseg]) + tr > INT32_MAX) break;
        a.seg[a.nseg] = Seg{nullptr, nullptr, nullptr, const_cast<float*>(Ms[i]), Ps[i] + c0, Qs[i] + c0, 0, ns[i], ms[i], rb,
                            static_cast<int32_t>(poff), rs[i], 0};
        poff += (int64_t(cdiv(ns[i], kE2RowsPerBlock)) * ms[i] * rb + 3) / 4;
        if ((rb + 3) / 4 > cg) cg = (rb + 3) / 4;
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        red_start[a.nseg + 1] = red_start[a.nseg] + tr;
        a.nseg++;
        i++;
      }
      if (a.nseg == 0) continue;
      PSGD_LAUNCH_CG(psgd_mtp_kernel, cg, a.tile_start[a.nseg], st, a);
      HPX_HIP(hipGetLastError());
      for (int k = 0; k <= a.nseg; k++) a.tile_start[k] = red_start[k];
      HPX_LAUNCH("psgd_qreduce_kernel", psgd_qreduce_kernel, dim3(a.tile_start[a.nseg]), dim3(kThreads), st, a);
      HPX_HIP(hipGetLastError());
    }
  }
  return HPX_OK;
}

HPX_API int hpx_powersgd_decode(int count, const float* const* Ps, const float* const* Qs, float* const* Ms,
                                float* const* residuals, float* const* grads, const int64_t* numels,
                                const int32_t* ns, const int32_t* ms, const int32_t* rs, hpx_stream_t stream) {
  hpx::clear_error();
  HPX_ARG(count >= 0, "hpx_powersgd_decode: negative count");
  if (count == 0) return HPX_OK;
  HPX_ARG(Ps && Qs && Ms && residuals && grads && numels && ns && ms && rs, "hpx_powersgd_decode: null argument array");
  int max_rank = 1;
  int rc = check_dims("hpx_powersgd_decode", Batch{count, ns, ms, rs}, &max_rank);
  if (rc != HPX_OK) return rc;
  for (int i = 0; i < count; i++) {
    HPX_ARG(Ps[i] && Qs[i] && Ms[i] && residuals[i] && grads[i], "hpx_powersgd_decode: matrix %d has a null pointer", i);
    HPX_ARG(numels[i] >= 0 && numels[i] <= int64_t(ns[i]) * ms[i], "hpx_powersgd_decode: matrix %d: numel %lld exceeds n*m", i,
            static_cast<long long>(numels[i]));
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  Args a;
  a.partials = nullptr;
  for (int c0 = 0; c0 < max_rank; c0 += kPassCols) {
    int i = 0;
    while (i < count) {
      a.nseg = 0;
      a.tile_start[0] = 0;
      int cg = 1;
      while (i < count && a.nseg < kMaxSeg) {
        const int rb = block_cols(rs[i], c0);
        if (rb == 0) { i++; continue; }
        const int32_t t = cdiv(ms[i], kStrip) * cdiv(ns[i], kDecRowsPerBlock);
        if (int64_t(a.tile_start[a.nseg]) + t > INT32_MAX) break;
        const int32_t mode = (c0 ? kOntoM : 0) | (c0 + kPassCols < rs[i] ? kKeepGrad : 0);
        a.seg[a.nseg] = Seg{grads[i], residuals[i], Qs[i] + c0, Ms[i], const_cast<float*>(Ps[i]) + c0, nullptr, numels[i], ns[i],
                            ms[i], rb, 0, rs[i], mode};
        if ((rb + 3) / 4 > cg) cg = (rb + 3) / 4;
        a.tile_start[a.nseg + 1] = a.tile_start[a.nseg] + t;
        a.nseg++;
        i++;
      }
      if (a.nseg == 0) continue;
      // One read and three writes per element: held to two workgroups per CU (LDS the kernel never touches,
      // hpx_common.h), the 36 matrices of the configuration decode in 755 us instead of 792 (three per CU: 776).
      PSGD_LAUNCH_CG_LDS(psgd_decode_kernel, cg, a.tile_start[a.nseg], hpx::kWriteStreamPadLds2, st, a);
      HPX_HIP(hipGetLastError());
    }
  }
  return HPX_OK;
}
