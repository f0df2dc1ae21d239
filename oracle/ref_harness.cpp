// Host-only build of the REFERENCE's own algorithm bodies, for validating the
// plain-C oracle.  TEST INFRASTRUCTURE: only built where the reference checkout
// is present (never copied, never shipped), output goes to oracle/_ref/.
//
// The reference bodies are policy-templated Thrust code; rocThrust's serial
// (thrust::host) and OpenMP (thrust::omp::par) backends execute them on the
// CPU.  One seam is needed: the reference's operate_memory/get_policy_general.h
// unconditionally includes Thrust's CUDA backend, which does not exist on this
// platform, so its include guard is taken here and the host-side `get_policy`
// (plain memcpy, no-op synchronise: the behaviour of its host and OpenMP
// specialisations) is supplied instead.  All arithmetic, functors, pass
// structure and Thrust algorithm calls come from the reference headers.
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <vector>

#include <thrust/execution_policy.h>
#include <thrust/extrema.h>
#include <thrust/for_each.h>
#include <thrust/system/omp/execution_policy.h>

#define ZQ_CPP_LIB_OPERATE_MEMORY_GET_POLICY_INL_H
namespace zq_cpp_lib {
namespace operate_memory {
template <typename P>
struct get_policy {
  static P get(void*) { return P(); }
  static void memcpyOut(void* d, const void* s, uint32_t n, void*) { std::memcpy(d, s, n); }
  static void memcpyIn(void* d, const void* s, uint32_t n, void*) { std::memcpy(d, s, n); }
  static void memcpyDoubleIn(void* d, const void* s, uint32_t n, void*) { std::memcpy(d, s, n); }
  static void streamSynchronize(void*) {}
};
}  // namespace operate_memory
}  // namespace zq_cpp_lib

#include "ZQ_CPP_LIB/gradient_compression_body/tbq_body.h"
#include "ZQ_CPP_LIB/gradient_compression_body/terngrad_body.h"
#include "ZQ_CPP_LIB/gradient_compression_body/gd_body.h"

namespace gcb = zq_cpp_lib::gradient_compression_body;
using host_pol = thrust::detail::host_t;
using omp_pol = thrust::system::omp::detail::par_t;
#define API extern "C" __attribute__((visibility("default")))

// policy: 0 = thrust::host (serial), 1 = thrust::omp::par
#define DISPATCH(policy, CALL)          \
  do {                                  \
    if (policy) {                       \
      using P = omp_pol;                \
      P pol;                            \
      return CALL;                      \
    } else {                            \
      using P = host_pol;               \
      P pol;                            \
      return CALL;                      \
    }                                   \
  } while (0)

API int ref_tbq_encode(float* g, int32_t n, float* r, uint8_t* out, float thr, int policy) {
  DISPATCH(policy, (gcb::tbq_body<P>(g, n, r, n, out, (n + 3) / 4, thr, pol, nullptr)));
}

API int ref_tbq_decode(float* out, int32_t n, uint8_t* in, float thr, int is_add, int policy) {
  DISPATCH(policy, (gcb::tbq_r_body<P>(out, n, in, (n + 3) / 4, thr, is_add, pol, nullptr)));
}

// Whole-body TernGrad encode.  Reproducible only with enable_random == 0: the
// body reads the clock for the random seed.
API int ref_terngrad_encode(float* x, int32_t n, uint8_t* out, int32_t out_size, uint8_t bitwidth,
                            int32_t enable_random, int policy) {
  std::vector<float*> ins{x};
  std::vector<int32_t> ns{n};
  std::vector<uint8_t*> outs{out};
  std::vector<int32_t> osz{out_size};
  std::vector<uint8_t> bw{bitwidth};
  std::vector<int32_t> rnd{enable_random};
  DISPATCH(policy, (gcb::terngrad_body<P>(ins, ns, outs, osz, bw, rnd, pol, nullptr)));
}

// The reference's seeded payload functor applied to full bytes, given the
// scalars; lets a test fix the seed the body would take from the clock.
template <typename P>
static int tg_payload_random(float* x, int32_t nbytes, uint8_t* payload, uint8_t bitwidth,
                             uint8_t dpb_lg2, float mn, float gi, unsigned long long seed) {
  P pol;
  thrust::counting_iterator<int32_t> b(0);
  thrust::transform(pol, b, b + nbytes, payload,
                    gcb::compress_with_random(x, bitwidth, dpb_lg2, mn, gi, seed));
  return 0;
}
API int ref_terngrad_payload_random(float* x, int32_t nbytes, uint8_t* payload, uint8_t bitwidth,
                                    uint8_t dpb_lg2, float mn, float gi, unsigned long long seed,
                                    int policy) {
  if (policy) return tg_payload_random<omp_pol>(x, nbytes, payload, bitwidth, dpb_lg2, mn, gi, seed);
  return tg_payload_random<host_pol>(x, nbytes, payload, bitwidth, dpb_lg2, mn, gi, seed);
}

API int ref_terngrad_decode(float* out, int32_t n, uint8_t* in, int32_t in_size, int is_add,
                            int policy) {
  std::vector<float*> outs{out};
  std::vector<int32_t> ns{n};
  std::vector<uint8_t*> ins{in};
  std::vector<int32_t> isz{in_size};
  std::vector<int> adds{is_add};
  DISPATCH(policy, (gcb::terngrad_r_body<P>(outs, ns, ins, isz, adds, pol, nullptr)));
}

// Whole-body GradDrop encode (clock-seeded sample; `out` doubles as scratch and
// must hold 4*ceil(N*sample_rate) bytes and 4+8*candidates bytes).
API int ref_gd_encode(float* g, int32_t n, float* r, uint8_t* out, double sample_rate,
                      double drop_ratio, int policy) {
  DISPATCH(policy, (gcb::gd_body<P>(g, n, r, n, out, sample_rate, drop_ratio, pol, nullptr)));
}

// The reference's sampling functor with a caller-chosen seed.
API int ref_gd_sample(float* sample, float* r, int32_t n, int32_t sample_cnt,
                      unsigned long long seed) {
  thrust::for_each(thrust::host, thrust::counting_iterator<int32_t>(0),
                   thrust::counting_iterator<int32_t>(sample_cnt),
                   gcb::generate_sample_G(sample, r, n, seed));
  return 0;
}

// Seeded GradDrop encode: the reference's functors and Thrust calls in the
// order gd_body issues them, with the clock value replaced by `seed`.
template <typename P>
static int gd_seeded(float* G_in, int32_t N, float* R, uint8_t* out, double sample_rate,
                     double drop_ratio, unsigned long long seed, int32_t* info) {
  P policy;
  double s_percent = 1 - drop_ratio;
  int32_t sample_cnt = static_cast<int32_t>(std::ceil(N * sample_rate));
  int32_t expected_selected = static_cast<int32_t>(std::ceil(N * s_percent));
  float* sample_G = reinterpret_cast<float*>(out);
  thrust::transform(policy, G_in, G_in + N, R, R, thrust::plus<float>());
  float* G = R;
  thrust::for_each(policy, thrust::counting_iterator<int32_t>(0),
                   thrust::counting_iterator<int32_t>(sample_cnt),
                   gcb::generate_sample_G(sample_G, G, N, seed));
  thrust::sort(policy, sample_G, sample_G + sample_cnt, thrust::greater<float>());
  int32_t threshold_index = static_cast<int32_t>(sample_cnt * s_percent);
  float threshold = sample_G[threshold_index];
  int32_t* S_index = reinterpret_cast<int32_t*>(out + 4);
  int32_t* S_index_end =
      thrust::copy_if(policy, thrust::counting_iterator<int32_t>(0),
                      thrust::counting_iterator<int32_t>(N), G, S_index, gcb::greater(threshold));
  int32_t selected_num = S_index_end - S_index;
  if (info) {
    info[0] = selected_num;
    std::memcpy(&info[2], &threshold, 4);
  }
  if (selected_num > expected_selected) {
    thrust::sort(policy, S_index, S_index_end, gcb::cmp_float_data_by_int32_index(G));
    selected_num = expected_selected;
    S_index_end = S_index + selected_num;
  }
  if (info) info[1] = selected_num;
  int32_t out_size = 4 + selected_num * 2 * 4;
  std::memcpy(out, &out_size, 4);
  if (selected_num == 0) return 0;
  float* S_value = reinterpret_cast<float*>(S_index_end);
  thrust::for_each(policy, thrust::counting_iterator<int32_t>(0),
                   thrust::counting_iterator<int32_t>(selected_num),
                   gcb::generate_S_value(S_index, S_value, G));
  return 0;
}
API int ref_gd_encode_seeded(float* g, int32_t n, float* r, uint8_t* out, double sample_rate,
                             double drop_ratio, unsigned long long seed, int32_t* info,
                             int policy) {
  if (policy) return gd_seeded<omp_pol>(g, n, r, out, sample_rate, drop_ratio, seed, info);
  return gd_seeded<host_pol>(g, n, r, out, sample_rate, drop_ratio, seed, info);
}

API int ref_gd_decode(uint8_t* in, int32_t in_size, float* out, int32_t out_size, int is_add,
                      int policy) {
  std::vector<uint8_t*> ins{in};
  std::vector<int32_t> isz{in_size};
  std::vector<float*> outs{out};
  std::vector<int32_t> osz{out_size};
  std::vector<int> adds{is_add};
  DISPATCH(policy, (gcb::gd_r_body<P>(ins, isz, outs, osz, adds, pol, nullptr)));
}

// naive_random.hpp generators, for the LCG known answers.
API uint32_t ref_lcg_kth(uint32_t seed, int k) {
  zq_cpp_lib::naive_random r;
  r.srand(seed);  // one draw already taken
  uint32_t v = 0;
  // srand() discards draw 1; expose draw k >= 2 as the (k-1)-th rand() after it
  for (int i = 1; i < k; i++) v = r.rand();
  return v;
}
API float ref_real01(uint32_t seed, int k) {
  zq_cpp_lib::naive_real_random<float> r(0.0, 1.0);
  r.srand(seed);
  float v = 0;
  for (int i = 1; i < k; i++) v = r();
  return v;
}
