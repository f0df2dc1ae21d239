// C++ drivers with the reference's signatures over the C ABI (see hp_cuda_shim.h).
#include "hp_cuda_shim.h"

#include <cstdio>
#include <iostream>

#include "hpx.h"

#define SHIM_API __attribute__((visibility("default")))

namespace {
template <typename T>
const T* const* cptrs(std::vector<T*>& v) { return const_cast<const T* const*>(v.data()); }
std::vector<int32_t> to_i32(const std::vector<int>& v) { return std::vector<int32_t>(v.begin(), v.end()); }
// The completion contract of the reference's drivers: what a driver queued on `stream` has run when it returns.
int finished(hipStream_t stream) { return hipStreamSynchronize(stream) == hipSuccess ? 0 : HPX_ERR_HIP; }
}  // namespace

SHIM_API void hp_cuda_terngrad(std::vector<float*>& in_floats, std::vector<int32_t>& in_float_sizes,
                               std::vector<uint8_t*>& out_uint8_ts, std::vector<int32_t>& out_uint8_t_sizes,
                               std::vector<uint8_t>& bitwidths, std::vector<int32_t>& enable_randoms,
                               hipStream_t stream) {
  int ret = hpx_terngrad_encode(static_cast<int>(in_floats.size()), cptrs(in_floats), in_float_sizes.data(),
                                out_uint8_ts.data(), out_uint8_t_sizes.data(), bitwidths.data(),
                                enable_randoms.data(), nullptr, stream);
  // The reference returns with complete messages: terngrad_body waits for the stream after its last quantise
  // launch (terngrad_body.h:285), and its scheduler copies B on another stream straight afterwards with no event
  // in between (hp_cuda.cpp:464-468).  The status call waits for launches that meet at a grid barrier and encodes
  // again what an expired barrier left unwritten; finished() then waits for everything else queued here.
  if (!ret) ret = hpx_terngrad_encode_status(stream);
  if (!ret) ret = finished(stream);
  if (ret) printf("ret=%d %s\n", ret, hpx_last_error());  // hp_cuda_kernel.cu:63
}

SHIM_API void hp_cuda_terngradr(std::vector<float*>& out_floats, std::vector<int32_t>& out_float_sizes,
                                std::vector<uint8_t*>& in_uint8_ts, std::vector<int32_t>& in_uint8_t_sizes,
                                std::vector<int>& is_add_tos, hipStream_t stream) {
  std::vector<int32_t> adds = to_i32(is_add_tos);
  int ret = hpx_terngrad_decode(static_cast<int>(out_floats.size()), out_floats.data(), out_float_sizes.data(),
                                cptrs(in_uint8_ts), in_uint8_t_sizes.data(), adds.data(), stream);
  // The reference parses the header on the host and fails there; here the check
  // ran on the device, so ask for its result (waits for the stream, as the
  // reference's own header copy does, terngrad_body.h:334-340).
  if (!ret) ret = hpx_terngrad_decode_status(stream);
  if (ret) printf("ret=%d %s\n", ret, hpx_last_error());  // hp_cuda_kernel.cu:229
}

SHIM_API void hp_cuda_tbq(std::vector<float*>& to_compress_floats, std::vector<int32_t>& to_compress_float_sizes,
                          std::vector<float*>& residual_floats, std::vector<int32_t>& /*residual_float_sizes*/,
                          std::vector<uint8_t*>& out_uint8_ts, std::vector<int32_t>& /*out_uint8_t_sizes*/,
                          std::vector<float>& thresholds, hipStream_t stream) {
  int ret = hpx_tbq_encode(static_cast<int>(to_compress_floats.size()), cptrs(to_compress_floats),
                           to_compress_float_sizes.data(), residual_floats.data(), out_uint8_ts.data(),
                           thresholds.data(), stream);
  if (ret) std::cout << "Call tbq_body failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
  (void)hipStreamSynchronize(stream);  // hp_cuda_kernel.cu:157
}

SHIM_API void hp_cuda_tbqr(std::vector<float*>& out_floats, std::vector<int32_t>& out_float_sizes,
                           std::vector<uint8_t*>& in_uint8_ts, std::vector<int32_t>& /*in_uint8_t_sizes*/,
                           std::vector<float>& thresholds, std::vector<int>& is_add_tos, hipStream_t stream) {
  std::vector<int32_t> adds = to_i32(is_add_tos);
  int ret = hpx_tbq_decode(static_cast<int>(out_floats.size()), out_floats.data(), out_float_sizes.data(),
                           cptrs(in_uint8_ts), thresholds.data(), adds.data(), stream);
  if (ret) std::cout << "Call tbq_body failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
  (void)hipStreamSynchronize(stream);  // hp_cuda_kernel.cu:197
}

SHIM_API void hp_cuda_gd(std::vector<float*>& in_floats, std::vector<int32_t>& Ns, std::vector<float*>& residuals,
                         std::vector<int32_t>& /*residual_sizes*/, std::vector<uint8_t*>& out_uint8_ts,
                         std::vector<double>& sample_rates, std::vector<double>& drop_ratios, hipStream_t stream) {
  int ret = hpx_gd_encode(static_cast<int>(in_floats.size()), cptrs(in_floats), Ns.data(), residuals.data(),
                          out_uint8_ts.data(), sample_rates.data(), drop_ratios.data(), nullptr, stream);
  // gd_body's launches are blocking Thrust calls and it waits for the stream at gd_body.h:161 and :201, so the
  // reference's scheduler copies B on its data stream right after this call, which it makes on the null
  // stream (hp_cuda.cpp:292-313).
  if (!ret) ret = finished(stream);
  if (ret) std::cout << "Call gd_body failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
}

SHIM_API void hp_cuda_gdr(std::vector<uint8_t*>& in_uint8_ts, std::vector<int32_t>& in_uint8_t_sizes,
                          std::vector<float*>& out_floats, std::vector<int32_t>& out_float_sizes,
                          std::vector<int>& is_add_tos, hipStream_t stream) {
  std::vector<int32_t> adds = to_i32(is_add_tos);
  int ret = hpx_gd_decode(static_cast<int>(in_uint8_ts.size()), cptrs(in_uint8_ts), in_uint8_t_sizes.data(),
                          out_floats.data(), out_float_sizes.data(), adds.data(), stream);
  // The scheduler encodes the tensors decoded here next, on ANOTHER stream (hp_cuda.cpp:284-301: hp_cuda_gdr on
  // the compute stream, hp_cuda_gd on the null stream; pool streams do not wait for the null stream).
  if (!ret) ret = finished(stream);
  if (ret) std::cout << "Call gdr_body failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
}
