// The reference's kernel-driver functions (declared in hp_cuda.cpp:18-82, defined
// in hp_cuda_kernel.cu:30-230) with their own names, argument lists and order,
// implemented over the C ABI of include/hpx.h.  hp_cuda.cpp only needs
// `cudaStream_t` spelled `hipStream_t`; linking libhpx.so instead of compiling
// hp_cuda_kernel.cu then swaps the whole kernel layer.
//
// Like the reference drivers they print and go on when a body fails, and the two
// TBQ functions wait for the stream before returning (hp_cuda_kernel.cu:157, :197).
// The RNG seed is taken from the wall clock as in the reference bodies.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <vector>

void hp_cuda_terngrad(std::vector<float*>& in_floats, std::vector<int32_t>& in_float_sizes,
                      std::vector<uint8_t*>& out_uint8_ts, std::vector<int32_t>& out_uint8_t_sizes,
                      std::vector<uint8_t>& bitwidths, std::vector<int32_t>& enable_randoms, hipStream_t stream);

void hp_cuda_terngradr(std::vector<float*>& out_floats, std::vector<int32_t>& out_float_sizes,
                       std::vector<uint8_t*>& in_uint8_ts, std::vector<int32_t>& in_uint8_t_sizes,
                       std::vector<int>& is_add_tos, hipStream_t stream);

void hp_cuda_tbqr(std::vector<float*>& out_floats, std::vector<int32_t>& out_float_sizes,
                  std::vector<uint8_t*>& in_uint8_ts, std::vector<int32_t>& in_uint8_t_sizes,
                  std::vector<float>& thresholds, std::vector<int>& is_add_tos, hipStream_t stream);

void hp_cuda_tbq(std::vector<float*>& to_compress_floats, std::vector<int32_t>& to_compress_float_sizes,
                 std::vector<float*>& residual_floats, std::vector<int32_t>& residual_float_sizes,
                 std::vector<uint8_t*>& out_uint8_ts, std::vector<int32_t>& out_uint8_t_sizes,
                 std::vector<float>& thresholds, hipStream_t stream);

void hp_cuda_gd(std::vector<float*>& in_floats, std::vector<int32_t>& Ns, std::vector<float*>& residuals,
                std::vector<int32_t>& residual_sizes, std::vector<uint8_t*>& out_uint8_ts,
                std::vector<double>& sample_rates, std::vector<double>& drop_ratios, hipStream_t stream);

void hp_cuda_gdr(std::vector<uint8_t*>& in_uint8_ts, std::vector<int32_t>& in_uint8_t_sizes,
                 std::vector<float*>& out_floats, std::vector<int32_t>& out_float_sizes,
                 std::vector<int>& is_add_tos, hipStream_t stream);
