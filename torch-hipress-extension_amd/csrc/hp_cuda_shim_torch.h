// The three PowerSGD drivers of the reference (hp_cuda.cpp:85-106,
// hp_cuda_kernel.cu:232-301) with their own signatures, header-only because they
// take torch tensors: include this from hp_cuda.cpp in a PyTorch-ROCm build, with
// `c10::cuda::CUDAStream` being the HIP stream wrapper there.  M is n x m,
// Q is m x r, P is n x r, all contiguous fp32 device tensors.
#pragma once
#include <hip/hip_runtime_api.h>
#include <torch/extension.h>

#include <iostream>
#include <memory>
#include <vector>

#include "hpx.h"

namespace hp_cuda_shim_detail {
using TensorList = std::vector<std::shared_ptr<torch::Tensor>>;
struct Dims {
  std::vector<int32_t> n, m, r;
  Dims(TensorList& Ms, TensorList& Qs) {
    for (size_t i = 0; i < Ms.size(); i++) {
      n.push_back(static_cast<int32_t>(Ms[i]->size(0)));
      m.push_back(static_cast<int32_t>(Ms[i]->size(1)));
      r.push_back(static_cast<int32_t>(Qs[i]->size(1)));
    }
  }
};
inline std::vector<float*> ptrs(TensorList& ts) {
  std::vector<float*> p;
  for (auto& t : ts) p.push_back(t->data_ptr<float>());
  return p;
}
inline std::vector<int64_t> numels(TensorList& ts) {
  std::vector<int64_t> n;
  for (auto& t : ts) n.push_back(t->numel());
  return n;
}
template <typename T>
const T* const* cp(std::vector<T*>& v) { return const_cast<const T* const*>(v.data()); }
// A driver returns when what it queued has run: the reference's scheduler publishes a task's name right after
// the calls, having waited for its data stream only (hp_cuda.cpp:729-768), and its consumers read P, Q and the gradient on streams of their own.
template <typename Stream>
int finished(Stream& stream) { return hipStreamSynchronize(stream.stream()) == hipSuccess ? 0 : HPX_ERR_HIP; }
}  // namespace hp_cuda_shim_detail

template <typename Stream>
void hp_cuda_powersgd_encode1(std::vector<std::shared_ptr<torch::Tensor>>& grads,
                              std::vector<std::shared_ptr<torch::Tensor>>& residuals,
                              std::vector<std::shared_ptr<torch::Tensor>>& Qs,
                              std::vector<std::shared_ptr<torch::Tensor>>& Ms,
                              std::vector<std::shared_ptr<torch::Tensor>>& Ps, Stream& stream) {
  using namespace hp_cuda_shim_detail;
  Dims d(Ms, Qs);
  auto g = ptrs(grads), r = ptrs(residuals), q = ptrs(Qs), m = ptrs(Ms), p = ptrs(Ps);
  auto ne = numels(grads);
  int ret = hpx_powersgd_encode1(static_cast<int>(g.size()), cp(g), ne.data(), cp(r), cp(q), m.data(), p.data(),
                                 d.n.data(), d.m.data(), d.r.data(), stream.stream());
  if (!ret) ret = finished(stream);
  if (ret) std::cout << "Call powersgd encode1 failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
}

template <typename Stream>
void hp_cuda_powersgd_encode2(std::vector<std::shared_ptr<torch::Tensor>>& Ps,
                              std::vector<std::shared_ptr<torch::Tensor>>& Ms,
                              std::vector<std::shared_ptr<torch::Tensor>>& Qs, Stream& stream) {
  using namespace hp_cuda_shim_detail;
  Dims d(Ms, Qs);
  auto p = ptrs(Ps), m = ptrs(Ms), q = ptrs(Qs);
  int ret = hpx_powersgd_encode2(static_cast<int>(p.size()), p.data(), cp(m), q.data(), d.n.data(), d.m.data(),
                                 d.r.data(), stream.stream());
  if (!ret) ret = finished(stream);
  if (ret) std::cout << "Call powersgd encode2 failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
}

template <typename Stream>
void hp_cuda_powersgd_decode(std::vector<std::shared_ptr<torch::Tensor>>& Ps,
                             std::vector<std::shared_ptr<torch::Tensor>>& Qs,
                             std::vector<std::shared_ptr<torch::Tensor>>& Ms,
                             std::vector<std::shared_ptr<torch::Tensor>>& residuals,
                             std::vector<std::shared_ptr<torch::Tensor>>& grads, Stream& stream) {
  using namespace hp_cuda_shim_detail;
  Dims d(Ms, Qs);
  auto p = ptrs(Ps), q = ptrs(Qs), m = ptrs(Ms), r = ptrs(residuals), g = ptrs(grads);
  auto ne = numels(grads);
  int ret = hpx_powersgd_decode(static_cast<int>(p.size()), cp(p), cp(q), m.data(), r.data(), g.data(), ne.data(),
                                d.n.data(), d.m.data(), d.r.data(), stream.stream());
  if (!ret) ret = finished(stream);
  if (ret) std::cout << "Call powersgd decode failed, ret = " << ret << ". " << hpx_last_error() << std::endl;
}
