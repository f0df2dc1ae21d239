// hp_cuda_drivers: Python access to the nine kernel-driver functions with the reference's own C++
// signatures (declared in hp_cuda.cpp:18-102, defined in hp_cuda_kernel.cu): the six vector-based ones
// exported by libhpx.so (hp_cuda_shim.h) and the three PowerSGD ones over torch tensors
// (hp_cuda_shim_torch.h).  Each function below builds its argument vectors the way the reference's
// scheduler loops do (hp_cuda.cpp:284-301, :464-477, :610-611, :729-752) from lists of torch tensors and
// calls the driver on torch's current stream; nothing is returned, as in the reference.
//
// The reference has no such module (its drivers are only reachable through the scheduler); this one
// exists so that the drop-in signatures themselves are compiled and exercised by the GPU tests.
// Host C++ only.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include "hp_cuda_shim.h"
#include "hp_cuda_shim_torch.h"

namespace {

using Tensors = std::vector<torch::Tensor>;

void check(const Tensors& ts, const char* what) {
  for (const auto& t : ts) {
    TORCH_CHECK(t.is_cuda(), what, " must be CUDA tensors");
    TORCH_CHECK(t.is_contiguous(), what, " must be contiguous");
  }
}
std::vector<float*> f32_ptrs(const Tensors& ts) {
  std::vector<float*> p;
  for (const auto& t : ts) p.push_back(static_cast<float*>(t.data_ptr()));
  return p;
}
std::vector<uint8_t*> u8_ptrs(const Tensors& ts) {
  std::vector<uint8_t*> p;
  for (const auto& t : ts) p.push_back(static_cast<uint8_t*>(t.data_ptr()));
  return p;
}
std::vector<int32_t> sizes(const Tensors& ts) {
  std::vector<int32_t> n;
  for (const auto& t : ts) n.push_back(static_cast<int32_t>(t.numel()));
  return n;
}
std::vector<std::shared_ptr<torch::Tensor>> shared(const Tensors& ts) {
  std::vector<std::shared_ptr<torch::Tensor>> v;
  for (const auto& t : ts) v.push_back(std::make_shared<torch::Tensor>(t));
  return v;
}
hipStream_t current_stream() { return c10::hip::getCurrentHIPStream().stream(); }

void terngrad(Tensors ins, Tensors outs, std::vector<uint8_t> bitwidths, std::vector<int32_t> enable_randoms) {
  check(ins, "inputs"); check(outs, "outputs");
  auto in = f32_ptrs(ins); auto in_sizes = sizes(ins);
  auto out = u8_ptrs(outs); auto out_sizes = sizes(outs);
  hp_cuda_terngrad(in, in_sizes, out, out_sizes, bitwidths, enable_randoms, current_stream());
}
void terngradr(Tensors outs, Tensors ins, std::vector<int> is_add_tos) {
  check(ins, "inputs"); check(outs, "outputs");
  auto out = f32_ptrs(outs); auto out_sizes = sizes(outs);
  auto in = u8_ptrs(ins); auto in_sizes = sizes(ins);
  hp_cuda_terngradr(out, out_sizes, in, in_sizes, is_add_tos, current_stream());
}
void tbq(Tensors grads, Tensors residuals, Tensors outs, std::vector<float> thresholds) {
  check(grads, "gradients"); check(residuals, "residuals"); check(outs, "outputs");
  auto g = f32_ptrs(grads); auto g_sizes = sizes(grads);
  auto r = f32_ptrs(residuals); auto r_sizes = sizes(residuals);
  auto out = u8_ptrs(outs); auto out_sizes = sizes(outs);
  hp_cuda_tbq(g, g_sizes, r, r_sizes, out, out_sizes, thresholds, current_stream());
}
void tbqr(Tensors outs, Tensors ins, std::vector<float> thresholds, std::vector<int> is_add_tos) {
  check(ins, "inputs"); check(outs, "outputs");
  auto out = f32_ptrs(outs); auto out_sizes = sizes(outs);
  auto in = u8_ptrs(ins); auto in_sizes = sizes(ins);
  hp_cuda_tbqr(out, out_sizes, in, in_sizes, thresholds, is_add_tos, current_stream());
}
void gd(Tensors grads, Tensors residuals, Tensors outs, std::vector<double> sample_rates, std::vector<double> drop_ratios) {
  check(grads, "gradients"); check(residuals, "residuals"); check(outs, "outputs");
  auto g = f32_ptrs(grads); auto Ns = sizes(grads);
  auto r = f32_ptrs(residuals); auto r_sizes = sizes(residuals);
  auto out = u8_ptrs(outs);
  hp_cuda_gd(g, Ns, r, r_sizes, out, sample_rates, drop_ratios, current_stream());
}
void gdr(Tensors ins, std::vector<int32_t> in_sizes, Tensors outs, std::vector<int> is_add_tos) {
  check(ins, "inputs"); check(outs, "outputs");
  auto in = u8_ptrs(ins);
  auto out = f32_ptrs(outs); auto out_sizes = sizes(outs);
  hp_cuda_gdr(in, in_sizes, out, out_sizes, is_add_tos, current_stream());
}
void powersgd_encode1(Tensors grads, Tensors residuals, Tensors Qs, Tensors Ms, Tensors Ps) {
  check(grads, "gradients"); check(residuals, "residuals"); check(Qs, "Qs"); check(Ms, "Ms"); check(Ps, "Ps");
  auto g = shared(grads), r = shared(residuals), q = shared(Qs), m = shared(Ms), p = shared(Ps);
  auto stream = c10::hip::getCurrentHIPStream();
  hp_cuda_powersgd_encode1(g, r, q, m, p, stream);
}
void powersgd_encode2(Tensors Ps, Tensors Ms, Tensors Qs) {
  check(Ps, "Ps"); check(Ms, "Ms"); check(Qs, "Qs");
  auto p = shared(Ps), m = shared(Ms), q = shared(Qs);
  auto stream = c10::hip::getCurrentHIPStream();
  hp_cuda_powersgd_encode2(p, m, q, stream);
}
void powersgd_decode(Tensors Ps, Tensors Qs, Tensors Ms, Tensors residuals, Tensors grads) {
  check(Ps, "Ps"); check(Qs, "Qs"); check(Ms, "Ms"); check(residuals, "residuals"); check(grads, "gradients");
  auto p = shared(Ps), q = shared(Qs), m = shared(Ms), r = shared(residuals), g = shared(grads);
  auto stream = c10::hip::getCurrentHIPStream();
  hp_cuda_powersgd_decode(p, q, m, r, g, stream);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "the nine hp_cuda_* kernel drivers with the reference's C++ signatures, callable on lists of tensors";
  m.def("hp_cuda_terngrad", &terngrad);
  m.def("hp_cuda_terngradr", &terngradr);
  m.def("hp_cuda_tbq", &tbq);
  m.def("hp_cuda_tbqr", &tbqr);
  m.def("hp_cuda_gd", &gd);
  m.def("hp_cuda_gdr", &gdr);
  m.def("hp_cuda_powersgd_encode1", &powersgd_encode1);
  m.def("hp_cuda_powersgd_encode2", &powersgd_encode2);
  m.def("hp_cuda_powersgd_decode", &powersgd_decode);
}
