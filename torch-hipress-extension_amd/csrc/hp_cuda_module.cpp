// hp_cuda: the reference's Python-visible extension module (PYBIND11_MODULE at
// hp_cuda.cpp:1073-1080) as a compiled torch extension over the scheduler of
// libhpx.so (include/hpx_sched.h).
//
//   init(alg_name, alg_paras, device_id, rank_id, size) -> bool       hp_cuda.cpp:824-874
//   end() -> bool                                                     hp_cuda.cpp:883-890
//   getResults(task_id) -> list[str]                                  hp_cuda.cpp:1043-1066
//   submit_task(name, tensor, B, C, is_root, task_id) -> bool         hp_cuda.cpp:984-1013
//   submit_task(name, tensor, residual, B, C, is_root, task_id)       hp_cuda.cpp:936-981
//   submit_task(name, tensor, residual, M, P, Q, task_id)             hp_cuda.cpp:1015-1041
//
// Same names, argument order, overload set and input checks (device tensors
// for tensor/residual/B/M/P/Q, a host tensor for C, all contiguous:
// hp_cuda.cpp:107-111, :942-945, :1015-1019).  Like the reference's Task
// (hp_cuda.h:28-51) a submitted task holds its tensors until the scheduler is
// done with them.  `wait`, `error_count` and `last_error` are additions.
//
// This file contains no device code and makes no HIP call: the scheduler owns
// its streams; here tensors are only checked and turned into pointers.
#include <torch/extension.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "hpx_sched.h"

namespace {

std::mutex g_mu;
std::unordered_map<uint64_t, std::vector<torch::Tensor>> g_in_flight;  // serial -> tensors of a task

void check_device_input(const torch::Tensor& x, const char* what) {
  TORCH_CHECK(x.is_cuda(), what, " must be a CUDA tensor");
  TORCH_CHECK(x.is_contiguous(), what, " must be contiguous");
}
void check_host_input(const torch::Tensor& x, const char* what) {
  TORCH_CHECK(!x.is_cuda(), what, " must be a CPU tensor");
  TORCH_CHECK(x.is_contiguous(), what, " must be contiguous");
}

// Drops the tensors of every task the scheduler has finished with.
void release_done() {
  uint64_t serials[256];
  for (;;) {
    const int64_t n = hpx_sched_take_done(serials, 256);
    {
      std::lock_guard<std::mutex> lock(g_mu);
      for (int64_t i = 0; i < n; i++) g_in_flight.erase(serials[i]);
    }
    if (n < 256) break;
  }
}

bool submit(const std::string& name, hpx_task_t& t, std::vector<torch::Tensor> keep) {
  release_done();
  t.name = name.c_str();
  uint64_t serial = 0;
  if (hpx_sched_submit(&t, &serial) != 0) {
    const std::string text = hpx_sched_error();
    // check_thread(), hp_cuda.cpp:892-900: submitting to a scheduler that is not running is an error
    TORCH_CHECK(text.find("not running") == std::string::npos, text);
    return false;  // the library has printed the reference's message
  }
  std::lock_guard<std::mutex> lock(g_mu);
  g_in_flight.emplace(serial, std::move(keep));
  return true;
}

bool init(const std::string& alg_name, const std::unordered_map<std::string, double>& alg_paras, int device_id,
          int rank_id, int size) {
  std::vector<const char*> keys;
  std::vector<double> values;
  for (const auto& kv : alg_paras) {
    keys.push_back(kv.first.c_str());
    values.push_back(kv.second);
  }
  return hpx_sched_init(alg_name.c_str(), keys.data(), values.data(), static_cast<int>(keys.size()), device_id,
                        rank_id, size) == 0;
}

bool end() {
  {
    pybind11::gil_scoped_release nogil;  // joins the worker thread
    hpx_sched_end();
  }
  release_done();
  return true;
}

bool submit_task_without_residual(const std::string& name, torch::Tensor tensor, torch::Tensor B, torch::Tensor C,
                                  int is_root, int task_id) {
  check_device_input(tensor, "tensor");
  check_device_input(B, "B");
  check_host_input(C, "C");
  hpx_task_t t{};
  t.task_id = task_id;
  t.is_root = is_root;
  t.tensor = static_cast<float*>(tensor.data_ptr());
  t.tensor_numel = tensor.numel();
  t.B = static_cast<uint8_t*>(B.data_ptr());
  t.B_bytes = B.numel() * B.element_size();
  t.C = static_cast<uint8_t*>(C.data_ptr());
  t.C_bytes = C.numel() * C.element_size();
  return submit(name, t, {tensor, B, C});
}

bool submit_task_with_residual(const std::string& name, torch::Tensor tensor, torch::Tensor residual, torch::Tensor B,
                               torch::Tensor C, int is_root, int task_id) {
  check_device_input(tensor, "tensor");
  check_device_input(residual, "residual");
  check_device_input(B, "B");
  check_host_input(C, "C");
  hpx_task_t t{};
  t.task_id = task_id;
  t.is_root = is_root;
  t.tensor = static_cast<float*>(tensor.data_ptr());
  t.tensor_numel = tensor.numel();
  t.residual = static_cast<float*>(residual.data_ptr());
  t.residual_numel = residual.numel();
  t.B = static_cast<uint8_t*>(B.data_ptr());
  t.B_bytes = B.numel() * B.element_size();
  t.C = static_cast<uint8_t*>(C.data_ptr());
  t.C_bytes = C.numel() * C.element_size();
  return submit(name, t, {tensor, residual, B, C});
}

bool submit_task_for_powersgd(const std::string& name, torch::Tensor tensor, torch::Tensor residual, torch::Tensor M,
                              torch::Tensor P, torch::Tensor Q, int task_id) {
  check_device_input(tensor, "tensor");
  check_device_input(residual, "residual");
  check_device_input(M, "M");
  check_device_input(P, "P");
  check_device_input(Q, "Q");
  TORCH_CHECK(M.dim() == 2 && P.dim() == 2 && Q.dim() == 2, "M, P and Q must be matrices");
  hpx_task_t t{};
  t.task_id = task_id;
  t.is_root = 0;
  t.tensor = static_cast<float*>(tensor.data_ptr());
  t.tensor_numel = tensor.numel();
  t.residual = static_cast<float*>(residual.data_ptr());
  t.residual_numel = residual.numel();
  t.M = static_cast<float*>(M.data_ptr());
  t.P = static_cast<float*>(P.data_ptr());
  t.Q = static_cast<float*>(Q.data_ptr());
  t.n = static_cast<int32_t>(M.size(0));
  t.m = static_cast<int32_t>(M.size(1));
  t.r = static_cast<int32_t>(P.size(1));
  return submit(name, t, {tensor, residual, M, P, Q});
}

std::vector<std::string> get_results(int task_id) {
  std::vector<std::string> out;
  std::vector<char> buf(1 << 16);
  for (;;) {
    const int64_t n = hpx_sched_get_results(task_id, buf.data(), static_cast<int64_t>(buf.size()));
    if (n <= 0) break;  // negative: the library has printed the reference's message
    const char* p = buf.data();
    for (int64_t i = 0; i < n; i++) {
      out.emplace_back(p);
      p += out.back().size() + 1;
    }
  }
  release_done();
  return out;
}

bool wait_for(int task_id, int timeout_ms) {
  pybind11::gil_scoped_release nogil;
  return hpx_sched_wait(task_id, timeout_ms) == 1;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "gradient compression tasks on MI355X (drop-in for the reference's hp_cuda extension)";
  m.def("init", &init, "init");
  m.def("end", &end, "end");
  m.def("getResults", &get_results, "get results");
  m.def("submit_task", &submit_task_without_residual, "submit task without residual");
  m.def("submit_task", &submit_task_with_residual, "submit task with residual");
  m.def("submit_task", &submit_task_for_powersgd, "submit task for powersgd");
  m.def("wait", &wait_for, pybind11::arg("task_id"), pybind11::arg("timeout_ms") = 1000,
        "block until getResults(task_id) would return something (True) or the time is up (False)");
  m.def("error_count", []() { return hpx_sched_error_count(); });
  m.def("last_error", []() { return std::string(hpx_sched_error()); });
  m.attr("COMP_TASK") = HPX_COMP_TASK;
  m.attr("DECOMP_TASK") = HPX_DECOMP_TASK;
  m.attr("ROOT_DECOMP_COMP_TASK") = HPX_ROOT_DECOMP_COMP_TASK;
  m.attr("POWERSGD_ENCODE1") = HPX_POWERSGD_ENCODE1;
  m.attr("POWERSGD_ENCODE2") = HPX_POWERSGD_ENCODE2;
  m.attr("POWERSGD_DECODE") = HPX_POWERSGD_DECODE;
}
