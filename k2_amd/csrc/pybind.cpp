// pybind11 host module `_k2_amd`: the two native functions that k2's Python layer calls for the
// mutual-information recursion, with the reference's names and keyword arguments
// (k2/python/csrc/torch/mutual_information.cu:26-67), implemented over the C-ABI of libk2amd.so.
//
// Differences from the reference's host code, on purpose:
//   * launches go to torch's CURRENT HIP stream of the tensors' device (the reference uses the
//     legacy default stream, k2/python/csrc/torch/mutual_information_cuda.cu:712,784);
//   * the GIL is released around the launches;
//   * CPU tensors are rejected: this library has no CPU path.
#include <torch/extension.h>

// PyTorch-ROCm names its HIP devices "cuda"; these are the guard and stream types that go with it
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "k2_amd.h"

namespace {

void Check(int status) {
  TORCH_CHECK(status == K2AMD_OK, "k2_amd: ", k2amd_status_string(status));
}

int DtypeCode(const torch::Tensor &t) {
  if (t.scalar_type() == torch::kFloat) return K2AMD_F32;
  if (t.scalar_type() == torch::kDouble) return K2AMD_F64;
  TORCH_CHECK(false, "k2_amd: unsupported dtype ", t.scalar_type(), " (float32 / float64 only)");
  return -1;
}

// One workspace per (device, stream): grown on demand, initialised once; the kernels leave it
// ready for the next call.  Kept for the life of the process.
struct WorkspaceCache {
  std::mutex mu;
  std::map<std::pair<int, void *>, torch::Tensor> bufs;

  torch::Tensor Get(size_t bytes, const torch::Device &dev, void *stream) {
    if (bytes == 0) return torch::Tensor();
    std::lock_guard<std::mutex> lock(mu);
    auto key = std::make_pair(static_cast<int>(dev.index()), stream);
    auto it = bufs.find(key);
    if (it == bufs.end() || static_cast<size_t>(it->second.numel()) < bytes) {
      const int64_t n = static_cast<int64_t>(std::max(bytes, static_cast<size_t>(1) << 20));
      torch::Tensor ws = torch::empty({n}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
      Check(k2amd_mi_workspace_init(ws.data_ptr(), static_cast<size_t>(n), stream));
      bufs[key] = ws;
      return ws;
    }
    return it->second;
  }
};

WorkspaceCache &Cache() {
  static WorkspaceCache *cache = new WorkspaceCache();  // never destroyed: outlives torch's teardown
  return *cache;
}

struct Shape {
  int B, S, T, modified;
};

// The checks of k2/python/csrc/torch/mutual_information_cpu.cu:53-77, as RuntimeError.
Shape CheckInputs(const torch::Tensor &px, const torch::Tensor &py,
                  const torch::optional<torch::Tensor> &boundary, const torch::Tensor &p) {
  TORCH_CHECK(px.dim() == 3, "px must be 3-dimensional");
  TORCH_CHECK(py.dim() == 3, "py must be 3-dimensional");
  TORCH_CHECK(p.dim() == 3, "p must be 3-dimensional");
  TORCH_CHECK(px.is_cuda(), "k2_amd runs on MI355X only: px is on ", px.device(),
              " (there is no CPU path)");
  TORCH_CHECK(py.device() == px.device() && p.device() == px.device(),
              "inputs must be on the same device");
  TORCH_CHECK(px.scalar_type() == py.scalar_type() && px.scalar_type() == p.scalar_type(),
              "px, py and p must have the same dtype");
  const int64_t B = px.size(0), S = px.size(1), T = py.size(2);
  TORCH_CHECK(px.size(2) == T || px.size(2) == T + 1, "px.size(2) must be T or T+1");
  TORCH_CHECK(py.size(0) == B && py.size(1) == S + 1, "py must have shape [B][S+1][T]");
  TORCH_CHECK(p.size(0) == B && p.size(1) == S + 1 && p.size(2) == T + 1,
              "p must have shape [B][S+1][T+1]");
  TORCH_CHECK(p.is_contiguous(), "p must be contiguous");
  if (boundary.has_value() && boundary->defined()) {
    TORCH_CHECK(boundary->scalar_type() == torch::kLong, "boundary must be int64");
    TORCH_CHECK(boundary->dim() == 2 && boundary->size(0) == B && boundary->size(1) == 4,
                "boundary must have shape [B][4]");
    TORCH_CHECK(boundary->device() == px.device(), "boundary must be on px's device");
  }
  return Shape{static_cast<int>(B), static_cast<int>(S), static_cast<int>(T),
               px.size(2) == T ? 1 : 0};
}

torch::Tensor MutualInformationForward(torch::Tensor px, torch::Tensor py,
                                       torch::optional<torch::Tensor> boundary, torch::Tensor p) {
  const Shape sh = CheckInputs(px, py, boundary, p);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(px.device());
  px = px.contiguous();
  py = py.contiguous();
  torch::Tensor bd;
  if (boundary.has_value() && boundary->defined()) bd = boundary->contiguous();
  torch::Tensor ans = torch::empty({sh.B}, px.options());
  const int dt = DtypeCode(px);
  void *stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(px.device().index()).stream();
  torch::Tensor ws = Cache().Get(k2amd_mi_workspace_bytes(sh.B, sh.S, sh.T, sh.modified, dt),
                                 px.device(), stream);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_mi_forward(px.data_ptr(), py.data_ptr(),
                           bd.defined() ? bd.data_ptr<int64_t>() : nullptr, p.data_ptr(),
                           ans.data_ptr(), sh.B, sh.S, sh.T, sh.modified, dt,
                           ws.defined() ? ws.data_ptr() : nullptr,
                           ws.defined() ? static_cast<size_t>(ws.numel()) : 0, stream));
  }
  return ans;
}

std::vector<torch::Tensor> MutualInformationBackward(torch::Tensor px, torch::Tensor py,
                                                     torch::optional<torch::Tensor> boundary,
                                                     torch::Tensor p, torch::Tensor ans_grad) {
  const Shape sh = CheckInputs(px, py, boundary, p);
  TORCH_CHECK(ans_grad.dim() == 1 && ans_grad.size(0) == sh.B, "ans_grad must have shape [B]");
  TORCH_CHECK(ans_grad.device() == px.device() && ans_grad.scalar_type() == px.scalar_type(),
              "ans_grad must match px in device and dtype");
  TORCH_CHECK(ans_grad.is_contiguous(), "ans_grad must be contiguous");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(px.device());
  px = px.contiguous();
  py = py.contiguous();
  torch::Tensor bd;
  if (boundary.has_value() && boundary->defined()) bd = boundary->contiguous();
  // every element is written by the kernels, so plain `empty` serves where the reference needs
  // `zeros` (k2/python/csrc/torch/mutual_information_cpu.cu:160-166)
  torch::Tensor px_grad = torch::empty_like(px), py_grad = torch::empty_like(py);
  const int dt = DtypeCode(px);
  void *stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(px.device().index()).stream();
  torch::Tensor ws = Cache().Get(k2amd_mi_workspace_bytes(sh.B, sh.S, sh.T, sh.modified, dt),
                                 px.device(), stream);
  {
    pybind11::gil_scoped_release release;
    // like the reference's device path, ans_grad is overwritten with the gradient that reached
    // the origin (k2/python/csrc/torch/mutual_information_cuda.cu:661-663)
    Check(k2amd_mi_backward(px.data_ptr(), py.data_ptr(),
                            bd.defined() ? bd.data_ptr<int64_t>() : nullptr, p.data_ptr(),
                            ans_grad.data_ptr(), px_grad.data_ptr(), py_grad.data_ptr(), sh.B, sh.S,
                            sh.T, sh.modified, dt, /*overwrite_ans_grad=*/1,
                            ws.defined() ? ws.data_ptr() : nullptr,
                            ws.defined() ? static_cast<size_t>(ws.numel()) : 0, stream));
  }
  return {px_grad, py_grad};
}

}  // namespace

PYBIND11_MODULE(_k2_amd, m) {
  m.doc() = "MI355X host layer of the k2 mutual-information recursion";
  m.def("mutual_information_forward", &MutualInformationForward, pybind11::arg("px"),
        pybind11::arg("py"), pybind11::arg("boundary"), pybind11::arg("p"));
  m.def("mutual_information_backward", &MutualInformationBackward, pybind11::arg("px"),
        pybind11::arg("py"), pybind11::arg("boundary"), pybind11::arg("p"),
        pybind11::arg("ans_grad"));
  m.def("version", []() { return k2amd_version(); });
}
