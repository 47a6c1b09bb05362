// TEST INFRASTRUCTURE ONLY.  C-ABI wrapper around the reference's own CPU
// implementation (k2/python/csrc/torch/mutual_information_cpu.cu), which the
// Makefile beside this file compiles in place from /root/reference into
// oracle/_ref/.  It exists so the restatement in mi_oracle.c can be checked
// bit-for-bit against the real code, and so bench.py can time the real code
// as the CPU baseline.  No reference source is copied: this file only
// declares the two entry points (k2/python/csrc/torch/mutual_information.h:80-106)
// and forwards raw buffers to them through torch::from_blob.
#include <torch/torch.h>

#include <cstdint>
#include <cstring>
#include <vector>

namespace k2 {
torch::Tensor MutualInformationCpu(torch::Tensor px, torch::Tensor py,
                                   torch::optional<torch::Tensor> boundary,
                                   torch::Tensor p);
std::vector<torch::Tensor> MutualInformationBackwardCpu(
    torch::Tensor px, torch::Tensor py, torch::optional<torch::Tensor> boundary,
    torch::Tensor p, torch::Tensor ans_grad);
}  // namespace k2

namespace {
torch::ScalarType DType(int is_f64) {
  return is_f64 ? torch::kFloat64 : torch::kFloat32;
}
torch::Tensor Wrap(const void *data, std::vector<int64_t> sizes, torch::ScalarType t) {
  return torch::from_blob(const_cast<void *>(data), sizes, torch::TensorOptions().dtype(t));
}
}  // namespace

extern "C" {

// Returns 0 on success, 1 if the reference threw.
int k2ref_mi_forward(const void *px, const void *py, const int64_t *boundary, void *p,
                     void *ans, int B, int S, int T, int modified, int is_f64) {
  try {
    auto dt = DType(is_f64);
    const int T1 = modified ? T : T + 1;
    auto px_t = Wrap(px, {B, S, T1}, dt), py_t = Wrap(py, {B, S + 1, T}, dt),
         p_t = Wrap(p, {B, S + 1, T + 1}, dt);
    torch::optional<torch::Tensor> bd;
    if (boundary) bd = Wrap(boundary, {B, 4}, torch::kInt64);
    auto out = k2::MutualInformationCpu(px_t, py_t, bd, p_t).contiguous();
    std::memcpy(ans, out.data_ptr(), out.numel() * out.element_size());
    return 0;
  } catch (...) {
    return 1;
  }
}

int k2ref_mi_backward(const void *px, const void *py, const int64_t *boundary, const void *p,
                      const void *ans_grad, void *px_grad, void *py_grad, int B, int S, int T,
                      int modified, int is_f64) {
  try {
    auto dt = DType(is_f64);
    const int T1 = modified ? T : T + 1;
    auto px_t = Wrap(px, {B, S, T1}, dt), py_t = Wrap(py, {B, S + 1, T}, dt),
         p_t = Wrap(p, {B, S + 1, T + 1}, dt), g_t = Wrap(ans_grad, {B}, dt);
    torch::optional<torch::Tensor> bd;
    if (boundary) bd = Wrap(boundary, {B, 4}, torch::kInt64);
    auto outs = k2::MutualInformationBackwardCpu(px_t, py_t, bd, p_t, g_t);
    auto gx = outs[0].contiguous(), gy = outs[1].contiguous();
    std::memcpy(px_grad, gx.data_ptr(), gx.numel() * gx.element_size());
    std::memcpy(py_grad, gy.data_ptr(), gy.numel() * gy.element_size());
    return 0;
  } catch (...) {
    return 1;
  }
}

}  // extern "C"
