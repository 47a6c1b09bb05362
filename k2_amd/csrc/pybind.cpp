// pybind11 host module `_k2_amd`: the two native functions that k2's Python layer calls for the
// mutual-information recursion, with the reference's names and keyword arguments
// (k2/python/csrc/torch/mutual_information.cu:26-67), and host functions for the fused builders
// that replace the reference's torch-op chains, all implemented over the C-ABI of libk2amd.so.
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
#include <ATen/hip/HIPEvent.h>

#include <algorithm>
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

  // the buffer of (device, stream) if there is one
  torch::Tensor Find(const torch::Device &dev, void *stream) {
    std::lock_guard<std::mutex> lock(mu);
    auto it = bufs.find(std::make_pair(static_cast<int>(dev.index()), stream));
    return it == bufs.end() ? torch::Tensor() : it->second;
  }

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

WorkspaceCache &Cache();

// Synchronises the stream of every cached workspace and reads its error flag.  A workspace whose
// kernels gave up a wait (their ans came out as NaN) is initialised again, so that the calls after
// this one work; returns how many were.  No counterpart in the reference.
int64_t MutualInformationRecoverWorkspaces() {
  WorkspaceCache &cache = Cache();
  std::lock_guard<std::mutex> lock(cache.mu);
  int64_t recovered = 0;
  for (auto &kv : cache.bufs) {
    torch::Tensor &ws = kv.second;
    c10::hip::HIPGuardMasqueradingAsCUDA guard(ws.device());
    const int status = k2amd_mi_workspace_status(ws.data_ptr(), kv.first.second);
    if (status == K2AMD_ERR_TIMEOUT) {
      Check(k2amd_mi_workspace_init(ws.data_ptr(), static_cast<size_t>(ws.numel()), kv.first.second));
      ++recovered;
    } else {
      Check(status);
    }
  }
  return recovered;
}

// The buffer that the pipelined kernels use on `like`'s device and current stream, or None where
// no call has needed one yet (for diagnostics and for tests that force its error flag from the
// host).  No counterpart in the reference.
pybind11::object MutualInformationWorkspace(const torch::Tensor &like) {
  TORCH_CHECK(like.is_cuda(), "k2_amd: a device tensor names the device");
  void *stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(like.device().index()).stream();
  torch::Tensor ws = Cache().Find(like.device(), stream);
  if (!ws.defined()) return pybind11::none();
  return pybind11::cast(ws);
}

WorkspaceCache &Cache() {
  static WorkspaceCache *cache = new WorkspaceCache();  // never destroyed: outlives torch's teardown
  return *cache;
}

struct Shape {
  int B, S, T, modified;
};

// The checks of k2/python/csrc/torch/mutual_information_cpu.cu:53-77, as RuntimeError.
// `lattice`: p (or, where p is left out, the log-derivative tensor that stands in for it); null
// for a call without either.
Shape CheckInputs(const torch::Tensor &px, const torch::Tensor &py,
                  const torch::optional<torch::Tensor> &boundary, const torch::Tensor *lattice) {
  TORCH_CHECK(px.dim() == 3, "px must be 3-dimensional");
  TORCH_CHECK(py.dim() == 3, "py must be 3-dimensional");
  TORCH_CHECK(px.is_cuda(), "k2_amd runs on MI355X only: px is on ", px.device(),
              " (there is no CPU path)");
  TORCH_CHECK(py.device() == px.device(), "inputs must be on the same device");
  TORCH_CHECK(px.scalar_type() == py.scalar_type(), "px and py must have the same dtype");
  const int64_t B = px.size(0), S = px.size(1), T = py.size(2);
  TORCH_CHECK(px.size(2) == T || px.size(2) == T + 1, "px.size(2) must be T or T+1");
  TORCH_CHECK(py.size(0) == B && py.size(1) == S + 1, "py must have shape [B][S+1][T]");
  if (lattice != nullptr) {
    const torch::Tensor &p = *lattice;
    TORCH_CHECK(p.dim() == 3, "p must be 3-dimensional");
    TORCH_CHECK(p.device() == px.device(), "inputs must be on the same device");
    TORCH_CHECK(px.scalar_type() == p.scalar_type(), "px, py and p must have the same dtype");
    TORCH_CHECK(p.size(0) == B && p.size(1) == S + 1 && p.size(2) == T + 1,
                "p must have shape [B][S+1][T+1]");
    TORCH_CHECK(p.is_contiguous(), "p must be contiguous");
  }
  if (boundary.has_value() && boundary->defined()) {
    TORCH_CHECK(boundary->scalar_type() == torch::kLong, "boundary must be int64");
    TORCH_CHECK(boundary->dim() == 2 && boundary->size(0) == B && boundary->size(1) == 4,
                "boundary must have shape [B][4]");
    TORCH_CHECK(boundary->device() == px.device(), "boundary must be on px's device");
  }
  return Shape{static_cast<int>(B), static_cast<int>(S), static_cast<int>(T),
               px.size(2) == T ? 1 : 0};
}

// log_deriv: optional tensor shaped and typed like p that carries the px-edge log-derivatives
// from the forward call to the backward call of the same inputs (k2amd_mi_forward_keep /
// k2amd_mi_backward_kept in include/k2_amd.h).
// p may be None where log_deriv stands in for it (see the header); the one that is given first
// goes through CheckInputs, the other is compared with it.
bool Given(const torch::optional<torch::Tensor> &t) { return t.has_value() && t->defined(); }
const torch::Tensor &LatticeOf(const torch::optional<torch::Tensor> &p,
                               const torch::optional<torch::Tensor> &log_deriv) {
  TORCH_CHECK(Given(p) || Given(log_deriv), "p may only be None where log_deriv is given");
  return Given(p) ? *p : *log_deriv;
}
void *CheckLogDeriv(const torch::optional<torch::Tensor> &log_deriv, const torch::Tensor &lattice) {
  if (!Given(log_deriv)) return nullptr;
  TORCH_CHECK(log_deriv->sizes() == lattice.sizes() &&
                  log_deriv->scalar_type() == lattice.scalar_type() &&
                  log_deriv->device() == lattice.device() && log_deriv->is_contiguous(),
              "log_deriv must be a contiguous tensor with p's shape, dtype and device");
  return log_deriv->data_ptr();
}

bool MutualInformationKeepsLogDeriv(torch::Tensor px, torch::Tensor py) {
  TORCH_CHECK(px.dim() == 3 && py.dim() == 3, "px and py must have three dimensions");
  const int B = static_cast<int>(px.size(0)), S = static_cast<int>(px.size(1)),
            T = static_cast<int>(py.size(2)), modified = px.size(2) == T ? 1 : 0;
  const int dt = DtypeCode(px);
  return k2amd_mi_keeps_log_deriv(B, S, T, modified, dt,
                                  k2amd_mi_workspace_bytes(B, S, T, modified, dt) > 0) != 0;
}

torch::Tensor MutualInformationForward(torch::Tensor px, torch::Tensor py,
                                       torch::optional<torch::Tensor> boundary,
                                       torch::optional<torch::Tensor> p,
                                       torch::optional<torch::Tensor> log_deriv) {
  const torch::Tensor &lattice = LatticeOf(p, log_deriv);
  const Shape sh = CheckInputs(px, py, boundary, &lattice);
  void *kept = CheckLogDeriv(log_deriv, lattice);
  void *p_ptr = Given(p) ? p->data_ptr() : nullptr;
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
    Check(k2amd_mi_forward_keep(px.data_ptr(), py.data_ptr(),
                                bd.defined() ? bd.data_ptr<int64_t>() : nullptr, p_ptr,
                                ans.data_ptr(), kept, sh.B, sh.S, sh.T, sh.modified, dt,
                                ws.defined() ? ws.data_ptr() : nullptr,
                                ws.defined() ? static_cast<size_t>(ws.numel()) : 0, stream));
  }
  return ans;
}

std::vector<torch::Tensor> MutualInformationBackward(torch::Tensor px, torch::Tensor py,
                                                     torch::optional<torch::Tensor> boundary,
                                                     torch::optional<torch::Tensor> p,
                                                     torch::Tensor ans_grad,
                                                     torch::optional<torch::Tensor> log_deriv) {
  const torch::Tensor &lattice = LatticeOf(p, log_deriv);
  const Shape sh = CheckInputs(px, py, boundary, &lattice);
  const void *kept = CheckLogDeriv(log_deriv, lattice);
  const void *p_ptr = Given(p) ? p->data_ptr() : nullptr;
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
    Check(k2amd_mi_backward_kept(px.data_ptr(), py.data_ptr(),
                                 bd.defined() ? bd.data_ptr<int64_t>() : nullptr, p_ptr, kept,
                                 ans_grad.data_ptr(), px_grad.data_ptr(), py_grad.data_ptr(), sh.B,
                                 sh.S, sh.T, sh.modified, dt, /*overwrite_ans_grad=*/1,
                                 ws.defined() ? ws.data_ptr() : nullptr,
                                 ws.defined() ? static_cast<size_t>(ws.numel()) : 0, stream));
  }
  return {px_grad, py_grad};
}

bool MutualInformationForwardBackwardSupported(torch::Tensor px, torch::Tensor py) {
  TORCH_CHECK(px.dim() == 3 && py.dim() == 3, "px and py must have three dimensions");
  if (!px.is_cuda()) return false;
  const int B = static_cast<int>(px.size(0)), S = static_cast<int>(px.size(1)),
            T = static_cast<int>(py.size(2)), modified = px.size(2) == T ? 1 : 0;
  const int dt = DtypeCode(px);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(px.device());  // the answer depends on the device
  return k2amd_mi_forward_backward_supported(B, S, T, modified, dt,
                                             k2amd_mi_workspace_bytes(B, S, T, modified, dt) > 0) != 0;
}

bool MutualInformationForwardBackwardAdvised(torch::Tensor px, torch::Tensor py) {
  TORCH_CHECK(px.dim() == 3 && py.dim() == 3, "px and py must have three dimensions");
  if (!px.is_cuda()) return false;
  const int B = static_cast<int>(px.size(0)), S = static_cast<int>(px.size(1)),
            T = static_cast<int>(py.size(2)), modified = px.size(2) == T ? 1 : 0;
  const int dt = DtypeCode(px);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(px.device());  // the answer depends on the device
  return k2amd_mi_forward_backward_advised(B, S, T, modified, dt,
                                           k2amd_mi_workspace_bytes(B, S, T, modified, dt) > 0) != 0;
}

// The two calls above in one launch (k2amd_mi_forward_backward): returns {ans, px_grad, py_grad}
// and overwrites ans_grad like MutualInformationBackward.
std::vector<torch::Tensor> MutualInformationForwardBackward(torch::Tensor px, torch::Tensor py,
                                                            torch::optional<torch::Tensor> boundary,
                                                            torch::optional<torch::Tensor> ans_grad) {
  TORCH_CHECK(px.dim() == 3 && py.dim() == 3, "px and py must have three dimensions");
  TORCH_CHECK(px.is_cuda(), "k2_amd runs on MI355X only: px is on ", px.device(),
              " (there is no CPU path)");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(px.device());
  const Shape sh = CheckInputs(px, py, boundary, nullptr);
  void *seed = nullptr;  // None: every score has gradient 1
  if (ans_grad.has_value() && ans_grad->defined()) {
    TORCH_CHECK(ans_grad->dim() == 1 && ans_grad->size(0) == sh.B, "ans_grad must have shape [B]");
    TORCH_CHECK(ans_grad->device() == px.device() && ans_grad->scalar_type() == px.scalar_type(),
                "ans_grad must match px in device and dtype");
    TORCH_CHECK(ans_grad->is_contiguous(), "ans_grad must be contiguous");
    seed = ans_grad->data_ptr();
  }
  px = px.contiguous();
  py = py.contiguous();
  torch::Tensor bd;
  if (boundary.has_value() && boundary->defined()) bd = boundary->contiguous();
  torch::Tensor ans = torch::empty({sh.B}, px.options());
  torch::Tensor px_grad = torch::empty_like(px), py_grad = torch::empty_like(py);
  const int dt = DtypeCode(px);
  // the launch's scratch (the px-edge log-derivatives of both halves of every lattice)
  const size_t scratch_bytes = k2amd_mi_forward_backward_scratch_bytes(sh.B, sh.S, sh.T, sh.modified, dt);
  torch::Tensor scratch = torch::empty({static_cast<int64_t>(std::max<size_t>(scratch_bytes, 4))},
                                       px.options().dtype(torch::kUInt8));
  void *stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(px.device().index()).stream();
  torch::Tensor ws = Cache().Get(k2amd_mi_workspace_bytes(sh.B, sh.S, sh.T, sh.modified, dt),
                                 px.device(), stream);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_mi_forward_backward(px.data_ptr(), py.data_ptr(),
                                    bd.defined() ? bd.data_ptr<int64_t>() : nullptr, ans.data_ptr(),
                                    scratch.data_ptr(), static_cast<size_t>(scratch.numel()), seed,
                                    px_grad.data_ptr(), py_grad.data_ptr(), sh.B, sh.S, sh.T, sh.modified, dt,
                                    /*overwrite_ans_grad=*/1, ws.defined() ? ws.data_ptr() : nullptr,
                                    ws.defined() ? static_cast<size_t>(ws.numel()) : 0, stream));
  }
  return {ans, px_grad, py_grad};
}

// ---------------------------------------------------------------------------------------------
// The fused builders that replace the torch-op chains of k2/python/k2/rnnt_loss.py.  Each mirrors
// the C-ABI entry point of the same name (include/k2_amd.h): outputs are allocated here, raw
// pointers go down, tensors come back.  Inputs must be contiguous and on one ROCm device.

void *StreamOf(const torch::Tensor &t) {
  return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}
void RequireDevice(const torch::Tensor &t, const char *name) {
  TORCH_CHECK(t.is_cuda(), "k2_amd runs on MI355X only: ", name, " is on ", t.device(),
              " (there is no CPU path)");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}
// The kernels index every tensor of a call with the sizes taken from ONE of them, so a tensor of
// another shape, element size or device would be read out of bounds: each host function below
// checks all of its tensors with these before a pointer goes down (RuntimeError, nothing launched).
void Expect(const torch::Tensor &t, const char *name, c10::ScalarType dtype, const torch::Device &dev,
            std::initializer_list<int64_t> shape) {
  RequireDevice(t, name);
  TORCH_CHECK(t.scalar_type() == dtype && t.device() == dev && t.sizes() == torch::IntArrayRef(shape),
              "k2_amd: ", name, " must be ", dtype, " ", torch::IntArrayRef(shape), " on ", dev, ", got ",
              t.scalar_type(), " ", t.sizes(), " on ", t.device());
}
void ExpectOptional(const torch::optional<torch::Tensor> &t, const char *name, c10::ScalarType dtype,
                    const torch::Device &dev, std::initializer_list<int64_t> shape) {
  if (t.has_value() && t->defined()) Expect(*t, name, dtype, dev, shape);
}
// a float32 / float64 device tensor with n dimensions: the tensor the sizes of a call are read from
void ExpectFloat(const torch::Tensor &t, const char *name, int64_t n) {
  RequireDevice(t, name);
  DtypeCode(t);
  TORCH_CHECK(t.dim() == n, "k2_amd: ", name, " must have ", n, " dimensions, got ", t.dim());
}
void ExpectRnntType(int rnnt_type) {
  TORCH_CHECK(rnnt_type == K2AMD_REGULAR || rnnt_type == K2AMD_MODIFIED || rnnt_type == K2AMD_CONSTRAINED,
              "k2_amd: unknown rnnt_type code ", rnnt_type);
}
void ExpectSymbol(int symbol, int64_t C) {
  TORCH_CHECK(symbol >= 0 && symbol < C, "k2_amd: termination_symbol ", symbol, " outside [0, ", C, ")");
}
const int64_t *I64(const torch::optional<torch::Tensor> &t) {
  if (!t.has_value() || !t->defined()) return nullptr;
  TORCH_CHECK(t->scalar_type() == torch::kLong && t->is_contiguous() && t->is_cuda(),
              "index tensors must be contiguous int64 device tensors");
  return t->data_ptr<int64_t>();
}
int T1Of(int T, int rnnt_type) { return rnnt_type == K2AMD_REGULAR ? T + 1 : T; }
void ExpectLatticeGrads(const torch::Tensor &px_grad, const torch::Tensor &py_grad,
                        const torch::optional<torch::Tensor> &seq_scale, c10::ScalarType dtype,
                        const torch::Device &dev, int64_t B, int64_t S, int64_t T, int rnnt_type) {
  Expect(px_grad, "px_grad", dtype, dev, {B, S, T1Of(static_cast<int>(T), rnnt_type)});
  Expect(py_grad, "py_grad", dtype, dev, {B, S + 1, T});
  ExpectOptional(seq_scale, "seq_scale", dtype, dev, {B});
}

// get_rnnt_logprobs: returns (px, py, lm_probs, am_probs, denom)
std::vector<torch::Tensor> LogprobsSimpleForward(torch::Tensor lm, torch::Tensor am,
                                                 torch::Tensor symbols, int termination_symbol,
                                                 int rnnt_type,
                                                 torch::optional<torch::Tensor> boundary) {
  ExpectFloat(am, "am", 3);
  ExpectFloat(lm, "lm", 3);
  ExpectRnntType(rnnt_type);
  const int B = am.size(0), T = am.size(1), C = am.size(2), S = lm.size(1) - 1;
  Expect(lm, "lm", am.scalar_type(), am.device(), {B, S + 1, C});
  Expect(symbols, "symbols", torch::kLong, am.device(), {B, S});
  ExpectOptional(boundary, "boundary", torch::kLong, am.device(), {B, 4});
  ExpectSymbol(termination_symbol, C);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(am.device());
  auto opt = am.options();
  torch::Tensor px = torch::empty({B, S, T1Of(T, rnnt_type)}, opt), py = torch::empty({B, S + 1, T}, opt);
  torch::Tensor lm_probs = torch::empty_like(lm), am_probs = torch::empty_like(am);
  torch::Tensor lm_max = torch::empty({B, S + 1}, opt), am_max = torch::empty({B, T}, opt);
  torch::Tensor denom = torch::empty({B, S + 1, T}, opt);
  void *stream = StreamOf(am);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_logprobs_simple_forward(
        lm.data_ptr(), am.data_ptr(), I64(symbols), I64(boundary), px.data_ptr(), py.data_ptr(),
        lm_probs.data_ptr(), am_probs.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(),
        denom.data_ptr(), B, S, T, C, termination_symbol, rnnt_type, DtypeCode(am), stream));
  }
  return {px, py, lm_probs, am_probs, denom};
}

// seq_scale of the *_backward entry points: [B], contiguous, dtype and device of the gradients
const void *ScalePtr(const torch::optional<torch::Tensor> &seq_scale, const torch::Tensor &px_grad) {
  if (!seq_scale.has_value() || !seq_scale->defined()) return nullptr;
  TORCH_CHECK(seq_scale->dim() == 1 && seq_scale->size(0) == px_grad.size(0) &&
                  seq_scale->scalar_type() == px_grad.scalar_type() &&
                  seq_scale->device() == px_grad.device() && seq_scale->is_contiguous(),
              "seq_scale must be a contiguous [B] tensor with the gradients' dtype and device");
  return seq_scale->data_ptr();
}

std::vector<torch::Tensor> LogprobsSimpleBackward(torch::Tensor px_grad, torch::Tensor py_grad,
                                                  torch::Tensor symbols,
                                                  torch::optional<torch::Tensor> boundary,
                                                  torch::Tensor lm_probs, torch::Tensor am_probs,
                                                  torch::Tensor denom, int termination_symbol,
                                                  int rnnt_type,
                                                  torch::optional<torch::Tensor> seq_scale) {
  ExpectFloat(am_probs, "am_probs", 3);
  ExpectFloat(lm_probs, "lm_probs", 3);
  ExpectRnntType(rnnt_type);
  const int B = am_probs.size(0), T = am_probs.size(1), C = am_probs.size(2), S = lm_probs.size(1) - 1;
  const auto dtype = am_probs.scalar_type();
  const auto dev = am_probs.device();
  Expect(lm_probs, "lm_probs", dtype, dev, {B, S + 1, C});
  Expect(denom, "denom", dtype, dev, {B, S + 1, T});
  Expect(symbols, "symbols", torch::kLong, dev, {B, S});
  ExpectOptional(boundary, "boundary", torch::kLong, dev, {B, 4});
  ExpectLatticeGrads(px_grad, py_grad, seq_scale, dtype, dev, B, S, T, rnnt_type);
  ExpectSymbol(termination_symbol, C);
  const void *scale = ScalePtr(seq_scale, px_grad);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(am_probs.device());
  torch::Tensor lm_grad = torch::empty_like(lm_probs), am_grad = torch::empty_like(am_probs);
  // the products' operand [B][S+1][T], then the gradients' sums along s and along t
  torch::Tensor q = torch::empty(
      {static_cast<int64_t>(k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T))}, denom.options());
  void *stream = StreamOf(am_probs);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_logprobs_simple_backward(
        px_grad.data_ptr(), py_grad.data_ptr(), scale, I64(symbols), I64(boundary), lm_probs.data_ptr(),
        am_probs.data_ptr(), denom.data_ptr(), lm_grad.data_ptr(), am_grad.data_ptr(), q.data_ptr(),
        static_cast<size_t>(q.numel()), B, S, T, C, termination_symbol, rnnt_type, DtypeCode(am_probs), stream));
  }
  return {lm_grad, am_grad};
}

// get_rnnt_logprobs_smoothed (k2/python/k2/rnnt_loss.py:1471-1704): the simple builder on the
// lattice without a boundary, then the marginal terms and the mix.  Returns (px, py, lm_probs,
// am_probs, denom, lm_max, am_max, lm_norm, am_norm, unigram); all but the first two are for the
// backward.
std::vector<torch::Tensor> LogprobsSmoothedForward(torch::Tensor lm, torch::Tensor am, torch::Tensor symbols,
                                                   int termination_symbol, double lm_only_scale,
                                                   double am_only_scale, int rnnt_type,
                                                   torch::optional<torch::Tensor> boundary) {
  ExpectFloat(am, "am", 3);
  ExpectFloat(lm, "lm", 3);
  ExpectRnntType(rnnt_type);
  const int B = am.size(0), T = am.size(1), C = am.size(2), S = lm.size(1) - 1;
  Expect(lm, "lm", am.scalar_type(), am.device(), {B, S + 1, C});
  Expect(symbols, "symbols", torch::kLong, am.device(), {B, S});
  ExpectOptional(boundary, "boundary", torch::kLong, am.device(), {B, 4});
  ExpectSymbol(termination_symbol, C);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(am.device());
  auto opt = am.options();
  const int joint_type = rnnt_type == K2AMD_REGULAR ? K2AMD_REGULAR : K2AMD_MODIFIED;
  torch::Tensor px_joint = torch::empty({B, S, T1Of(T, rnnt_type)}, opt), py_joint = torch::empty({B, S + 1, T}, opt);
  torch::Tensor px = torch::empty_like(px_joint), py = torch::empty_like(py_joint);
  torch::Tensor lm_probs = torch::empty_like(lm), am_probs = torch::empty_like(am);
  torch::Tensor lm_max = torch::empty({B, S + 1}, opt), am_max = torch::empty({B, T}, opt);
  torch::Tensor lm_norm = torch::empty({B, S + 1}, opt), am_norm = torch::empty({B, T}, opt);
  torch::Tensor denom = torch::empty({B, S + 1, T}, opt), unigram = torch::empty({2, C}, opt);
  torch::Tensor scratch =
      torch::empty({static_cast<int64_t>(k2amd_rnnt_smoothed_scratch_elements(B, S, T, C))}, opt);
  void *stream = StreamOf(am);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_logprobs_simple_forward(
        lm.data_ptr(), am.data_ptr(), I64(symbols), nullptr, px_joint.data_ptr(), py_joint.data_ptr(),
        lm_probs.data_ptr(), am_probs.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(), denom.data_ptr(), B, S, T,
        C, termination_symbol, joint_type, DtypeCode(am), stream));
    Check(k2amd_rnnt_smoothed_forward(
        lm.data_ptr(), am.data_ptr(), I64(symbols), I64(boundary), lm_probs.data_ptr(), am_probs.data_ptr(),
        lm_max.data_ptr(), am_max.data_ptr(), px_joint.data_ptr(), py_joint.data_ptr(), px.data_ptr(),
        py.data_ptr(), lm_norm.data_ptr(), am_norm.data_ptr(), unigram.data_ptr(), scratch.data_ptr(),
        static_cast<size_t>(scratch.numel()), lm_only_scale, am_only_scale, B, S, T, C, termination_symbol,
        rnnt_type, DtypeCode(am), stream));
  }
  return {px, py, lm_probs, am_probs, denom, lm_max, am_max, lm_norm, am_norm, unigram};
}

// (lm_grad, am_grad): the simple builder's backward with the gradients scaled by
// 1 - lm_only_scale - am_only_scale, then the marginal terms' gradients added.
std::vector<torch::Tensor> LogprobsSmoothedBackward(
    torch::Tensor px_grad, torch::Tensor py_grad, torch::Tensor symbols, torch::optional<torch::Tensor> boundary,
    torch::Tensor lm_probs, torch::Tensor am_probs, torch::Tensor denom, torch::Tensor lm_max, torch::Tensor am_max,
    torch::Tensor lm_norm, torch::Tensor am_norm, torch::Tensor unigram, int termination_symbol,
    double lm_only_scale, double am_only_scale, int rnnt_type, torch::optional<torch::Tensor> seq_scale) {
  ExpectFloat(am_probs, "am_probs", 3);
  ExpectFloat(lm_probs, "lm_probs", 3);
  ExpectRnntType(rnnt_type);
  const int B = am_probs.size(0), T = am_probs.size(1), C = am_probs.size(2), S = lm_probs.size(1) - 1;
  const auto dtype = am_probs.scalar_type();
  const auto dev = am_probs.device();
  Expect(lm_probs, "lm_probs", dtype, dev, {B, S + 1, C});
  Expect(denom, "denom", dtype, dev, {B, S + 1, T});
  Expect(lm_max, "lm_max", dtype, dev, {B, S + 1});
  Expect(lm_norm, "lm_norm", dtype, dev, {B, S + 1});
  Expect(am_max, "am_max", dtype, dev, {B, T});
  Expect(am_norm, "am_norm", dtype, dev, {B, T});
  Expect(unigram, "unigram", dtype, dev, {2, C});
  Expect(symbols, "symbols", torch::kLong, dev, {B, S});
  ExpectOptional(boundary, "boundary", torch::kLong, dev, {B, 4});
  ExpectLatticeGrads(px_grad, py_grad, seq_scale, dtype, dev, B, S, T, rnnt_type);
  ExpectSymbol(termination_symbol, C);
  const void *scale = ScalePtr(seq_scale, px_grad);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  const double joint_scale = 1.0 - lm_only_scale - am_only_scale;
  torch::Tensor joint_seq_scale = scale != nullptr ? (*seq_scale * joint_scale).contiguous()
                                                   : torch::full({B}, joint_scale, am_probs.options());
  torch::Tensor lm_grad = torch::empty_like(lm_probs), am_grad = torch::empty_like(am_probs);
  torch::Tensor q = torch::empty(
      {static_cast<int64_t>(k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T))}, denom.options());
  torch::Tensor scratch =
      torch::empty({static_cast<int64_t>(k2amd_rnnt_smoothed_scratch_elements(B, S, T, C))}, denom.options());
  void *stream = StreamOf(am_probs);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_logprobs_simple_backward(
        px_grad.data_ptr(), py_grad.data_ptr(), joint_seq_scale.data_ptr(), I64(symbols), I64(boundary),
        lm_probs.data_ptr(), am_probs.data_ptr(), denom.data_ptr(), lm_grad.data_ptr(), am_grad.data_ptr(),
        q.data_ptr(), static_cast<size_t>(q.numel()), B, S, T, C, termination_symbol, rnnt_type,
        DtypeCode(am_probs), stream));
    Check(k2amd_rnnt_smoothed_backward(
        px_grad.data_ptr(), py_grad.data_ptr(), scale, I64(symbols), I64(boundary), lm_probs.data_ptr(),
        am_probs.data_ptr(), lm_max.data_ptr(), am_max.data_ptr(), lm_norm.data_ptr(), am_norm.data_ptr(),
        unigram.data_ptr(), lm_grad.data_ptr(), am_grad.data_ptr(), scratch.data_ptr(),
        static_cast<size_t>(scratch.numel()), lm_only_scale, am_only_scale, B, S, T, C, termination_symbol,
        rnnt_type, DtypeCode(am_probs), stream));
  }
  return {lm_grad, am_grad};
}

// get_rnnt_logprobs_joint: returns (px, py, normalizers)
std::vector<torch::Tensor> LogprobsJointForward(torch::Tensor logits, torch::Tensor symbols,
                                                int termination_symbol, int rnnt_type,
                                                torch::optional<torch::Tensor> boundary) {
  ExpectFloat(logits, "logits", 4);
  ExpectRnntType(rnnt_type);
  const int B = logits.size(0), T = logits.size(1), S = logits.size(2) - 1, C = logits.size(3);
  Expect(symbols, "symbols", torch::kLong, logits.device(), {B, S});
  ExpectOptional(boundary, "boundary", torch::kLong, logits.device(), {B, 4});
  ExpectSymbol(termination_symbol, C);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
  auto opt = logits.options();
  torch::Tensor px = torch::empty({B, S, T1Of(T, rnnt_type)}, opt), py = torch::empty({B, S + 1, T}, opt);
  torch::Tensor norm = torch::empty({B, T, S + 1}, opt);
  void *stream = StreamOf(logits);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_logprobs_joint_forward(logits.data_ptr(), I64(symbols), I64(boundary),
                                            px.data_ptr(), py.data_ptr(), norm.data_ptr(), B, S, T, C,
                                            termination_symbol, rnnt_type, DtypeCode(logits), stream));
  }
  return {px, py, norm};
}

torch::Tensor LogprobsJointBackward(torch::Tensor logits, torch::Tensor norm, torch::Tensor px_grad,
                                    torch::Tensor py_grad, torch::Tensor symbols,
                                    torch::optional<torch::Tensor> boundary, int termination_symbol,
                                    int rnnt_type, torch::optional<torch::Tensor> seq_scale) {
  ExpectFloat(logits, "logits", 4);
  ExpectRnntType(rnnt_type);
  const int B = logits.size(0), T = logits.size(1), S = logits.size(2) - 1, C = logits.size(3);
  Expect(norm, "normalizers", logits.scalar_type(), logits.device(), {B, T, S + 1});
  Expect(symbols, "symbols", torch::kLong, logits.device(), {B, S});
  ExpectOptional(boundary, "boundary", torch::kLong, logits.device(), {B, 4});
  ExpectLatticeGrads(px_grad, py_grad, seq_scale, logits.scalar_type(), logits.device(), B, S, T, rnnt_type);
  ExpectSymbol(termination_symbol, C);
  const void *scale = ScalePtr(seq_scale, px_grad);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
  torch::Tensor grad = torch::empty_like(logits);
  void *stream = StreamOf(logits);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_logprobs_joint_backward(logits.data_ptr(), norm.data_ptr(), px_grad.data_ptr(),
                                             py_grad.data_ptr(), scale, I64(symbols), I64(boundary),
                                             grad.data_ptr(), B, S, T, C, termination_symbol, rnnt_type,
                                             DtypeCode(logits), stream));
  }
  return grad;
}

// get_rnnt_logprobs_pruned, or get_hat_logprobs_pruned with hat = true: returns
// (px, py, normalizers)
std::vector<torch::Tensor> LogprobsPrunedForward(torch::Tensor logits, torch::Tensor symbols,
                                                 torch::Tensor ranges, int termination_symbol,
                                                 torch::optional<torch::Tensor> boundary,
                                                 int rnnt_type, bool hat) {
  ExpectFloat(logits, "logits", 4);
  ExpectRnntType(rnnt_type);
  TORCH_CHECK(symbols.dim() == 2, "k2_amd: symbols must have 2 dimensions");
  const int B = logits.size(0), T = logits.size(1), R = logits.size(2), C = logits.size(3);
  const int S = symbols.size(1);
  Expect(symbols, "symbols", torch::kLong, logits.device(), {B, S});
  Expect(ranges, "ranges", torch::kLong, logits.device(), {B, T, R});
  ExpectOptional(boundary, "boundary", torch::kLong, logits.device(), {B, 4});
  ExpectSymbol(hat ? 0 : termination_symbol, C);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
  auto opt = logits.options();
  torch::Tensor px = torch::empty({B, S, T1Of(T, rnnt_type)}, opt), py = torch::empty({B, S + 1, T}, opt);
  torch::Tensor norm = torch::empty({B, T, R}, opt);
  void *stream = StreamOf(logits);
  {
    pybind11::gil_scoped_release release;
    if (hat)
      Check(k2amd_rnnt_hat_logprobs_pruned_forward(logits.data_ptr(), I64(symbols), I64(ranges),
                                                   I64(boundary), px.data_ptr(), py.data_ptr(),
                                                   norm.data_ptr(), B, S, T, R, C, rnnt_type,
                                                   DtypeCode(logits), stream));
    else
      Check(k2amd_rnnt_logprobs_pruned_forward(logits.data_ptr(), I64(symbols), I64(ranges),
                                               I64(boundary), px.data_ptr(), py.data_ptr(),
                                               norm.data_ptr(), B, S, T, R, C, termination_symbol,
                                               rnnt_type, DtypeCode(logits), stream));
  }
  return {px, py, norm};
}

torch::Tensor LogprobsPrunedBackward(torch::Tensor logits, torch::Tensor norm, torch::Tensor px_grad,
                                     torch::Tensor py_grad, torch::Tensor symbols, torch::Tensor ranges,
                                     torch::optional<torch::Tensor> boundary, int termination_symbol,
                                     int rnnt_type, bool hat,
                                     torch::optional<torch::Tensor> seq_scale) {
  ExpectFloat(logits, "logits", 4);
  ExpectRnntType(rnnt_type);
  TORCH_CHECK(symbols.dim() == 2, "k2_amd: symbols must have 2 dimensions");
  const int B = logits.size(0), T = logits.size(1), R = logits.size(2), C = logits.size(3);
  const int S = symbols.size(1);
  Expect(norm, "normalizers", logits.scalar_type(), logits.device(), {B, T, R});
  Expect(symbols, "symbols", torch::kLong, logits.device(), {B, S});
  Expect(ranges, "ranges", torch::kLong, logits.device(), {B, T, R});
  ExpectOptional(boundary, "boundary", torch::kLong, logits.device(), {B, 4});
  ExpectLatticeGrads(px_grad, py_grad, seq_scale, logits.scalar_type(), logits.device(), B, S, T, rnnt_type);
  ExpectSymbol(hat ? 0 : termination_symbol, C);
  const void *scale = ScalePtr(seq_scale, px_grad);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
  torch::Tensor grad = torch::empty_like(logits);
  void *stream = StreamOf(logits);
  {
    pybind11::gil_scoped_release release;
    if (hat)
      Check(k2amd_rnnt_hat_logprobs_pruned_backward(
          logits.data_ptr(), norm.data_ptr(), px_grad.data_ptr(), py_grad.data_ptr(), scale,
          I64(symbols), I64(ranges), I64(boundary), grad.data_ptr(), B, S, T, R, C, rnnt_type, DtypeCode(logits),
          stream));
    else
      Check(k2amd_rnnt_logprobs_pruned_backward(
          logits.data_ptr(), norm.data_ptr(), px_grad.data_ptr(), py_grad.data_ptr(), scale,
          I64(symbols), I64(ranges), I64(boundary), grad.data_ptr(), B, S, T, R, C, termination_symbol, rnnt_type,
          DtypeCode(logits), stream));
  }
  return grad;
}

// device part of get_rnnt_prune_ranges (deprecated: of get_rnnt_prune_ranges_deprecated);
// s_range is the final value
torch::Tensor PruneRanges(torch::Tensor px_grad, torch::Tensor py_grad, torch::Tensor boundary,
                          int s_range, bool deprecated) {
  ExpectFloat(px_grad, "px_grad", 3);
  ExpectFloat(py_grad, "py_grad", 3);
  const int B = px_grad.size(0), S = px_grad.size(1), T1 = px_grad.size(2), T = py_grad.size(2);
  TORCH_CHECK(T1 == T || T1 == T + 1, "k2_amd: px_grad.size(2) must be T or T+1");
  Expect(py_grad, "py_grad", px_grad.scalar_type(), px_grad.device(), {B, S + 1, T});
  Expect(boundary, "boundary", torch::kLong, px_grad.device(), {B, 4});
  TORCH_CHECK(s_range >= 1 && s_range <= S + 1, "k2_amd: s_range ", s_range, " outside [1, S + 1 = ", S + 1, "]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(px_grad.device());
  torch::Tensor ranges = torch::empty({B, T, s_range}, px_grad.options().dtype(torch::kLong));
  void *stream = StreamOf(px_grad);
  {
    pybind11::gil_scoped_release release;
    auto entry = deprecated ? k2amd_rnnt_prune_ranges_deprecated : k2amd_rnnt_prune_ranges;
    Check(entry(px_grad.data_ptr(), py_grad.data_ptr(), I64(boundary), ranges.data_ptr<int64_t>(),
                B, S, T, T1 == T ? 1 : 0, s_range, DtypeCode(px_grad), stream));
  }
  return ranges;
}

torch::Tensor PruneGather(torch::Tensor lm, torch::Tensor ranges) {
  ExpectFloat(lm, "lm", 3);
  TORCH_CHECK(ranges.dim() == 3, "k2_amd: ranges must have 3 dimensions");
  const int B = lm.size(0), S1 = lm.size(1), D = lm.size(2), T = ranges.size(1), R = ranges.size(2);
  Expect(ranges, "ranges", torch::kLong, lm.device(), {B, T, R});
  c10::hip::HIPGuardMasqueradingAsCUDA guard(lm.device());
  torch::Tensor out = torch::empty({B, T, R, D}, lm.options());
  void *stream = StreamOf(lm);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_prune_gather(lm.data_ptr(), I64(ranges), out.data_ptr(), B, S1, T, R, D,
                                  DtypeCode(lm), stream));
  }
  return out;
}

torch::Tensor PruneGatherBackward(torch::Tensor grad, torch::Tensor ranges, int S1) {
  ExpectFloat(grad, "grad", 4);
  const int B = grad.size(0), T = grad.size(1), R = grad.size(2), D = grad.size(3);
  Expect(ranges, "ranges", torch::kLong, grad.device(), {B, T, R});
  TORCH_CHECK(S1 >= 1, "k2_amd: S1 must be positive");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(grad.device());
  torch::Tensor lm_grad = torch::empty({B, S1, D}, grad.options());
  void *stream = StreamOf(grad);
  {
    pybind11::gil_scoped_release release;
    Check(k2amd_rnnt_prune_gather_backward(grad.data_ptr(), I64(ranges), lm_grad.data_ptr(), B, S1, T,
                                           R, D, DtypeCode(grad), stream));
  }
  return lm_grad;
}

// _k2.pruned_ranges_to_lattice (k2/python/csrc/torch/pruned_ranges_to_lattice.cu:265-281).  The
// lattice comes back as its parts: (state_splits [B+1], arc_splits [states+1],
// arcs int32 [arcs][4] with the score's bits in column 3, arc_map int32 [arcs]).
std::vector<torch::Tensor> PrunedRangesToLattice(torch::Tensor ranges, torch::Tensor frames,
                                                 torch::Tensor symbols, torch::Tensor logits) {
  TORCH_CHECK(ranges.dim() == 3, "ranges should be 3-dimensional");
  TORCH_CHECK(frames.dim() == 1, "frames should be 1-dimensional");
  TORCH_CHECK(symbols.dim() == 2, "symbols should be 2-dimensional");
  TORCH_CHECK(logits.dim() == 4, "logits should be 4-dimensional");
  TORCH_CHECK(ranges.scalar_type() == torch::kInt && frames.scalar_type() == torch::kInt,
              "ranges and frames must be int32");
  TORCH_CHECK(symbols.scalar_type() == torch::kLong, "symbols must be int64");
  RequireDevice(ranges, "ranges");
  RequireDevice(frames, "frames");
  RequireDevice(symbols, "symbols");
  TORCH_CHECK(logits.is_cuda(), "k2_amd runs on MI355X only: logits is on ", logits.device(),
              " (there is no CPU path)");
  TORCH_CHECK(frames.device() == ranges.device() && symbols.device() == ranges.device() &&
                  logits.device() == ranges.device(),
              "inputs must be on the same device");
  const int B = ranges.size(0), T = ranges.size(1), R = ranges.size(2);
  const int S = symbols.size(1), C = logits.size(3);
  TORCH_CHECK(frames.size(0) == B && symbols.size(0) == B && logits.size(0) == B &&
                  logits.size(1) == T && logits.size(2) == R,
              "shapes of ranges, frames, symbols and logits do not agree");
  int dtype = K2AMD_F32;
  if (logits.scalar_type() == torch::kDouble) dtype = K2AMD_F64;
  else if (logits.scalar_type() == torch::kHalf) dtype = K2AMD_F16;
  else TORCH_CHECK(logits.scalar_type() == torch::kFloat, "logits must be float32, float64 or float16");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(ranges.device());
  auto i32 = ranges.options();
  torch::Tensor arc_local = torch::empty({B, T * R + 1}, i32), seq_arcs = torch::empty({std::max(B, 1)}, i32);
  // (one buffer for the two prefix sums: their totals then come to the host in one copy)
  torch::Tensor splits = torch::empty({2, B + 1}, i32);
  torch::Tensor state_splits = splits[0], arc_base = splits[1];
  void *stream = StreamOf(ranges);
  Check(k2amd_lattice_count(ranges.data_ptr<int32_t>(), frames.data_ptr<int32_t>(),
                            arc_local.data_ptr<int32_t>(), seq_arcs.data_ptr<int32_t>(),
                            state_splits.data_ptr<int32_t>(), arc_base.data_ptr<int32_t>(), B, T, R,
                            stream));
  // the one host read on this path (the reference reads the same totals to size its arrays)
  const torch::Tensor totals = splits.select(1, B).cpu();
  const int n_states = totals[0].item<int32_t>(), n_arcs = totals[1].item<int32_t>();
  torch::Tensor arc_splits = B > 0 ? torch::empty({n_states + 1}, i32) : torch::zeros({1}, i32);
  torch::Tensor arcs = torch::empty({n_arcs, 4}, i32), arc_map = torch::empty({n_arcs}, i32);
  const int64_t strides[4] = {logits.stride(0), logits.stride(1), logits.stride(2), logits.stride(3)};
  Check(k2amd_lattice_fill(ranges.data_ptr<int32_t>(), frames.data_ptr<int32_t>(), I64(symbols),
                           logits.data_ptr(), strides, state_splits.data_ptr<int32_t>(),
                           arc_base.data_ptr<int32_t>(), arc_local.data_ptr<int32_t>(),
                           arc_splits.data_ptr<int32_t>(), arcs.data_ptr(),
                           arc_map.data_ptr<int32_t>(), B, T, R, S, C, dtype, stream));
  return {state_splits, arc_splits, arcs, arc_map};
}

}  // namespace

namespace {

// prods [N][B] of joint_mutual_information_recursion (k2/python/k2/mutual_information.py:404-417):
// px, py lists of N tensors shaped like px_grad and py_grad.
torch::Tensor MutualInformationJointProducts(std::vector<torch::Tensor> px, std::vector<torch::Tensor> py,
                                             torch::Tensor px_grad, torch::Tensor py_grad) {
  const int N = static_cast<int>(px.size());
  TORCH_CHECK(N >= 1 && py.size() == px.size(), "as many px as py, at least one of each");
  ExpectFloat(px_grad, "px_grad", 3);
  const auto dtype = px_grad.scalar_type();
  const auto dev = px_grad.device();
  auto same = [&](const torch::Tensor &t, const char *name, const torch::Tensor &like) {
    RequireDevice(t, name);
    TORCH_CHECK(t.scalar_type() == dtype && t.device() == dev && t.sizes() == like.sizes(), "k2_amd: ",
                name, " must be ", dtype, " ", like.sizes(), " on ", dev, ", got ", t.scalar_type(), " ",
                t.sizes(), " on ", t.device());
  };
  TORCH_CHECK(py_grad.dim() == 3 && py_grad.size(0) == px_grad.size(0), "py_grad must be [B][S+1][T]");
  same(py_grad, "py_grad", py_grad);
  std::vector<const void *> xs(N), ys(N);
  for (int n = 0; n < N; ++n) {
    same(px[n], "px[n]", px_grad);
    same(py[n], "py[n]", py_grad);
    xs[n] = px[n].data_ptr();
    ys[n] = py[n].data_ptr();
  }
  const int B = px_grad.size(0);
  const long long kx = B ? px_grad.numel() / B : 0, ky = B ? py_grad.numel() / B : 0;
  c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
  torch::Tensor prods = torch::empty({N, B}, px_grad.options());
  torch::Tensor partial = torch::empty(
      {static_cast<int64_t>(k2amd_mi_joint_products_scratch_elements(N, B))}, px_grad.options());
  void *stream = StreamOf(px_grad);
  Check(k2amd_mi_joint_products(xs.data(), ys.data(), N, px_grad.data_ptr(), py_grad.data_ptr(),
                                prods.data_ptr(), partial.data_ptr(), B, kx, ky, DtypeCode(px_grad), stream));
  return prods;
}

}  // namespace

// The rows of a [B][4] boundary tensor on their way to the host: a non-blocking copy into pinned
// memory on the tensor's current stream and an event behind it.  Rows() waits for that event
// alone (not for what was queued after the copy) and returns the rows as tuples of Python
// integers, what k2's range asserts read (k2/python/k2/mutual_information.py:284-289).
// The error flag of the stream's workspace for the pipelined kernels rides along: a launch that
// gave up a bounded wait (its scores came out as NaN, and so would those of every later launch on
// that workspace) is reported here, at the caller's next call, as a RuntimeError, and the
// workspace is initialised again so that the call after that one works.
class BoundaryRead {
 public:
  explicit BoundaryRead(const torch::Tensor &boundary) {
    TORCH_CHECK(boundary.is_cuda() && boundary.dim() == 2 && boundary.size(1) == 4 &&
                    boundary.scalar_type() == torch::kLong,
                "boundary must be a [B][4] int64 tensor on the device");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(boundary.device());
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(boundary.device().index());
    pinned_ = torch::empty(boundary.sizes(), torch::TensorOptions().dtype(torch::kLong).pinned_memory(true));
    pinned_.copy_(boundary, /*non_blocking=*/true);
    stream_ = stream.stream();
    workspace_ = Cache().Find(boundary.device(), stream_);
    if (workspace_.defined()) {
      flag_ = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt).pinned_memory(true));
      Check(k2amd_mi_workspace_status_async(workspace_.data_ptr(),
                                            reinterpret_cast<unsigned *>(flag_.data_ptr<int>()), stream_));
    }
    event_.record(stream);
  }
  pybind11::tuple Rows() {
    {
      pybind11::gil_scoped_release release;
      event_.synchronize();
    }
    if (flag_.defined() && flag_.data_ptr<int>()[0] != 0) {
      flag_.data_ptr<int>()[0] = 0;  // (reported once)
      c10::hip::HIPGuardMasqueradingAsCUDA guard(workspace_.device());
      Check(k2amd_mi_workspace_init(workspace_.data_ptr(), static_cast<size_t>(workspace_.numel()), stream_));
      TORCH_CHECK(false, "k2_amd: ", k2amd_status_string(K2AMD_ERR_TIMEOUT),
                  ": an earlier launch of the mutual-information kernels on this stream gave up waiting for a "
                  "neighbouring workgroup, so its scores and gradients (NaN) are invalid; the workspace has "
                  "been initialised again, the next call will work");
    }
    const int64_t B = pinned_.size(0);
    const int64_t *v = pinned_.data_ptr<int64_t>();
    pybind11::tuple rows(B);
    for (int64_t b = 0; b < B; ++b)
      rows[b] = pybind11::make_tuple(v[4 * b], v[4 * b + 1], v[4 * b + 2], v[4 * b + 3]);
    return rows;
  }

 private:
  torch::Tensor pinned_, flag_, workspace_;
  void *stream_ = nullptr;
  at::cuda::CUDAEvent event_;
};

PYBIND11_MODULE(_k2_amd, m) {
  m.doc() = "MI355X host layer of the k2 mutual-information recursion";
  pybind11::class_<BoundaryRead>(m, "BoundaryRead")
      .def(pybind11::init<const torch::Tensor &>(), pybind11::arg("boundary"))
      .def("rows", &BoundaryRead::Rows);
  m.def("mutual_information_forward", &MutualInformationForward, pybind11::arg("px"),
        pybind11::arg("py"), pybind11::arg("boundary"), pybind11::arg("p"),
        pybind11::arg("log_deriv") = pybind11::none());
  m.def("mutual_information_recover_workspaces", &MutualInformationRecoverWorkspaces);
  m.def("mutual_information_workspace", &MutualInformationWorkspace, pybind11::arg("like"));
  m.def("mutual_information_joint_products", &MutualInformationJointProducts, pybind11::arg("px"),
        pybind11::arg("py"), pybind11::arg("px_grad"), pybind11::arg("py_grad"));
  m.def("mutual_information_keeps_log_deriv", &MutualInformationKeepsLogDeriv, pybind11::arg("px"),
        pybind11::arg("py"));
  m.def("mutual_information_backward", &MutualInformationBackward, pybind11::arg("px"),
        pybind11::arg("py"), pybind11::arg("boundary"), pybind11::arg("p"),
        pybind11::arg("ans_grad"), pybind11::arg("log_deriv") = pybind11::none());
  m.def("mutual_information_forward_backward_supported", &MutualInformationForwardBackwardSupported,
        pybind11::arg("px"), pybind11::arg("py"));
  m.def("mutual_information_forward_backward_advised", &MutualInformationForwardBackwardAdvised,
        pybind11::arg("px"), pybind11::arg("py"));
  m.def("mutual_information_forward_backward", &MutualInformationForwardBackward,
        pybind11::arg("px"), pybind11::arg("py"), pybind11::arg("boundary"),
        pybind11::arg("ans_grad"));
  m.def("version", []() { return k2amd_version(); });
  m.def("logprobs_simple_forward", &LogprobsSimpleForward);
  m.def("logprobs_simple_backward", &LogprobsSimpleBackward);
  m.def("logprobs_smoothed_forward", &LogprobsSmoothedForward);
  m.def("logprobs_smoothed_backward", &LogprobsSmoothedBackward);
  m.def("smoothed_supported", [](int B, int S, int T, int C, int dtype) {
    return k2amd_rnnt_smoothed_supported(B, S, T, C, dtype) != 0;
  });
  m.def("logprobs_joint_forward", &LogprobsJointForward);
  m.def("logprobs_joint_backward", &LogprobsJointBackward);
  m.def("logprobs_pruned_forward", &LogprobsPrunedForward);
  m.def("logprobs_pruned_backward", &LogprobsPrunedBackward);
  m.def("prune_ranges", &PruneRanges, pybind11::arg("px_grad"), pybind11::arg("py_grad"),
        pybind11::arg("boundary"), pybind11::arg("s_range"), pybind11::arg("deprecated") = false);
  m.def("prune_gather", &PruneGather);
  m.def("prune_gather_backward", &PruneGatherBackward);
  m.def("pruned_ranges_to_lattice", &PrunedRangesToLattice, pybind11::arg("ranges"),
        pybind11::arg("frames"), pybind11::arg("symbols"), pybind11::arg("logits"));
}
