// extern "C" entry points of the MI recursion: argument checks and kernel selection.
#include <atomic>
#include <cstdlib>
#include <cstring>

#include "common.h"
#include "mi_internal.h"

using namespace k2amd;

namespace {

bool ShapeOk(int B, int S, int T) {
  if (B < 0 || S < 0 || T < 0) return false;
  // kernels index one sequence's lattice with 32-bit offsets
  return ((int64_t)S + 1) * ((int64_t)T + 1) < (int64_t)1 << 31;
}

// Switches for tests and comparisons, read at every call: K2AMD_MI_PATH=generic forces the exact
// log-domain kernels; K2AMD_MI_PATH=two-launches keeps the pipelined kernels but never serves the
// single launch; K2AMD_MI_PATH=single-launch advises the single launch wherever it is served.
bool PathIs(const char *name) {
  const char *e = std::getenv("K2AMD_MI_PATH");
  return e != nullptr && std::strcmp(e, name) == 0;
}
bool ForceGeneric() { return PathIs("generic"); }

// ---- scratch of the entry point that allocates nothing (k2amd_mi_forward_noalloc) --------------
// One array per device that loads this library, held until the process ends.  The name below is a
// host-side stand-in for the symbol, NOT a device address: host code only ever uses the pointer
// that hipGetSymbolAddress returned for the device that is current (ScratchOfCurrentDevice).
constexpr size_t kScratchBytes = K2AMD_MI_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// Device address of `scratch` on the current device (asked of the runtime once per device
// ordinal, with that device current), or nullptr.
void *ScratchOfCurrentDevice() {
  static std::atomic<void *> ptrs[64];  // nullptr = not asked yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  void *ptr = ptrs[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    ptrs[dev].store(ptr, std::memory_order_release);  // every thread would store the same address
  }
  return ptr;
}

}  // namespace

extern "C" {

int k2amd_version(void) { return K2AMD_VERSION; }

const char *k2amd_status_string(int status) {
  switch (status) {
    case K2AMD_OK: return "ok";
    case K2AMD_ERR_INVALID_ARGUMENT: return "invalid argument";
    case K2AMD_ERR_UNSUPPORTED: return "unsupported size for this build";
    case K2AMD_ERR_WORKSPACE: return "workspace missing or too small";
    case K2AMD_ERR_LAUNCH: return "HIP launch error";
    case K2AMD_ERR_TIMEOUT: return "in-kernel wait timed out; workspace must be re-initialised";
    case K2AMD_ERR_SCRATCH_LIMIT: return "shape needs more scratch than the static array of the no-allocation entry point holds";
    default: return "unknown status";
  }
}

size_t k2amd_mi_workspace_bytes(int B, int S, int T, int modified, int dtype) {
  (void)modified;
  if (!ShapeOk(B, S, T) || B == 0) return 0;
  if (dtype == K2AMD_F64) return MiWaveSupports(B, S, T) ? MiWaveWorkspaceBytes(B, S, T) : 0;
  if (dtype != K2AMD_F32) return 0;
  return MiFastWorkspaceBytes(B, S, T);
}

int k2amd_mi_workspace_init(void *workspace, size_t workspace_bytes, void *stream) {
  return MiFastWorkspaceInit(workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int k2amd_mi_workspace_status(const void *workspace, void *stream) {
  if (workspace == nullptr) return K2AMD_ERR_INVALID_ARGUMENT;
  unsigned header[4] = {0, 0, 0, 0};
  if (hipMemcpyAsync(header, workspace, sizeof(header), hipMemcpyDeviceToHost,
                     static_cast<hipStream_t>(stream)) != hipSuccess ||
      hipStreamSynchronize(static_cast<hipStream_t>(stream)) != hipSuccess)
    return K2AMD_ERR_LAUNCH;
  return header[2] != 0 ? K2AMD_ERR_TIMEOUT : K2AMD_OK;  // FastHeader::error
}

int k2amd_mi_workspace_status_async(const void *workspace, unsigned *host_flag, void *stream) {
  if (workspace == nullptr || host_flag == nullptr) return K2AMD_ERR_INVALID_ARGUMENT;
  // FastHeader::error is the third word of the buffer
  if (hipMemcpyAsync(host_flag, static_cast<const unsigned *>(workspace) + 2, sizeof(unsigned),
                     hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)) != hipSuccess)
    return K2AMD_ERR_LAUNCH;
  return K2AMD_OK;
}

int k2amd_mi_keeps_log_deriv(int B, int S, int T, int modified, int dtype, int has_workspace) {
  return dtype == K2AMD_F32 && has_workspace && ShapeOk(B, S, T) && B > 0 && !ForceGeneric() &&
         MiFastSupports(B, S, T, modified ? 1 : 0);
}

int k2amd_mi_forward(const void *px, const void *py, const int64_t *boundary, void *p, void *ans,
                     int B, int S, int T, int modified, int dtype, void *workspace,
                     size_t workspace_bytes, void *stream) {
  return k2amd_mi_forward_keep(px, py, boundary, p, ans, nullptr, B, S, T, modified, dtype,
                               workspace, workspace_bytes, stream);
}

int k2amd_mi_forward_keep(const void *px, const void *py, const int64_t *boundary, void *p,
                          void *ans, void *log_deriv, int B, int S, int T, int modified, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream) {
  if (!ShapeOk(B, S, T) || (dtype != K2AMD_F32 && dtype != K2AMD_F64)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0) return K2AMD_OK;
  if (!ans || (!px && S > 0) || (!py && T > 0)) return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  modified = modified ? 1 : 0;
  const bool fast = dtype == K2AMD_F32 && workspace != nullptr && !ForceGeneric() && MiFastSupports(B, S, T, modified);
  // p may be left out only where the log-derivative tensor stands in for it
  if (!p && !(fast && log_deriv)) return K2AMD_ERR_INVALID_ARGUMENT;
  // fp32 with a workspace takes the pipelined throughput path (fp64 has its own, further down);
  // without a workspace the exact one-workgroup-per-sequence kernels run.
  if (fast) {
    if (workspace_bytes < MiFastWorkspaceBytes(B, S, T)) return K2AMD_ERR_WORKSPACE;
    return MiForwardFast((const float *)px, (const float *)py, boundary, (float *)p, (float *)ans,
                         (float *)log_deriv, B, S, T, modified, workspace, workspace_bytes, st);
  }
  if (dtype == K2AMD_F32)
    return MiForwardGeneric<float>((const float *)px, (const float *)py, boundary, (float *)p,
                                   (float *)ans, B, S, T, modified, st);
  // fp64 with a workspace: one wavefront per 64-row chunk, pipelined
  if (workspace != nullptr && !ForceGeneric() && MiWaveSupports(B, S, T)) {
    if (workspace_bytes < MiWaveWorkspaceBytes(B, S, T)) return K2AMD_ERR_WORKSPACE;
    return MiForwardWave((const double *)px, (const double *)py, boundary, (double *)p, (double *)ans,
                         B, S, T, modified, workspace, workspace_bytes, st);
  }
  return MiForwardGeneric<double>((const double *)px, (const double *)py, boundary, (double *)p,
                                  (double *)ans, B, S, T, modified, st);
}

int k2amd_mi_forward_noalloc(const void *px, const void *py, const int64_t *boundary, void *p,
                             void *ans, int B, int S, int T, int modified, int dtype, void *stream) {
  if (!ShapeOk(B, S, T) || (dtype != K2AMD_F32 && dtype != K2AMD_F64)) return K2AMD_ERR_INVALID_ARGUMENT;
  // scratch only where the pipelined kernels will take the shape: what the exact kernels serve
  // (no rows or no columns, tensors of 2 GiB and more) needs none and is never refused for it
  const bool pipelined = !ForceGeneric() && B > 0 &&
                         (dtype == K2AMD_F32 ? MiFastSupports(B, S, T, modified ? 1 : 0) : MiWaveSupports(B, S, T));
  const size_t need = pipelined ? k2amd_mi_workspace_bytes(B, S, T, modified, dtype) : 0;
  if (need > kScratchBytes) return K2AMD_ERR_SCRATCH_LIMIT;
  // set-up (also for B == 0, so that a caller can have it done ahead of its first real call)
  void *ws = ScratchOfCurrentDevice();
  if (ws == nullptr) return K2AMD_ERR_LAUNCH;
  if (B == 0) return K2AMD_OK;
  if (need > 0) {
    // The array keeps what the last call on this device left in it, whichever stream and shape
    // that was, and a launch that gave up a wait leaves words behind: every call starts by
    // putting the part it uses back into the initial state (a fill kernel, stream-ordered in
    // front of the recursion).
    const int status = MiFastWorkspaceInit(ws, need, static_cast<hipStream_t>(stream));
    if (status != K2AMD_OK) return status;
  }
  return k2amd_mi_forward_keep(px, py, boundary, p, ans, nullptr, B, S, T, modified, dtype,
                               need > 0 ? ws : nullptr, need, stream);
}

int k2amd_mi_noalloc_status(void *stream) {
  void *ws = ScratchOfCurrentDevice();
  if (ws == nullptr) return K2AMD_ERR_LAUNCH;
  return k2amd_mi_workspace_status(ws, stream);
}

int k2amd_mi_backward(const void *px, const void *py, const int64_t *boundary, const void *p,
                      void *ans_grad, void *px_grad, void *py_grad, int B, int S, int T,
                      int modified, int dtype, int overwrite_ans_grad, void *workspace,
                      size_t workspace_bytes, void *stream) {
  return k2amd_mi_backward_kept(px, py, boundary, p, nullptr, ans_grad, px_grad, py_grad, B, S, T,
                                modified, dtype, overwrite_ans_grad, workspace, workspace_bytes,
                                stream);
}

int k2amd_mi_backward_kept(const void *px, const void *py, const int64_t *boundary, const void *p,
                           const void *log_deriv, void *ans_grad, void *px_grad, void *py_grad,
                           int B, int S, int T, int modified, int dtype, int overwrite_ans_grad,
                           void *workspace, size_t workspace_bytes, void *stream) {
  (void)py;
  if (!ShapeOk(B, S, T) || (dtype != K2AMD_F32 && dtype != K2AMD_F64)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0) return K2AMD_OK;
  if (!ans_grad || (!px && S > 0) || (!px_grad && S > 0) || (!py_grad && T > 0))
    return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  modified = modified ? 1 : 0;
  const bool fast = dtype == K2AMD_F32 && workspace != nullptr && !ForceGeneric() && MiFastSupports(B, S, T, modified);
  if (!p && !(fast && log_deriv)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (fast) {
    if (workspace_bytes < MiFastWorkspaceBytes(B, S, T)) return K2AMD_ERR_WORKSPACE;
    return MiBackwardFast((const float *)px, (const float *)p, (const float *)log_deriv, boundary,
                          (float *)ans_grad,
                          (float *)px_grad, (float *)py_grad, B, S, T, modified,
                          overwrite_ans_grad, workspace, workspace_bytes, st);
  }
  if (dtype == K2AMD_F32)
    return MiBackwardGeneric<float>((const float *)px, (const float *)p, boundary,
                                    (float *)ans_grad, (float *)px_grad, (float *)py_grad, B, S, T,
                                    modified, overwrite_ans_grad, st);
  if (dtype == K2AMD_F64 && workspace != nullptr && !ForceGeneric() && MiWaveSupports(B, S, T)) {
    if (workspace_bytes < MiWaveWorkspaceBytes(B, S, T)) return K2AMD_ERR_WORKSPACE;
    return MiBackwardWave((const double *)px, (const double *)p, boundary, (double *)ans_grad,
                          (double *)px_grad, (double *)py_grad, B, S, T, modified, overwrite_ans_grad,
                          workspace, workspace_bytes, st);
  }
  return MiBackwardGeneric<double>((const double *)px, (const double *)p, boundary,
                                   (double *)ans_grad, (double *)px_grad, (double *)py_grad, B, S,
                                   T, modified, overwrite_ans_grad, st);
}

int k2amd_mi_forward_backward_supported(int B, int S, int T, int modified, int dtype,
                                        int has_workspace) {
  return dtype == K2AMD_F32 && has_workspace && ShapeOk(B, S, T) && B > 0 && !ForceGeneric() &&
         !PathIs("two-launches") && MiFusedSupports(B, S, T, modified ? 1 : 0);
}

int k2amd_mi_forward_backward_advised(int B, int S, int T, int modified, int dtype,
                                      int has_workspace) {
  return k2amd_mi_forward_backward_supported(B, S, T, modified, dtype, has_workspace) &&
         (MiFusedAdvised(B, S, T) || PathIs("single-launch"));
}

size_t k2amd_mi_forward_backward_scratch_bytes(int B, int S, int T, int modified, int dtype) {
  if (!k2amd_mi_forward_backward_supported(B, S, T, modified, dtype, 1)) return 0;
  return MiFusedScratchElems(B, S, T, modified ? 1 : 0) * sizeof(float);
}

int k2amd_mi_forward_backward(const void *px, const void *py, const int64_t *boundary, void *ans,
                              void *scratch, size_t scratch_bytes, void *ans_grad, void *px_grad,
                              void *py_grad, int B, int S, int T, int modified, int dtype,
                              int overwrite_ans_grad, void *workspace, size_t workspace_bytes,
                              void *stream) {
  if (!ShapeOk(B, S, T) || (dtype != K2AMD_F32 && dtype != K2AMD_F64)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0) return K2AMD_OK;
  if (!ans || !scratch || (!px && S > 0) || (!py && T > 0) || (!px_grad && S > 0) ||
      (!py_grad && T > 0))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (!k2amd_mi_forward_backward_supported(B, S, T, modified, dtype, workspace != nullptr))
    return K2AMD_ERR_UNSUPPORTED;
  if (workspace_bytes < MiFastWorkspaceBytes(B, S, T) ||
      scratch_bytes < k2amd_mi_forward_backward_scratch_bytes(B, S, T, modified, dtype))
    return K2AMD_ERR_WORKSPACE;
  return MiForwardBackwardFast((const float *)px, (const float *)py, boundary, (float *)ans,
                               (float *)scratch, (float *)ans_grad, (float *)px_grad,
                               (float *)py_grad, B, S, T, modified ? 1 : 0, overwrite_ans_grad,
                               workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

}  // extern "C"
