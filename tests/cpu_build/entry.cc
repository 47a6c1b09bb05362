// C entry points, for the host build of the kernels, to the exact mutual-information kernels,
// which the GPU library reaches through k2amd_mi_forward / k2amd_mi_backward (mi_capi.hip; that
// file also dispatches to the kernels that need the hardware and is not part of the host build).
#include "common.h"
#include "mi_internal.h"

// The host build has mi_capi.hip itself (argument checks and kernel selection) but none of the
// kernels that need the hardware: their launchers say "not served", as they do on the GPU for a
// shape outside their range, and every call then takes the exact kernels of mi_generic.hip.
namespace k2amd {
bool MiFastSupports(int, int, int, int) { return false; }
size_t MiFastWorkspaceBytes(int, int, int) { return 0; }
// (the fp64 wave kernels ARE part of the host build and share the fp32 kernels' workspace layout:
// a header of 64 words, zero, then words that hold the sentinel while nothing is published)
int MiFastWorkspaceInit(void *workspace, size_t workspace_bytes, hipStream_t) {
  if (workspace == nullptr || workspace_bytes < 256) return K2AMD_ERR_WORKSPACE;
  unsigned *words = static_cast<unsigned *>(workspace);
  for (size_t i = 0; i < 64; ++i) words[i] = 0;
  for (size_t i = 64; i < workspace_bytes / 4; ++i) words[i] = 0x7fc5a5a5u;
  return K2AMD_OK;
}
int MiForwardFast(const float *, const float *, const int64_t *, float *, float *, float *, int, int, int, int,
                  void *, size_t, hipStream_t) { return K2AMD_ERR_UNSUPPORTED; }
int MiBackwardFast(const float *, const float *, const float *, const int64_t *, float *, float *, float *, int,
                   int, int, int, int, void *, size_t, hipStream_t) { return K2AMD_ERR_UNSUPPORTED; }
bool MiFusedSupports(int, int, int, int) { return false; }
bool MiFusedAdvised(int, int, int) { return false; }
size_t MiFusedScratchElems(int, int, int, int) { return 0; }
int MiForwardBackwardFast(const float *, const float *, const int64_t *, float *, float *, float *, float *,
                          float *, int, int, int, int, int, void *, size_t, hipStream_t) {
  return K2AMD_ERR_UNSUPPORTED;
}
}  // namespace k2amd

extern "C" {

int cpu_mi_forward_generic(const void *px, const void *py, const int64_t *boundary, void *p, void *ans, int B,
                           int S, int T, int modified, int dtype) {
  if (dtype == K2AMD_F32)
    return k2amd::MiForwardGeneric<float>((const float *)px, (const float *)py, boundary, (float *)p, (float *)ans,
                                          B, S, T, modified, nullptr);
  return k2amd::MiForwardGeneric<double>((const double *)px, (const double *)py, boundary, (double *)p,
                                         (double *)ans, B, S, T, modified, nullptr);
}

int cpu_mi_backward_generic(const void *px, const void *p, const int64_t *boundary, void *ans_grad, void *px_grad,
                            void *py_grad, int B, int S, int T, int modified, int overwrite_ans_grad, int dtype) {
  if (dtype == K2AMD_F32)
    return k2amd::MiBackwardGeneric<float>((const float *)px, (const float *)p, boundary, (float *)ans_grad,
                                           (float *)px_grad, (float *)py_grad, B, S, T, modified,
                                           overwrite_ans_grad, nullptr);
  return k2amd::MiBackwardGeneric<double>((const double *)px, (const double *)p, boundary, (double *)ans_grad,
                                          (double *)px_grad, (double *)py_grad, B, S, T, modified,
                                          overwrite_ans_grad, nullptr);
}

}  // extern "C"
