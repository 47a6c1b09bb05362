// C entry points, for the host build of the kernels, to the exact mutual-information kernels by
// themselves: k2amd_mi_forward / k2amd_mi_backward (mi_capi.hip) choose between them and the
// pipelined kernels, and the tests also want the exact ones where the library would not take them.
#include "common.h"
#include "mi_internal.h"

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
