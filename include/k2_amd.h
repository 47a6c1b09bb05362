/*
 * C-ABI of libk2amd.so: the MI355X (gfx950) implementation of k2's RNN-T
 * mutual-information path.  Plain pointers and sizes only; every pointer is a
 * DEVICE pointer unless stated otherwise; tensors are dense row-major with the
 * last axis contiguous.  Every function returns K2AMD_OK (0) or a K2AMD_ERR_*
 * code and never throws; launches are asynchronous on `stream` (a hipStream_t,
 * NULL = the default stream).  No function synchronises the device.
 *
 * Each declaration cites the reference interface it replaces.
 */
#ifndef K2_AMD_H_
#define K2_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define K2AMD_VERSION 100
#define K2AMD_API __attribute__((visibility("default")))

enum k2amd_status {
  K2AMD_OK = 0,
  K2AMD_ERR_INVALID_ARGUMENT = 1, /* bad shape / null pointer / unknown enum */
  K2AMD_ERR_UNSUPPORTED = 2,      /* valid request this build cannot serve (size limit) */
  K2AMD_ERR_WORKSPACE = 3,        /* workspace missing or too small */
  K2AMD_ERR_LAUNCH = 4            /* HIP reported a launch error */
};

enum k2amd_dtype { K2AMD_F32 = 0, K2AMD_F64 = 1 };

/* rnnt_type of k2/python/k2/rnnt_loss.py:70 ("regular" | "modified" | "constrained") */
enum k2amd_rnnt_type { K2AMD_REGULAR = 0, K2AMD_MODIFIED = 1, K2AMD_CONSTRAINED = 2 };

K2AMD_API int k2amd_version(void);
K2AMD_API const char *k2amd_status_string(int status);

/* ------------------------------------------------------------------ MI recursion
 *
 * Shapes (k2/python/csrc/torch/mutual_information.h:30-79):
 *   px [B][S][T1]  with T1 = T (modified != 0) or T+1 (modified == 0)
 *   py [B][S+1][T]
 *   p  [B][S+1][T+1]   written inside each sequence's boundary box only
 *   boundary [B][4] int64 = (s_begin, t_begin, s_end, t_end) or NULL for (0,0,S,T)
 *   ans, ans_grad [B]
 *
 * Workspace: k2amd_mi_workspace_bytes() tells how many bytes of device scratch the
 * forward/backward kernels want for the given shape (may be 0).  The caller owns it.
 */
K2AMD_API size_t k2amd_mi_workspace_bytes(int B, int S, int T, int modified, int dtype);

/* Replaces _k2.mutual_information_forward (k2/python/csrc/torch/mutual_information.cu:26-44,
 * CPU semantics of k2/python/csrc/torch/mutual_information_cpu.cu:50-124):
 *   p[b,s_begin,t_begin] = 0
 *   p[b,s,t] = log_add(p[b,s-1,t+o] + px[b,s-1,t+o], p[b,s,t-1] + py[b,s,t-1]),  o = modified ? -1 : 0
 *   ans[b] = p[b,s_end,t_end]                                                                     */
K2AMD_API int k2amd_mi_forward(const void *px, const void *py, const int64_t *boundary, void *p, void *ans,
                     int B, int S, int T, int modified, int dtype, void *workspace,
                     size_t workspace_bytes, void *stream);

/* Replaces _k2.mutual_information_backward (k2/python/csrc/torch/mutual_information.cu:46-67,
 * semantics of k2/python/csrc/torch/mutual_information_cpu.cu:128-255).  Writes EVERY element of
 * px_grad [B][S][T1] and py_grad [B][S+1][T] (zeros outside the boundary box).  If
 * overwrite_ans_grad != 0, ans_grad[b] is replaced by the gradient that reached
 * p[b,s_begin,t_begin], which equals the incoming ans_grad[b] when the recursion is consistent
 * (k2/python/csrc/torch/mutual_information_cuda.cu:661-663).                                     */
K2AMD_API int k2amd_mi_backward(const void *px, const void *py, const int64_t *boundary, const void *p,
                      void *ans_grad, void *px_grad, void *py_grad, int B, int S, int T,
                      int modified, int dtype, int overwrite_ans_grad, void *workspace,
                      size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* K2_AMD_H_ */
