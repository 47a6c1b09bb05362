// Launchers shared between the translation units of the MI recursion.
#ifndef K2_AMD_CSRC_MI_INTERNAL_H_
#define K2_AMD_CSRC_MI_INTERNAL_H_

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace k2amd {

// Log-domain, one workgroup per sequence (mi_generic.hip).
template <typename T>
int MiForwardGeneric(const T *px, const T *py, const int64_t *boundary, T *p, T *ans, int B,
                     int S, int Tn, int modified, hipStream_t stream);
template <typename T>
int MiBackwardGeneric(const T *px, const T *p, const int64_t *boundary, T *ans_grad, T *px_grad,
                      T *py_grad, int B, int S, int Tn, int modified, int overwrite_ans_grad,
                      hipStream_t stream);

// fp32 throughput path: pipelined 63-row chunks, one chain wavefront per workgroup (mi_fast.hip).
bool MiFastSupports(int B, int S, int Tn, int modified);
size_t MiFastWorkspaceBytes(int B, int S, int Tn);
int MiFastWorkspaceInit(void *workspace, size_t workspace_bytes, hipStream_t stream);
// log_deriv (may be null): the forward also writes the logarithm of every cell's px-edge
// derivative there, laid out like p, and the backward given the same tensor reads it instead of
// p and px.
int MiForwardFast(const float *px, const float *py, const int64_t *boundary, float *p, float *ans,
                  float *log_deriv, int B, int S, int Tn, int modified, void *workspace,
                  size_t workspace_bytes, hipStream_t stream);
int MiBackwardFast(const float *px, const float *p, const float *log_deriv,
                   const int64_t *boundary, float *ans_grad, float *px_grad, float *py_grad, int B,
                   int S, int Tn, int modified, int overwrite_ans_grad, void *workspace,
                   size_t workspace_bytes, hipStream_t stream);

// Forward and backward in one launch; scratch holds MiFusedScratchElems floats (written, then
// read, by the launch itself).  MiFusedSupports: whether that kernel serves the shape.
bool MiFusedSupports(int B, int S, int Tn, int modified);
// Whether it is also the faster way on the current device (else: the two launches).
bool MiFusedAdvised(int B, int S, int Tn);
size_t MiFusedScratchElems(int B, int S, int Tn, int modified);
int MiForwardBackwardFast(const float *px, const float *py, const int64_t *boundary, float *ans,
                          float *scratch, float *ans_grad, float *px_grad, float *py_grad, int B,
                          int S, int Tn, int modified, int overwrite_ans_grad, void *workspace,
                          size_t workspace_bytes, hipStream_t stream);

// fp64 throughput path: pipelined 64-row chunks, one wavefront per chunk (mi_wave.hip); the
// workspace has the layout and the initial state of the fp32 one (MiFastWorkspaceInit).
bool MiWaveSupports(int B, int S, int Tn);
size_t MiWaveWorkspaceBytes(int B, int S, int Tn);
int MiForwardWave(const double *px, const double *py, const int64_t *boundary, double *p, double *ans,
                  int B, int S, int Tn, int modified, void *workspace, size_t workspace_bytes,
                  hipStream_t stream);
int MiBackwardWave(const double *px, const double *p, const int64_t *boundary, double *ans_grad,
                   double *px_grad, double *py_grad, int B, int S, int Tn, int modified,
                   int overwrite_ans_grad, void *workspace, size_t workspace_bytes, hipStream_t stream);

}  // namespace k2amd

#endif  // K2_AMD_CSRC_MI_INTERNAL_H_
