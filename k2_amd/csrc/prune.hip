// Pruning side of the RNN-T path: the integer prune ranges and the lm gather / scatter.
//   get_rnnt_prune_ranges  k2/python/k2/rnnt_loss.py:636-780
//   do_rnnt_pruning        k2/python/k2/rnnt_loss.py:913-954
#include "common.h"

namespace k2amd {
namespace {

constexpr int kPruneThreads = 256;

// Reverse running minimum of n ints held in LDS (Hillis-Steele on two rotating buffers).
// Returns the buffer that holds the result.  Every thread of the workgroup must call it.
__device__ int *SuffixMin(int *a, int *b, int n) {
  for (int off = 1; off < n; off <<= 1) {
    for (int t = threadIdx.x; t < n; t += kPruneThreads) {
      int v = a[t];
      if (t + off < n) v = min(v, a[t + off]);
      b[t] = v;
    }
    __syncthreads();
    int *tmp = a; a = b; b = tmp;
  }
  return a;
}

// One workgroup per sequence.  Frames are spread over the threads for the window search (reads
// of px_grad / py_grad are then contiguous along t), after which the two monotone passes of
// _adjust_pruning_lower_bound run as log-step scans in LDS.
//
// The window sum adds py_grad[b, s'+0 .. s'+R-1, t] first row to last in the input precision and
// subtracts px_grad[b, s'-1, t] afterwards (k2/python/k2/rnnt_loss.py:730-744); the arg-max keeps
// the first maximum (torch.argmax).
template <typename T>
__global__ __launch_bounds__(kPruneThreads) void PruneRangesKernel(
    const T *__restrict__ px_grad, const T *__restrict__ py_grad,
    const int64_t *__restrict__ boundary, int64_t *__restrict__ ranges, int S, int Tn,
    int modified, int R) {
  extern __shared__ int lds[];
  int *buf0 = lds, *buf1 = lds + Tn;
  const int b = blockIdx.x;
  const int T1 = modified ? Tn : Tn + 1;
  const int S1 = S + 1;
  const int n_win = S1 - R + 1;
  const T *gx = px_grad + (size_t)b * S * T1;
  const T *gy = py_grad + (size_t)b * S1 * Tn;
  const int64_t s_end = boundary[4 * b + 2], t_end = boundary[4 * b + 3];
  int64_t pad64 = s_end - R + 1;
  const int pad = pad64 < 0 ? 0 : (int)pad64;
  for (int t = threadIdx.x; t < Tn; t += kPruneThreads) {
    int best = 0;
    if (t < t_end - 1) {
      T best_v = 0;
      for (int w = 0; w < n_win; ++w) {
        T acc = gy[(size_t)w * Tn + t];
        for (int k = 1; k < R; ++k) acc = acc + gy[(size_t)(w + k) * Tn + t];
        const T v = acc - (w == 0 ? T(0) : gx[(size_t)(w - 1) * T1 + t]);
        if (w == 0 || v > best_v) { best_v = v; best = w; }
      }
    } else {
      best = pad;
    }
    buf0[t] = best;
  }
  __syncthreads();
  const int ramp = (modified ? 2 : R) - 1;
  int *cur = SuffixMin(buf0, buf1, Tn);
  int *other = cur == buf0 ? buf1 : buf0;
  for (int t = threadIdx.x; t < Tn; t += kPruneThreads) cur[t] = -(cur[t] - ramp * t);
  __syncthreads();
  cur = SuffixMin(cur, other, Tn);
  for (int t = threadIdx.x; t < Tn; t += kPruneThreads) {
    int v = cur[t];
    v = v < 0 ? 0 : v;
    const int64_t s_begin = -(int64_t)(v - ramp * t);
    int64_t *out = ranges + ((size_t)b * Tn + t) * R;
    for (int k = 0; k < R; ++k) out[k] = s_begin + k;
  }
}

template <typename T>
__global__ void GatherKernel(const T *__restrict__ lm, const int64_t *__restrict__ ranges,
                             T *__restrict__ out, int S1, int TR, int D, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / D;
    const int d = (int)(i - row * D);
    const size_t b = row / TR;
    const int64_t s = ranges[row];
    out[i] = (s >= 0 && s < S1) ? lm[(b * S1 + (size_t)s) * D + d] : T(0);
  }
}

template <typename T>
__global__ void ZeroKernel(T *__restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = T(0);
}

// Hardware floating-point atomics: several (t,k) of one sequence point at the same lm row.
template <typename T>
__global__ void ScatterAddKernel(const T *__restrict__ grad, const int64_t *__restrict__ ranges,
                                 T *__restrict__ lm_grad, int S1, int TR, int D, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / D;
    const int d = (int)(i - row * D);
    const size_t b = row / TR;
    const int64_t s = ranges[row];
    if (s >= 0 && s < S1) unsafeAtomicAdd(lm_grad + (b * S1 + (size_t)s) * D + d, grad[i]);
  }
}

unsigned GridFor(size_t n) {
  size_t blocks = (n + 255) / 256;
  return (unsigned)(blocks > 8192 ? 8192 : (blocks == 0 ? 1 : blocks));
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

int k2amd_rnnt_prune_ranges(const void *px_grad, const void *py_grad, const int64_t *boundary,
                            int64_t *ranges, int B, int S, int T, int modified, int s_range,
                            int dtype, void *stream) {
  if (B < 0 || S < 0 || T < 0 || s_range < 1 || s_range > S + 1 || !boundary ||
      (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0 || T == 0) return K2AMD_OK;
  const size_t smem = 2 * (size_t)T * sizeof(int);
  if (smem > 64 * 1024 || (long long)S * T >= (1ll << 31)) return K2AMD_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  modified = modified ? 1 : 0;
  if (dtype == K2AMD_F32)
    hipLaunchKernelGGL(PruneRangesKernel<float>, dim3(B), dim3(kPruneThreads), smem, st, (const float *)px_grad, (const float *)py_grad, boundary, ranges, S, T, modified, s_range);
  else
    hipLaunchKernelGGL(PruneRangesKernel<double>, dim3(B), dim3(kPruneThreads), smem, st, (const double *)px_grad, (const double *)py_grad, boundary, ranges, S, T, modified, s_range);
  return LaunchStatus();
}

int k2amd_rnnt_prune_gather(const void *lm, const int64_t *ranges, void *lm_pruned, int B, int S1,
                            int T, int R, int D, int dtype, void *stream) {
  if (B < 0 || S1 < 0 || T < 0 || R < 0 || D < 0 || (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  const size_t n = (size_t)B * T * R * D;
  if (n == 0) return K2AMD_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    hipLaunchKernelGGL(GatherKernel<float>, dim3(GridFor(n)), dim3(256), 0, st, (const float *)lm, ranges, (float *)lm_pruned, S1, T * R, D, n);
  else
    hipLaunchKernelGGL(GatherKernel<double>, dim3(GridFor(n)), dim3(256), 0, st, (const double *)lm, ranges, (double *)lm_pruned, S1, T * R, D, n);
  return LaunchStatus();
}

int k2amd_rnnt_prune_gather_backward(const void *grad, const int64_t *ranges, void *lm_grad, int B,
                                     int S1, int T, int R, int D, int dtype, void *stream) {
  if (B < 0 || S1 < 0 || T < 0 || R < 0 || D < 0 || (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t n_out = (size_t)B * S1 * D, n = (size_t)B * T * R * D;
  if (n_out == 0) return K2AMD_OK;
  if (dtype == K2AMD_F32) {
    hipLaunchKernelGGL(ZeroKernel<float>, dim3(GridFor(n_out)), dim3(256), 0, st, (float *)lm_grad, n_out);
    if (n) hipLaunchKernelGGL(ScatterAddKernel<float>, dim3(GridFor(n)), dim3(256), 0, st, (const float *)grad, ranges, (float *)lm_grad, S1, T * R, D, n);
  } else {
    hipLaunchKernelGGL(ZeroKernel<double>, dim3(GridFor(n_out)), dim3(256), 0, st, (double *)lm_grad, n_out);
    if (n) hipLaunchKernelGGL(ScatterAddKernel<double>, dim3(GridFor(n)), dim3(256), 0, st, (const double *)grad, ranges, (double *)lm_grad, S1, T * R, D, n);
  }
  return LaunchStatus();
}

}  // extern "C"
