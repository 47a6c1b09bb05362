// Robust log-domain kernels for the mutual-information recursion (fp32 and fp64).
//
// One workgroup owns one sequence and sweeps its lattice one wavefront step at a time (the sweeps
// themselves are the device functions of mi_generic_impl.h).  Arithmetic follows k2's CPU loops
// term for term, so these kernels are the exact-semantics path: every dtype, every size, every
// -inf / NaN corner.
// They are latency-bound by design; the throughput path for fp32 lives in mi_fast.hip.
#include "common.h"
#include "mi_generic_impl.h"
#include "mi_internal.h"

namespace k2amd {
namespace {

constexpr int kThreads = 256;

template <typename T>
__global__ __launch_bounds__(kThreads) void MiForwardGenericKernel(
    const T *__restrict__ px, const T *__restrict__ py, const int64_t *__restrict__ boundary,
    T *__restrict__ p, T *__restrict__ ans, int S, int Tn, int modified) {
  HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
  T *prev = reinterpret_cast<T *>(smem_raw);
  T *cur = prev + (S + 2);
  const int b = blockIdx.x;
  const Box box = LoadBox(boundary, b, S, Tn);
  if (!box.ok) {
    if (threadIdx.x == 0) ans[b] = std::numeric_limits<T>::quiet_NaN();
    return;
  }
  const T end = MiForwardGenericSeq<T>(px, py, box, p, b, S, Tn, modified, Tn + 1, prev, cur);
  if (threadIdx.x == 0) ans[b] = end;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void MiBackwardGenericKernel(
    const T *__restrict__ px, const T *__restrict__ p, const int64_t *__restrict__ boundary,
    T *__restrict__ ans_grad, T *__restrict__ px_grad, T *__restrict__ py_grad, int S, int Tn,
    int modified, int overwrite_ans_grad) {
  HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
  T *gprev = reinterpret_cast<T *>(smem_raw);
  T *gcur = gprev + (S + 2);
  const int b = blockIdx.x;
  const Box box = LoadBox(boundary, b, S, Tn);
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  T *gx = px_grad + (size_t)b * S * T1;
  T *gy = py_grad + (size_t)b * (S + 1) * Tn;

  // Elements outside the region the sweep assigns are zero, as with the zero-filled buffers
  // the reference allocates when a boundary is given
  // (k2/python/csrc/torch/mutual_information_cpu.cu:160-166).
  {
    const int xs0 = box.ok ? box.s0 : 0, xs1 = box.ok ? box.s1 : 0;            // rows [s0, s1)
    const int xt0 = box.ok ? box.t0 : 0, xt1 = box.ok ? box.t1 + off + 1 : 0;  // cols [t0, t1+off]
    for (int idx = threadIdx.x; idx < S * T1; idx += kThreads) {
      const int s = idx / T1, t = idx - s * T1;
      if (!(s >= xs0 && s < xs1 && t >= xt0 && t < xt1)) gx[idx] = T(0);
    }
    const int ys0 = box.ok ? box.s0 : 0, ys1 = box.ok ? box.s1 + 1 : 0;  // rows [s0, s1]
    const int yt0 = box.ok ? box.t0 : 0, yt1 = box.ok ? box.t1 : 0;      // cols [t0, t1)
    for (int idx = threadIdx.x; idx < (S + 1) * Tn; idx += kThreads) {
      const int s = idx / Tn, t = idx - s * Tn;
      if (!(s >= ys0 && s < ys1 && t >= yt0 && t < yt1)) gy[idx] = T(0);
    }
  }
  if (!box.ok) return;
  const T at_origin = MiBackwardGenericSeq<T>(px, p, box, ans_grad[b], px_grad, py_grad, b, S, Tn,
                                              modified, Tn + 1, gprev, gcur);
  if (overwrite_ans_grad && threadIdx.x == 0) ans_grad[b] = at_origin;
}

}  // namespace

size_t MiGenericMaxRows(int dtype) {
  // two rotating LDS rows of S+2 values must fit the 64 KiB a workgroup may ask for
  const size_t elem = dtype == K2AMD_F64 ? 8 : 4;
  return (64 * 1024) / (2 * elem) - 2;
}

template <typename T>
int MiForwardGeneric(const T *px, const T *py, const int64_t *boundary, T *p, T *ans, int B,
                     int S, int Tn, int modified, hipStream_t stream) {
  const size_t smem = 2 * (size_t)(S + 2) * sizeof(T);
  if (smem > 64 * 1024) return K2AMD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(MiForwardGenericKernel<T>, dim3(B), dim3(kThreads), smem, stream, px, py,
                     boundary, p, ans, S, Tn, modified);
  return LaunchStatus();
}

template <typename T>
int MiBackwardGeneric(const T *px, const T *p, const int64_t *boundary, T *ans_grad, T *px_grad,
                      T *py_grad, int B, int S, int Tn, int modified, int overwrite_ans_grad,
                      hipStream_t stream) {
  const size_t smem = 2 * (size_t)(S + 2) * sizeof(T);
  if (smem > 64 * 1024) return K2AMD_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(MiBackwardGenericKernel<T>, dim3(B), dim3(kThreads), smem, stream, px, p,
                     boundary, ans_grad, px_grad, py_grad, S, Tn, modified, overwrite_ans_grad);
  return LaunchStatus();
}

template int MiForwardGeneric<float>(const float *, const float *, const int64_t *, float *,
                                     float *, int, int, int, int, hipStream_t);
template int MiForwardGeneric<double>(const double *, const double *, const int64_t *, double *,
                                      double *, int, int, int, int, hipStream_t);
template int MiBackwardGeneric<float>(const float *, const float *, const int64_t *, float *,
                                      float *, float *, int, int, int, int, int, hipStream_t);
template int MiBackwardGeneric<double>(const double *, const double *, const int64_t *, double *,
                                       double *, double *, int, int, int, int, int, hipStream_t);

}  // namespace k2amd
