// Robust log-domain kernels for the mutual-information recursion (fp32 and fp64).
//
// One workgroup owns one sequence and sweeps its lattice one wavefront step at a time (the sweeps
// themselves are the device functions of mi_generic_impl.h).  Arithmetic follows k2's CPU loops
// term for term, so these kernels are the exact-semantics path: every dtype, every size, every
// -inf / NaN corner.
// They are latency-bound by design; the throughput path for fp32 lives in mi_fast.hip.
//
// The sweep keeps the previous step's values in two LDS rows of S + 2 elements.  A sequence with
// more rows than 64 KiB of LDS hold (S > 8190 in fp32, 4094 in fp64) is swept by the same
// kernels without those rows (kRowsInLds = false): the previous step is read back from what the
// workgroup itself stored in p, px_grad and py_grad, with the same bits as a result.
// K2AMD_MI_GENERIC_ROWS=global selects that form for every shape (tests and comparisons).
#include <cstdlib>
#include <cstring>

#include "common.h"
#include "mi_generic_impl.h"
#include "mi_internal.h"

namespace k2amd {
namespace {

constexpr int kThreads = 256;

template <typename T, bool kRowsInLds>
__global__ __launch_bounds__(kThreads) void MiForwardGenericKernel(
    const T *__restrict__ px, const T *__restrict__ py, const int64_t *__restrict__ boundary,
    T *__restrict__ p, T *__restrict__ ans, int S, int Tn, int modified) {
  HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
  const int b = blockIdx.x;
  const Box box = LoadBox(boundary, b, S, Tn);
  if (!box.ok) {
    if (threadIdx.x == 0) ans[b] = std::numeric_limits<T>::quiet_NaN();
    return;
  }
  T end;
  if (kRowsInLds) {
    T *prev = reinterpret_cast<T *>(smem_raw);
    T *cur = prev + (S + 2);
    end = MiForwardGenericSeq<T>(px, py, box, p, b, S, Tn, modified, Tn + 1, prev, cur);
  } else {
    end = MiForwardRowsFromP<T>(px, py, box, p, b, S, Tn, modified, Tn + 1);
  }
  if (threadIdx.x == 0) ans[b] = end;
}

template <typename T, bool kRowsInLds>
__global__ __launch_bounds__(kThreads) void MiBackwardGenericKernel(
    const T *__restrict__ px, const T *__restrict__ p, const int64_t *__restrict__ boundary,
    T *__restrict__ ans_grad, T *__restrict__ px_grad, T *__restrict__ py_grad, int S, int Tn,
    int modified, int overwrite_ans_grad) {
  HIP_DYNAMIC_SHARED(unsigned char, smem_raw)
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
  T at_origin;
  if (kRowsInLds) {
    T *gprev = reinterpret_cast<T *>(smem_raw);
    T *gcur = gprev + (S + 2);
    at_origin = MiBackwardGenericSeq<T>(px, p, box, ans_grad[b], px_grad, py_grad, b, S, Tn,
                                        modified, Tn + 1, gprev, gcur);
  } else {
    at_origin = MiBackwardRowsFromGrads<T>(px, p, box, ans_grad[b], px_grad, py_grad, b, S, Tn,
                                           modified, Tn + 1);
  }
  if (overwrite_ans_grad && threadIdx.x == 0) ans_grad[b] = at_origin;
}

constexpr size_t kLdsRowsLimit = 64 * 1024;

// Whether a sequence's two rows go to LDS: they have to fit, and the switch must not say otherwise.
bool RowsInLds(size_t smem) {
  if (smem > kLdsRowsLimit) return false;
  const char *e = std::getenv("K2AMD_MI_GENERIC_ROWS");
  return !(e != nullptr && std::strcmp(e, "global") == 0);
}

}  // namespace

template <typename T>
int MiForwardGeneric(const T *px, const T *py, const int64_t *boundary, T *p, T *ans, int B,
                     int S, int Tn, int modified, hipStream_t stream) {
  const size_t smem = 2 * (size_t)(S + 2) * sizeof(T);
  if (RowsInLds(smem))
    hipLaunchKernelGGL((MiForwardGenericKernel<T, true>), dim3(B), dim3(kThreads), smem, stream, px,
                       py, boundary, p, ans, S, Tn, modified);
  else
    hipLaunchKernelGGL((MiForwardGenericKernel<T, false>), dim3(B), dim3(kThreads), 0, stream, px,
                       py, boundary, p, ans, S, Tn, modified);
  return LaunchStatus();
}

template <typename T>
int MiBackwardGeneric(const T *px, const T *p, const int64_t *boundary, T *ans_grad, T *px_grad,
                      T *py_grad, int B, int S, int Tn, int modified, int overwrite_ans_grad,
                      hipStream_t stream) {
  const size_t smem = 2 * (size_t)(S + 2) * sizeof(T);
  if (RowsInLds(smem))
    hipLaunchKernelGGL((MiBackwardGenericKernel<T, true>), dim3(B), dim3(kThreads), smem, stream, px,
                       p, boundary, ans_grad, px_grad, py_grad, S, Tn, modified, overwrite_ans_grad);
  else
    hipLaunchKernelGGL((MiBackwardGenericKernel<T, false>), dim3(B), dim3(kThreads), 0, stream, px,
                       p, boundary, ans_grad, px_grad, py_grad, S, Tn, modified, overwrite_ans_grad);
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
