// Robust log-domain kernels for the mutual-information recursion (fp32 and fp64).
//
// One workgroup owns one sequence and sweeps its lattice one wavefront step at a time:
//   regular lattice : step k holds the anti-diagonal  s + t = k   (cell (s,t) needs (s-1,t), (s,t-1))
//   modified lattice: step k holds the column         t = k       (cell (s,t) needs (s-1,t-1), (s,t-1))
// so in both cases a step depends on the previous step only, which lives in LDS (two rotating
// rows of S+1 values).  Arithmetic follows k2's CPU loops term for term
// (k2/python/csrc/torch/mutual_information_cpu.cu:89-121 forward, :179-251 backward), so these
// kernels are the exact-semantics path: every dtype, every size, every -inf / NaN corner.
// They are latency-bound by design; the throughput path for fp32 lives in mi_fast.hip.
#include "common.h"
#include "mi_internal.h"

namespace k2amd {
namespace {

constexpr int kThreads = 256;

template <typename T>
__global__ __launch_bounds__(kThreads) void MiForwardGenericKernel(
    const T *__restrict__ px, const T *__restrict__ py, const int64_t *__restrict__ boundary,
    T *__restrict__ p, T *__restrict__ ans, int S, int Tn, int modified) {
  extern __shared__ unsigned char smem_raw[];
  T *prev = reinterpret_cast<T *>(smem_raw);
  T *cur = prev + (S + 2);
  const int b = blockIdx.x;
  const Box box = LoadBox(boundary, b, S, Tn);
  if (!box.ok) {
    if (threadIdx.x == 0) ans[b] = std::numeric_limits<T>::quiet_NaN();
    return;
  }
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const int skew = modified ? 0 : 1;
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const T *pxb = px + (size_t)b * S * T1;
  const T *pyb = py + (size_t)b * (S + 1) * Tn;
  T *pb = p + (size_t)b * (S + 1) * (Tn + 1);
  const int K = nt + ns * skew;
  for (int k = 0; k <= K; ++k) {
    for (int i = threadIdx.x; i <= ns; i += kThreads) {
      const int j = k - i * skew;
      if (j < 0 || j > nt) continue;
      const int s = box.s0 + i, t = box.t0 + j;
      T v;
      if (i == 0) {
        v = (j == 0) ? T(0) : prev[0] + pyb[(size_t)s * Tn + t - 1];
      } else if (j == 0) {
        v = modified ? Real<T>::NegInf() : prev[i - 1] + pxb[(size_t)(s - 1) * T1 + t];
      } else {
        v = LogAdd<T>(prev[i - 1] + pxb[(size_t)(s - 1) * T1 + t + off],
                      prev[i] + pyb[(size_t)s * Tn + t - 1]);
      }
      cur[i] = v;
      pb[(size_t)s * (Tn + 1) + t] = v;
    }
    __syncthreads();
    T *tmp = prev; prev = cur; cur = tmp;
  }
  if (threadIdx.x == 0) ans[b] = prev[ns];
}

// exp(term1 - total) with the reference's guards
// (k2/python/csrc/torch/mutual_information_cpu.cu:195-211): a non-finite total counts as 0;
// a non-finite derivative sends no gradient either way (ok = false).
template <typename T>
__device__ __forceinline__ T PxDeriv(T term1, T total, bool *ok) {
  if (total - total != 0) total = 0;
  T d = Real<T>::Exp(term1 - total);
  *ok = (d - d == 0);
  return d;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void MiBackwardGenericKernel(
    const T *__restrict__ px, const T *__restrict__ p, const int64_t *__restrict__ boundary,
    T *__restrict__ ans_grad, T *__restrict__ px_grad, T *__restrict__ py_grad, int S, int Tn,
    int modified, int overwrite_ans_grad) {
  extern __shared__ unsigned char smem_raw[];
  T *gprev = reinterpret_cast<T *>(smem_raw);
  T *gcur = gprev + (S + 2);
  const int b = blockIdx.x;
  const Box box = LoadBox(boundary, b, S, Tn);
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const int skew = modified ? 0 : 1;
  const T *pxb = px + (size_t)b * S * T1;
  const T *pb = p + (size_t)b * (S + 1) * (Tn + 1);
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

  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const int K = nt + ns * skew;
  const T seed = ans_grad[b];
  for (int k = K; k >= 0; --k) {
    for (int i = threadIdx.x; i <= ns; i += kThreads) {
      const int j = k - i * skew;
      if (j < 0 || j > nt) continue;
      const int s = box.s0 + i, t = box.t0 + j;
      T a = 0, c = 0;
      // Gradient arriving through px[s][t]: from cell (s+1, t-off).
      const int jd = j - off;
      if (i < ns && jd <= nt) {
        const T gd = gprev[i + 1];
        if (jd == 0) {
          a = gd;  // first column of a regular lattice: p[s+1][t0] = p[s][t0] + px[s][t0]
        } else {
          bool ok;
          const T d1 = PxDeriv<T>(pb[(size_t)s * (Tn + 1) + t] + pxb[(size_t)s * T1 + t],
                                  pb[(size_t)(s + 1) * (Tn + 1) + t - off], &ok);
          a = ok ? d1 * gd : T(0);
        }
        gx[(size_t)s * T1 + t] = a;
      }
      // Gradient arriving through py[s][t]: from cell (s, t+1).
      if (j < nt) {
        const T gd = gprev[i];
        if (i == 0) {
          c = gd;  // first row: p[s0][t+1] = p[s0][t] + py[s0][t]
        } else {
          bool ok;
          const T d1 =
              PxDeriv<T>(pb[(size_t)(s - 1) * (Tn + 1) + t + 1 + off] +
                             pxb[(size_t)(s - 1) * T1 + t + 1 + off],
                         pb[(size_t)s * (Tn + 1) + t + 1], &ok);
          c = ok ? (T(1) - d1) * gd : T(0);
        }
        gy[(size_t)s * Tn + t] = c;
      }
      gcur[i] = (i == ns && j == nt) ? seed : a + c;
    }
    __syncthreads();
    T *tmp = gprev; gprev = gcur; gcur = tmp;
  }
  if (overwrite_ans_grad && threadIdx.x == 0) ans_grad[b] = gprev[0];
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
