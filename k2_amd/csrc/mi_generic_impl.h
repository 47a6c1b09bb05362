// Device functions of the exact log-domain recursion: one workgroup sweeps one sequence's lattice
// a wavefront step at a time,
//   regular lattice : step k holds the anti-diagonal  s + t = k   (cell (s,t) needs (s-1,t), (s,t-1))
//   modified lattice: step k holds the column         t = k       (cell (s,t) needs (s-1,t-1), (s,t-1))
// so a step depends on the previous step only, which lives in two rotating rows of S + 2 values
// that the caller provides (LDS).  Arithmetic follows k2's CPU loops term for term
// (k2/python/csrc/torch/mutual_information_cpu.cu:89-121 forward, :179-251 backward).  Used by the
// kernels of mi_generic.hip (every dtype, every -inf / NaN corner) and, for the sequences whose
// end cell no path reaches, by the single launch of mi_fast.hip.
//
// For sequences with more rows than LDS holds there is a second pair (MiForwardRowsFromP,
// MiBackwardRowsFromGrads) that keeps no rows at all: the previous step's values are what the
// workgroup itself stored in p (forward) or in px_grad / py_grad (backward: a cell's gradient is
// the sum of the two it sent on) one barrier earlier.  Same operands, same operations, same bits.
#ifndef K2_AMD_CSRC_MI_GENERIC_IMPL_H_
#define K2_AMD_CSRC_MI_GENERIC_IMPL_H_

#include "common.h"

namespace k2amd {

// Forward sweep of sequence b by the calling workgroup (all of its threads); p has rows of
// p_stride values.  Returns p[s_end][t_end] (to every thread).  The box must be valid.
template <typename T>
__device__ __forceinline__ T MiForwardGenericSeq(const T *__restrict__ px, const T *__restrict__ py,
                                                 const Box &box, T *__restrict__ p, int b, int S, int Tn,
                                                 int modified, int p_stride, T *prev, T *cur) {
  const int nthreads = blockDim.x;
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const int skew = modified ? 0 : 1;
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const T *pxb = px + (size_t)b * S * T1;
  const T *pyb = py + (size_t)b * (S + 1) * Tn;
  T *pb = p + (size_t)b * (S + 1) * p_stride;
  const int K = nt + ns * skew;
  for (int k = 0; k <= K; ++k) {
    for (int i = threadIdx.x; i <= ns; i += nthreads) {
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
      pb[(size_t)s * p_stride + t] = v;
    }
    __syncthreads();
    T *tmp = prev; prev = cur; cur = tmp;
  }
  return prev[ns];
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

// Backward sweep of sequence b by the calling workgroup, seeded with `seed` at the end cell;
// assigns px_grad / py_grad inside the box (what lies outside is the caller's to clear).
// Returns the gradient that reached the origin (to every thread).  The box must be valid.
template <typename T>
__device__ __forceinline__ T MiBackwardGenericSeq(const T *__restrict__ px, const T *__restrict__ p,
                                                  const Box &box, T seed, T *__restrict__ px_grad,
                                                  T *__restrict__ py_grad, int b, int S, int Tn,
                                                  int modified, int p_stride, T *gprev, T *gcur) {
  const int nthreads = blockDim.x;
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const int skew = modified ? 0 : 1;
  const T *pxb = px + (size_t)b * S * T1;
  const T *pb = p + (size_t)b * (S + 1) * p_stride;
  T *gx = px_grad + (size_t)b * S * T1;
  T *gy = py_grad + (size_t)b * (S + 1) * Tn;
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const int K = nt + ns * skew;
  for (int k = K; k >= 0; --k) {
    for (int i = threadIdx.x; i <= ns; i += nthreads) {
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
          const T d1 = PxDeriv<T>(pb[(size_t)s * p_stride + t] + pxb[(size_t)s * T1 + t],
                                  pb[(size_t)(s + 1) * p_stride + t - off], &ok);
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
              PxDeriv<T>(pb[(size_t)(s - 1) * p_stride + t + 1 + off] +
                             pxb[(size_t)(s - 1) * T1 + t + 1 + off],
                         pb[(size_t)s * p_stride + t + 1], &ok);
          c = ok ? (T(1) - d1) * gd : T(0);
        }
        gy[(size_t)s * Tn + t] = c;
      }
      gcur[i] = (i == ns && j == nt) ? seed : a + c;
    }
    __syncthreads();
    T *tmp = gprev; gprev = gcur; gcur = tmp;
  }
  return gprev[0];
}

// MiForwardGenericSeq without the two rows: the previous step is read back from p, which the
// workgroup wrote before the barrier that ended that step.  p must not alias px or py.
template <typename T>
__device__ __forceinline__ T MiForwardRowsFromP(const T *__restrict__ px, const T *__restrict__ py,
                                                const Box &box, T *p, int b, int S, int Tn,
                                                int modified, int p_stride) {
  const int nthreads = blockDim.x;
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const int skew = modified ? 0 : 1;
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const T *pxb = px + (size_t)b * S * T1;
  const T *pyb = py + (size_t)b * (S + 1) * Tn;
  T *pb = p + (size_t)b * (S + 1) * p_stride;
  const int K = nt + ns * skew;
  for (int k = 0; k <= K; ++k) {
    for (int i = threadIdx.x; i <= ns; i += nthreads) {
      const int j = k - i * skew;
      if (j < 0 || j > nt) continue;
      const int s = box.s0 + i, t = box.t0 + j;
      T v;
      if (i == 0) {
        v = (j == 0) ? T(0) : pb[(size_t)s * p_stride + t - 1] + pyb[(size_t)s * Tn + t - 1];
      } else if (j == 0) {
        v = modified ? Real<T>::NegInf()
                     : pb[(size_t)(s - 1) * p_stride + t] + pxb[(size_t)(s - 1) * T1 + t];
      } else {
        v = LogAdd<T>(pb[(size_t)(s - 1) * p_stride + t + off] + pxb[(size_t)(s - 1) * T1 + t + off],
                      pb[(size_t)s * p_stride + t - 1] + pyb[(size_t)s * Tn + t - 1]);
      }
      pb[(size_t)s * p_stride + t] = v;
    }
    __syncthreads();
  }
  return pb[(size_t)box.s1 * p_stride + box.t1];
}

// MiBackwardGenericSeq without the two rows: the gradient of a cell of the previous step is
// rebuilt as the sum of the px_grad and py_grad elements that the workgroup stored for it before
// the barrier that ended that step (the end cell's is the seed).  px_grad and py_grad must not
// alias px or p.
template <typename T>
__device__ __forceinline__ T MiBackwardRowsFromGrads(const T *__restrict__ px, const T *__restrict__ p,
                                                     const Box &box, T seed, T *px_grad, T *py_grad,
                                                     int b, int S, int Tn, int modified, int p_stride) {
  const int nthreads = blockDim.x;
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const int skew = modified ? 0 : 1;
  const T *pxb = px + (size_t)b * S * T1;
  const T *pb = p + (size_t)b * (S + 1) * p_stride;
  T *gx = px_grad + (size_t)b * S * T1;
  T *gy = py_grad + (size_t)b * (S + 1) * Tn;
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const int K = nt + ns * skew;
  // what MiBackwardGenericSeq keeps in gcur[i2] for cell (i2, j2)
  auto cell_grad = [&](int i2, int j2) -> T {
    if (i2 == ns && j2 == nt) return seed;
    const int s2 = box.s0 + i2, t2 = box.t0 + j2;
    T a = 0, c = 0;
    if (i2 < ns && j2 - off <= nt) a = gx[(size_t)s2 * T1 + t2];
    if (j2 < nt) c = gy[(size_t)s2 * Tn + t2];
    return a + c;
  };
  for (int k = K; k >= 0; --k) {
    for (int i = threadIdx.x; i <= ns; i += nthreads) {
      const int j = k - i * skew;
      if (j < 0 || j > nt) continue;
      const int s = box.s0 + i, t = box.t0 + j;
      const int jd = j - off;
      if (i < ns && jd <= nt) {
        const T gd = cell_grad(i + 1, jd);
        T a;
        if (jd == 0) {
          a = gd;
        } else {
          bool ok;
          const T d1 = PxDeriv<T>(pb[(size_t)s * p_stride + t] + pxb[(size_t)s * T1 + t],
                                  pb[(size_t)(s + 1) * p_stride + t - off], &ok);
          a = ok ? d1 * gd : T(0);
        }
        gx[(size_t)s * T1 + t] = a;
      }
      if (j < nt) {
        const T gd = cell_grad(i, j + 1);
        T c;
        if (i == 0) {
          c = gd;
        } else {
          bool ok;
          const T d1 =
              PxDeriv<T>(pb[(size_t)(s - 1) * p_stride + t + 1 + off] +
                             pxb[(size_t)(s - 1) * T1 + t + 1 + off],
                         pb[(size_t)s * p_stride + t + 1], &ok);
          c = ok ? (T(1) - d1) * gd : T(0);
        }
        gy[(size_t)s * Tn + t] = c;
      }
    }
    __syncthreads();
  }
  return cell_grad(0, 0);
}

}  // namespace k2amd

#endif  // K2_AMD_CSRC_MI_GENERIC_IMPL_H_
