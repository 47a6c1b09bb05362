// Shared host/device helpers for the gfx950 kernels of libk2amd.so.
#ifndef K2_AMD_CSRC_COMMON_H_
#define K2_AMD_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <limits>

#include "../../include/k2_amd.h"

namespace k2amd {

// a * b rounded on its own: the empty asm statement hides the product from the compiler, which
// would otherwise fuse it into a following addition (contraction is on for HIP code, and the
// *_rn intrinsics do not stop it).  Used where a result has to equal what separate elementwise
// kernels would have produced.
template <typename T>
__device__ __forceinline__ T MulRounded(T a, T b) {
  T r = a * b;
  asm volatile("" : "+v"(r));
  return r;
}


constexpr int kWave = 64;  // CDNA wavefront width

// Turns the last HIP error into a status code without clearing sticky state of other streams.
inline int LaunchStatus() { return hipGetLastError() == hipSuccess ? K2AMD_OK : K2AMD_ERR_LAUNCH; }

template <typename T>
struct Real;

template <>
struct Real<float> {
  // logf(FLT_EPSILON): below this difference log_add returns its larger operand
  // (k2/csrc/utils.h:511).
  static constexpr float kMinLogDiff = -15.9423847198486328125f;
  static __device__ __forceinline__ float Exp(float x) { return expf(x); }
  static __device__ __forceinline__ float Log1p(float x) { return log1pf(x); }
  static __device__ __forceinline__ float Log(float x) { return logf(x); }
  static __host__ __device__ __forceinline__ float NegInf() {
    return -std::numeric_limits<float>::infinity();
  }
};

template <>
struct Real<double> {
  // log(DBL_EPSILON) (k2/csrc/utils.h:512-513).
  static constexpr double kMinLogDiff = -36.0436533891171535515240975655615329742431640625;
  static __device__ __forceinline__ double Exp(double x) { return exp(x); }
  static __device__ __forceinline__ double Log1p(double x) { return log1p(x); }
  static __device__ __forceinline__ double Log(double x) { return log(x); }
  static __host__ __device__ __forceinline__ double NegInf() {
    return -std::numeric_limits<double>::infinity();
  }
};

// log(exp(x) + exp(y)) with k2's cut-off (k2/csrc/utils.h:518-563): the larger operand is
// returned unchanged when the smaller one is below it by more than log(epsilon); a NaN
// difference (both operands -inf) also returns x.
template <typename T>
__device__ __forceinline__ T LogAdd(T x, T y) {
  T diff;
  if (x < y) {
    diff = x - y;
    x = y;
  } else {
    diff = y - x;
  }
  if (diff >= Real<T>::kMinLogDiff) return x + Real<T>::Log1p(Real<T>::Exp(diff));
  return x;
}

struct Box {
  int s0, t0, s1, t1;
  bool ok;
};

// Reads one row of the int64 boundary tensor (or the default box) and range-checks it
// against (S, T) so that a corrupt boundary can never drive an out-of-bounds access.
__device__ __forceinline__ Box LoadBox(const int64_t *boundary, int b, int S, int T) {
  Box x;
  if (boundary == nullptr) {
    x.s0 = 0; x.t0 = 0; x.s1 = S; x.t1 = T; x.ok = true;
    return x;
  }
  int64_t s0 = boundary[4 * b + 0], t0 = boundary[4 * b + 1], s1 = boundary[4 * b + 2],
          t1 = boundary[4 * b + 3];
  x.ok = (0 <= s0 && s0 <= s1 && s1 <= S && 0 <= t0 && t0 <= t1 && t1 <= T);
  x.s0 = (int)s0; x.t0 = (int)t0; x.s1 = (int)s1; x.t1 = (int)t1;
  return x;
}

}  // namespace k2amd

#endif  // K2_AMD_CSRC_COMMON_H_
