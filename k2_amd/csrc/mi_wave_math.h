// exp and log(1 + exp(.)) in fp64 for the wave kernels of the mutual-information recursion:
// written out (range reduction + short polynomials, no table, no branch on the hot path) so that a
// recursion step does not pay for a general-purpose libm call.  Relative error against libm on
// 5e6 random arguments: exp 1e-14, log(1 + exp(d)) 4e-14 (d in [-37, 0]).
#ifndef K2_AMD_CSRC_MI_WAVE_MATH_H_
#define K2_AMD_CSRC_MI_WAVE_MATH_H_

#include <hip/hip_runtime.h>
#include <math.h>

namespace k2amd {

// A wavefront issues one instruction every few cycles whether or not it depends on the one before,
// so the polynomials are in Horner form (one multiply-add per coefficient, every coefficient an
// inline constant) rather than split for parallel evaluation.

// sum r^n / n!, n = 0 .. 11 (|r| <= 0.347: remainder 6e-15 relative)
__host__ __device__ __forceinline__ double ExpPoly(double r) {
  double q = 1.0 / 39916800;
  q = fma(q, r, 1.0 / 3628800);
  q = fma(q, r, 1.0 / 362880);
  q = fma(q, r, 1.0 / 40320);
  q = fma(q, r, 1.0 / 5040);
  q = fma(q, r, 1.0 / 720);
  q = fma(q, r, 1.0 / 120);
  q = fma(q, r, 1.0 / 24);
  q = fma(q, r, 1.0 / 6);
  q = fma(q, r, 0.5);
  q = fma(q, r, 1.0);
  return fma(q, r, 1.0);
}

// 2^k for k in [-1022, 1023], built in the exponent field
__host__ __device__ __forceinline__ double TwoTo(int k) {
  return __builtin_bit_cast(double, (unsigned long long)(1023 + k) << 52);
}

// exp(x) for x in [-700, 700]: k = round(x log2 e), r = x - k ln 2 (ln 2 in two pieces).
__host__ __device__ __forceinline__ double ExpInRange(double x) {
  const double k = rint(x * 1.4426950408889634074);
  double r = fma(k, -6.93147180369123816490e-01, x);
  r = fma(k, -1.90821492927058770002e-10, r);
  return ExpPoly(r) * TwoTo((int)k);
}

// exp(x) for any x (0 below the smallest normal number's logarithm, NaN for NaN).
__host__ __device__ __forceinline__ double FastExp(double x) {
  if (!(x > -708.0)) return x != x ? x : 0.0;
  if (x > 709.0) return INFINITY;
  return ExpInRange(x);
}

__host__ __device__ __forceinline__ float RcpF(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_rcpf(x);
#else
  return 1.0f / x;
#endif
}

// log(1 + exp(d)) for d in [-40, 0]: E = exp(d) in (0, 1]; u = 1 + E, halved when above sqrt 2;
// log u = 2 atanh(s) with s = (u - 1) / (u + 1), |s| <= 0.1716 (eight terms of the series: 3e-14).
__host__ __device__ __forceinline__ double Log1pExpNeg(double d) {
  const double E = ExpInRange(d);
  const bool big = E > 0.41421356237309503;  // u > sqrt 2: u / 2 - 1 = (E - 1) / 2, u / 2 + 1 = (E + 3) / 2
  const double num = big ? E - 1.0 : E, den = E + (big ? 3.0 : 2.0);
  const double add = big ? 6.93147180559945286227e-01 : 0.0;
  // s = num / den: a single-precision reciprocal (den in [2, 4]) and two Newton steps
  double rc = (double)RcpF((float)den);
  rc = rc * fma(-den, rc, 2.0);
  rc = rc * fma(-den, rc, 2.0);
  const double s = num * rc;
  const double z = s * s;
  double q = 1.0 / 15;
  q = fma(q, z, 1.0 / 13);
  q = fma(q, z, 1.0 / 11);
  q = fma(q, z, 1.0 / 9);
  q = fma(q, z, 1.0 / 7);
  q = fma(q, z, 1.0 / 5);
  q = fma(q, z, 1.0 / 3);
  q = fma(q, z, 1.0);
  return fma(s + s, q, add);
}

}  // namespace k2amd

#endif  // K2_AMD_CSRC_MI_WAVE_MATH_H_
