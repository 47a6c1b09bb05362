// The split of a joint score over the N inputs of joint_mutual_information_recursion
// (k2/python/k2/mutual_information.py:404-417):
//   prods[n][b] = sum_k px_grad[b][k] * clamp(px_n[b][k]) + sum_k py_grad[b][k] * clamp(py_n[b][k]),
// clamp(v) = max(v, lowest finite value): an input of -inf carries no occupation, and 0 * -inf
// would be NaN.  The reference forms it with torch ops over stacked copies of the inputs (stack,
// clamp, product, sum: five passes over N tensors); here every tensor is read once.
#include "common.h"

#include <limits>

namespace k2amd {
namespace {

constexpr int kJointMax = 8;      // inputs per call
constexpr int kJointChunks = 32;  // workgroups per (input, sequence)

struct JointInputs {
  const void *x[kJointMax];
  const void *y[kJointMax];
};

template <typename T>
__device__ __forceinline__ T ClampedDot(const T *__restrict__ grad, const T *__restrict__ v,
                                        long long begin, long long end) {
  const T lowest = std::numeric_limits<T>::lowest();
  T acc = 0;
  for (long long i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const T value = v[i];
    acc += grad[i] * (value < lowest ? lowest : value);  // (a NaN stays a NaN, as with torch.clamp)
  }
  return acc;
}

// partial[(n B + b) kJointChunks + chunk] = the chunk's share of prods[n][b].  The sums are added
// in a fixed order (a thread's elements, the lanes of a wavefront, the wavefronts, then the
// chunks in JointFinishKernel): the result does not depend on scheduling.
template <typename T>
__global__ __launch_bounds__(256) void JointPartialKernel(JointInputs in, const T *__restrict__ px_grad,
                                                          const T *__restrict__ py_grad,
                                                          T *__restrict__ partial, int B,
                                                          long long kx, long long ky) {
  __shared__ T sums[4];
  const int b = blockIdx.x / kJointChunks, chunk = blockIdx.x - b * kJointChunks, n = blockIdx.y;
  const long long lx = (kx + kJointChunks - 1) / kJointChunks, ly = (ky + kJointChunks - 1) / kJointChunks;
  const long long x0 = min((long long)chunk * lx, kx), x1 = min(x0 + lx, kx);
  const long long y0 = min((long long)chunk * ly, ky), y1 = min(y0 + ly, ky);
  T acc = ClampedDot(px_grad + (size_t)b * kx, static_cast<const T *>(in.x[n]) + (size_t)b * kx, x0, x1);
  acc += ClampedDot(py_grad + (size_t)b * ky, static_cast<const T *>(in.y[n]) + (size_t)b * ky, y0, y1);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) sums[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0)
    partial[((size_t)n * B + b) * kJointChunks + chunk] = (sums[0] + sums[1]) + (sums[2] + sums[3]);
}

template <typename T>
__global__ void JointFinishKernel(const T *__restrict__ partial, T *__restrict__ prods, int count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  T sum = 0;
  for (int c = 0; c < kJointChunks; ++c) sum += partial[(size_t)i * kJointChunks + c];
  prods[i] = sum;
}

template <typename T>
int JointProducts(const JointInputs &in, int N, const T *px_grad, const T *py_grad, T *prods,
                  T *partial, int B, long long kx, long long ky, hipStream_t st) {
  hipLaunchKernelGGL(JointPartialKernel<T>, dim3((unsigned)B * kJointChunks, N), dim3(256), 0, st, in, px_grad,
                     py_grad, partial, B, kx, ky);
  hipLaunchKernelGGL(JointFinishKernel<T>, dim3((N * B + 255) / 256), dim3(256), 0, st, partial, prods, N * B);
  return LaunchStatus();
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

size_t k2amd_mi_joint_products_scratch_elements(int N, int B) {
  return N > 0 && B > 0 ? (size_t)N * B * kJointChunks : 0;
}

int k2amd_mi_joint_products(const void *const *px, const void *const *py, int N, const void *px_grad,
                            const void *py_grad, void *prods, void *partial, int B, long long kx,
                            long long ky, int dtype, void *stream) {
  if (N < 1 || B < 0 || kx < 0 || ky < 0 || px == nullptr || py == nullptr) return K2AMD_ERR_INVALID_ARGUMENT;
  if (dtype != K2AMD_F32 && dtype != K2AMD_F64) return K2AMD_ERR_INVALID_ARGUMENT;
  if (N > kJointMax || (long long)N * B >= (1ll << 31) / kJointChunks) return K2AMD_ERR_UNSUPPORTED;
  if (B == 0) return K2AMD_OK;
  JointInputs in{};
  for (int n = 0; n < N; ++n) {
    in.x[n] = px[n];
    in.y[n] = py[n];
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return JointProducts<float>(in, N, (const float *)px_grad, (const float *)py_grad, (float *)prods, (float *)partial, B, kx, ky, st);
  return JointProducts<double>(in, N, (const double *)px_grad, (const double *)py_grad, (double *)prods, (double *)partial, B, kx, ky, st);
}

}  // extern "C"
