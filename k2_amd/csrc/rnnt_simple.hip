// get_rnnt_logprobs for the "simple" joiner (am + lm), forward and backward
// (k2/python/k2/rnnt_loss.py:65-225).
//
// Forward:  row maxima + exponentials of am and lm (one wavefront per row), then a batched
// [S+1 x C] * [C x T] product on the vector ALUs (LDS-tiled 64x64, the north star rules out MFMA
// for this 0.2 GFLOP contraction) whose epilogue takes the log, adds the maxima back and emits
// px / py directly, so the normaliser never makes a round trip through HBM as a separate tensor
// apart from the `denom` buffer kept for the backward.
// Backward: Q = (dpx + dpy) / denom, two more batched products (Q * am_probs, Q^T * lm_probs)
// scaled by the saved exponentials, plus the gathered symbol / termination terms.
#include "common.h"

namespace k2amd {
namespace {

template <typename T>
__device__ __forceinline__ T WaveMaxS(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, kWave));
  return v;
}
template <typename T>
__device__ __forceinline__ T WaveSumS(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// probs[row][c] = exp(x[row][c] - max_c x[row][c]); one wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void RowMaxExpKernel(const T *__restrict__ x,
                                                       T *__restrict__ probs,
                                                       T *__restrict__ row_max, long long rows,
                                                       int C) {
  const int lane = threadIdx.x & (kWave - 1);
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T *xr = x + (size_t)row * C;
  T m = Real<T>::NegInf();
  for (int c = lane; c < C; c += kWave) m = max(m, xr[c]);
  m = WaveMaxS(m);
  if (lane == 0) row_max[row] = m;
  T *pr = probs + (size_t)row * C;
  for (int c = lane; c < C; c += kWave) pr[c] = Real<T>::Exp(xr[c] - m);
}

// ---- batched product  acc[b][m][n] = sum_k A[b](m,k) * Bm[b](k,n)  with element strides --------
struct MatView {
  size_t batch;  // elements between consecutive b
  int row, col;  // strides of the (m or k) and (k or n) index
};

constexpr int kTile = 64, kTileK = 16, kPad = 4;

template <typename T, typename Epilogue>
__global__ __launch_bounds__(256) void BatchedProductKernel(const T *__restrict__ A, MatView av,
                                                            const T *__restrict__ Bm, MatView bv,
                                                            int M, int N, int K, Epilogue epi) {
  __shared__ T As[kTileK][kTile + kPad];
  __shared__ T Bs[kTileK][kTile + kPad];
  const int b = blockIdx.z;
  const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  const T *Ab = A + (size_t)b * av.batch;
  const T *Bb = Bm + (size_t)b * bv.batch;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 x 16 threads, 4 x 4 outputs each
  T acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0;
  const bool a_k_fast = av.col == 1;  // A(m,k): k contiguous
  const bool b_k_fast = bv.row == 1;  // B(k,n): k contiguous
  for (int k0 = 0; k0 < K; k0 += kTileK) {
    for (int idx = threadIdx.x; idx < kTile * kTileK; idx += 256) {
      int mm, kk;
      if (a_k_fast) { kk = idx % kTileK; mm = idx / kTileK; } else { mm = idx % kTile; kk = idx / kTile; }
      const int m = m0 + mm, k = k0 + kk;
      As[kk][mm] = (m < M && k < K) ? Ab[(size_t)m * av.row + (size_t)k * av.col] : T(0);
      int nn, k2;
      if (b_k_fast) { k2 = idx % kTileK; nn = idx / kTileK; } else { nn = idx % kTile; k2 = idx / kTile; }
      const int n = n0 + nn, kb = k0 + k2;
      Bs[k2][nn] = (n < N && kb < K) ? Bb[(size_t)kb * bv.row + (size_t)n * bv.col] : T(0);
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTileK; ++kk) {
      T a[4], bb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bb[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * bb[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < M && n < N) epi(b, m, n, acc[i][j]);
    }
}

template <typename T>
struct Tiny;
template <>
struct Tiny<float> { static constexpr float v = 1.17549435e-38f; };   // torch.finfo(float32).tiny
template <>
struct Tiny<double> { static constexpr double v = 2.2250738585072014e-308; };

// Forward epilogue: (m, n) = (s, t).
template <typename T>
struct ForwardEpilogue {
  const T *lm, *am, *lm_max, *am_max;
  const int64_t *symbols, *boundary;
  T *px, *py, *denom;
  int S, Tn, C, blank, rnnt_type;
  __device__ void operator()(int b, int s, int t, T acc) const {
    const T d = acc + Tiny<T>::v;
    denom[((size_t)b * (S + 1) + s) * Tn + t] = d;
    const T norm = (Real<T>::Log(d) + lm_max[(size_t)b * (S + 1) + s]) + am_max[(size_t)b * Tn + t];
    const T *lmr = lm + ((size_t)b * (S + 1) + s) * C;
    const T *amr = am + ((size_t)b * Tn + t) * C;
    py[((size_t)b * (S + 1) + s) * Tn + t] = (amr[blank] + lmr[blank]) - norm;
    if (s < S) {
      const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
      const int64_t sym = symbols[(size_t)b * S + s];
      T v = (sym >= 0 && sym < C) ? (amr[sym] + lmr[sym]) - norm : Real<T>::NegInf();
      if (rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t)
        v = Real<T>::NegInf();
      px[((size_t)b * S + s) * T1 + t] = v;
    }
  }
};

// Backward epilogue: out[b][m][n] = -scale[b][m][n] * acc  (scale = the saved exponentials).
template <typename T>
struct ScaleEpilogue {
  const T *scale;
  T *out;
  int M, N;
  __device__ void operator()(int b, int m, int n, T acc) const {
    const size_t i = ((size_t)b * M + m) * N + n;
    out[i] = -scale[i] * acc;
  }
};

template <typename T>
__global__ void ZeroKernelS(T *__restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = T(0);
}

template <typename T>
__global__ void LastColumnKernelS(T *__restrict__ px, int rows, int T1) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) px[(size_t)i * T1 + (T1 - 1)] = Real<T>::NegInf();
}

template <typename T>
__global__ void ConstrainedKernelS(T *__restrict__ px, const T *__restrict__ py, int B, int S,
                                   int Tn) {
  const size_t n = (size_t)B * S * Tn;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t b = i / ((size_t)S * Tn), rem = i - b * (size_t)S * Tn;
    px[i] += py[b * (size_t)(S + 1) * Tn + Tn + rem];
  }
}

// Effective gradients of the un-fixed px / py values at (b,s,t), t < T.
template <typename T>
struct GradView {
  const T *px_grad, *py_grad;
  const int64_t *boundary;
  int S, Tn, rnnt_type;
  __device__ __forceinline__ T Gx(int b, int s, int t) const {
    if (s >= S) return 0;
    if (rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t) return 0;
    const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
    return px_grad[((size_t)b * S + s) * T1 + t];
  }
  __device__ __forceinline__ T Gy(int b, int s, int t) const {
    T g = py_grad[((size_t)b * (S + 1) + s) * Tn + t];
    if (rnnt_type == K2AMD_CONSTRAINED && s >= 1) g += Gx(b, s - 1, t);
    return g;
  }
};

template <typename T>
__global__ void QKernel(GradView<T> gv, const T *__restrict__ denom, T *__restrict__ q, int B) {
  const size_t n = (size_t)B * (gv.S + 1) * gv.Tn;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const int t = (int)(i % gv.Tn);
    const int s = (int)((i / gv.Tn) % (gv.S + 1));
    const int b = (int)(i / ((size_t)gv.Tn * (gv.S + 1)));
    q[i] = (gv.Gx(b, s, t) + gv.Gy(b, s, t)) / denom[i];
  }
}

// lm_grad[b,s,sym[b,s]] += sum_t Gx; lm_grad[b,s,blank] += sum_t Gy.  One wavefront per (b,s).
template <typename T>
__global__ __launch_bounds__(256) void LmGatherTermsKernel(GradView<T> gv,
                                                           const int64_t *__restrict__ symbols,
                                                           T *__restrict__ lm_grad, int B, int C,
                                                           int blank) {
  const int lane = threadIdx.x & (kWave - 1);
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= B * (gv.S + 1)) return;
  const int b = row / (gv.S + 1), s = row - b * (gv.S + 1);
  T sx = 0, sy = 0;
  for (int t = lane; t < gv.Tn; t += kWave) {
    sx += gv.Gx(b, s, t);
    sy += gv.Gy(b, s, t);
  }
  sx = WaveSumS(sx);
  sy = WaveSumS(sy);
  if (lane == 0) {
    T *g = lm_grad + (size_t)row * C;
    if (s < gv.S) {
      const int64_t sym = symbols[(size_t)b * gv.S + s];
      if (sym >= 0 && sym < C) g[sym] += sx;
    }
    g[blank] += sy;
  }
}

// am_grad[b,t,sym[b,s]] += Gx(b,s,t) for every s (in order, so repeated symbols add
// deterministically); am_grad[b,t,blank] += sum_s Gy.  One thread per (b,t).
template <typename T>
__global__ void AmGatherTermsKernel(GradView<T> gv, const int64_t *__restrict__ symbols,
                                    T *__restrict__ am_grad, int B, int C, int blank) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= B * gv.Tn) return;
  const int b = i / gv.Tn, t = i - b * gv.Tn;
  T *g = am_grad + (size_t)i * C;
  T sy = 0;
  for (int s = 0; s <= gv.S; ++s) {
    if (s < gv.S) {
      const int64_t sym = symbols[(size_t)b * gv.S + s];
      if (sym >= 0 && sym < C) g[sym] += gv.Gx(b, s, t);
    }
    sy += gv.Gy(b, s, t);
  }
  g[blank] += sy;
}

template <typename T>
int SimpleForward(const T *lm, const T *am, const int64_t *symbols, const int64_t *boundary, T *px,
                  T *py, T *lm_probs, T *am_probs, T *lm_max, T *am_max, T *denom, int B, int S,
                  int Tn, int C, int blank, int rnnt_type, hipStream_t st) {
  const long long lm_rows = (long long)B * (S + 1), am_rows = (long long)B * Tn;
  if (lm_rows > 0)
    hipLaunchKernelGGL(RowMaxExpKernel<T>, dim3((unsigned)((lm_rows + 3) / 4)), dim3(256), 0, st, lm, lm_probs, lm_max, lm_rows, C);
  if (am_rows > 0)
    hipLaunchKernelGGL(RowMaxExpKernel<T>, dim3((unsigned)((am_rows + 3) / 4)), dim3(256), 0, st, am, am_probs, am_max, am_rows, C);
  const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
  if (rnnt_type == K2AMD_REGULAR && B * S > 0)
    hipLaunchKernelGGL(LastColumnKernelS<T>, dim3((B * S + 255) / 256), dim3(256), 0, st, px, B * S, T1);
  if (B > 0 && Tn > 0) {
    ForwardEpilogue<T> epi{lm, am, lm_max, am_max, symbols, boundary, px, py, denom, S, Tn, C, blank, rnnt_type};
    MatView av{(size_t)(S + 1) * C, C, 1};  // A(m=s, k=c) = lm_probs[b][s][c]
    MatView bv{(size_t)Tn * C, 1, C};       // B(k=c, n=t) = am_probs[b][t][c]
    dim3 grid((Tn + kTile - 1) / kTile, (S + 1 + kTile - 1) / kTile, B);
    hipLaunchKernelGGL((BatchedProductKernel<T, ForwardEpilogue<T>>), grid, dim3(256), 0, st, lm_probs, av, am_probs, bv, S + 1, Tn, C, epi);
    if (rnnt_type == K2AMD_CONSTRAINED && S > 0)
      hipLaunchKernelGGL(ConstrainedKernelS<T>, dim3(512), dim3(256), 0, st, px, py, B, S, Tn);
  }
  return LaunchStatus();
}

template <typename T>
int SimpleBackward(const T *px_grad, const T *py_grad, const int64_t *symbols,
                   const int64_t *boundary, const T *lm_probs, const T *am_probs, const T *denom,
                   T *lm_grad, T *am_grad, T *q, int B, int S, int Tn, int C, int blank,
                   int rnnt_type, hipStream_t st) {
  if (B == 0) return K2AMD_OK;
  GradView<T> gv{px_grad, py_grad, boundary, S, Tn, rnnt_type};
  if (Tn > 0) {
    hipLaunchKernelGGL(QKernel<T>, dim3(512), dim3(256), 0, st, gv, denom, q, B);
    {  // lm_grad[b][s][c] = -lm_probs * sum_t q[b][s][t] * am_probs[b][t][c]
      ScaleEpilogue<T> epi{lm_probs, lm_grad, S + 1, C};
      MatView av{(size_t)(S + 1) * Tn, Tn, 1};  // A(m=s, k=t) = q[b][s][t]
      MatView bv{(size_t)Tn * C, C, 1};         // B(k=t, n=c) = am_probs[b][t][c]
      dim3 grid((C + kTile - 1) / kTile, (S + 1 + kTile - 1) / kTile, B);
      hipLaunchKernelGGL((BatchedProductKernel<T, ScaleEpilogue<T>>), grid, dim3(256), 0, st, q, av, am_probs, bv, S + 1, C, Tn, epi);
    }
    {  // am_grad[b][t][c] = -am_probs * sum_s q[b][s][t] * lm_probs[b][s][c]
      ScaleEpilogue<T> epi{am_probs, am_grad, Tn, C};
      MatView av{(size_t)(S + 1) * Tn, 1, Tn};   // A(m=t, k=s) = q[b][s][t]
      MatView bv{(size_t)(S + 1) * C, C, 1};     // B(k=s, n=c) = lm_probs[b][s][c]
      dim3 grid((C + kTile - 1) / kTile, (Tn + kTile - 1) / kTile, B);
      hipLaunchKernelGGL((BatchedProductKernel<T, ScaleEpilogue<T>>), grid, dim3(256), 0, st, q, av, lm_probs, bv, Tn, C, S + 1, epi);
    }
    hipLaunchKernelGGL(AmGatherTermsKernel<T>, dim3((B * Tn + 255) / 256), dim3(256), 0, st, gv, symbols, am_grad, B, C, blank);
  } else {
    hipLaunchKernelGGL(ZeroKernelS<T>, dim3(256), dim3(256), 0, st, lm_grad, (size_t)B * (S + 1) * C);
  }
  hipLaunchKernelGGL(LmGatherTermsKernel<T>, dim3((B * (S + 1) + 3) / 4), dim3(256), 0, st, gv, symbols, lm_grad, B, C, blank);
  return LaunchStatus();
}

bool ArgsOk(int B, int S, int T, int C, int blank, int rnnt_type, int dtype) {
  if (B < 0 || S < 0 || T < 0 || C <= 0 || blank < 0 || blank >= C) return false;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return false;
  if (B > 65535) return false;  // grid.z
  return dtype == K2AMD_F32 || dtype == K2AMD_F64;
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

int k2amd_rnnt_logprobs_simple_forward(const void *lm, const void *am, const int64_t *symbols,
                                       const int64_t *boundary, void *px, void *py, void *lm_probs,
                                       void *am_probs, void *lm_max, void *am_max, void *denom,
                                       int B, int S, int T, int C, int termination_symbol,
                                       int rnnt_type, int dtype, void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SimpleForward<float>((const float *)lm, (const float *)am, symbols, boundary, (float *)px, (float *)py, (float *)lm_probs, (float *)am_probs, (float *)lm_max, (float *)am_max, (float *)denom, B, S, T, C, termination_symbol, rnnt_type, st);
  return SimpleForward<double>((const double *)lm, (const double *)am, symbols, boundary, (double *)px, (double *)py, (double *)lm_probs, (double *)am_probs, (double *)lm_max, (double *)am_max, (double *)denom, B, S, T, C, termination_symbol, rnnt_type, st);
}

int k2amd_rnnt_logprobs_simple_backward(const void *px_grad, const void *py_grad,
                                        const int64_t *symbols, const int64_t *boundary,
                                        const void *lm_probs, const void *am_probs,
                                        const void *denom, void *lm_grad, void *am_grad,
                                        void *q_scratch, int B, int S, int T, int C,
                                        int termination_symbol, int rnnt_type, int dtype,
                                        void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SimpleBackward<float>((const float *)px_grad, (const float *)py_grad, symbols, boundary, (const float *)lm_probs, (const float *)am_probs, (const float *)denom, (float *)lm_grad, (float *)am_grad, (float *)q_scratch, B, S, T, C, termination_symbol, rnnt_type, st);
  return SimpleBackward<double>((const double *)px_grad, (const double *)py_grad, symbols, boundary, (const double *)lm_probs, (const double *)am_probs, (const double *)denom, (double *)lm_grad, (double *)am_grad, (double *)q_scratch, B, S, T, C, termination_symbol, rnnt_type, st);
}

}  // extern "C"
