// Row-streaming kernels of the RNN-T log-prob builders that take joiner logits:
//   get_rnnt_logprobs_joint   logits [B][T][S+1][C]   (k2/python/k2/rnnt_loss.py:341-447)
//   get_rnnt_logprobs_pruned  logits [B][T][R][C]     (k2/python/k2/rnnt_loss.py:1180-1348)
//   get_hat_logprobs_pruned   logits [B][T][R][C]     (k2/python/k2/rnnt_loss.py:992-1177)
//
// Both are one streaming pass over the logits, one 64-lane wavefront per row of C logits held
// in registers (max and sum(exp) reduced across lanes), plus a small pass with one THREAD per
// row for the look-ups that decide which two log-probs a row contributes and where they go
// (ranges -> symbols -> logits: dependent round trips that a wavefront should pay for 64 rows
// at a time, not for one).  The backward mirrors it: a thread-per-row pass gathers each row's
// two incoming gradients, the streaming pass reads the row once and writes its gradient once.
// HBM traffic is the algorithmic minimum (logits read once forward; read once + written once
// backward).
#include "common.h"

namespace k2amd {
namespace {

constexpr int kRowsPerBlock = 4;  // one wavefront per row, 256 threads per workgroup
constexpr int kMaxRegs = 8;       // register-resident path covers C <= 64 * 8

template <typename T>
__device__ __forceinline__ T WaveMax(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, kWave));
  return v;
}
template <typename T>
__device__ __forceinline__ T WaveSum(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// 16-byte vectors of the element type, and the exponential used inside the row sums: the
// hardware exp2 path for fp32 (relative error ~1e-7, far inside the 1e-4 the loss is held to).
template <typename T> struct Vec16;
template <> struct Vec16<float> { typedef float4 type; static constexpr int kN = 4; };
template <> struct Vec16<double> { typedef double2 type; static constexpr int kN = 2; };
__device__ __forceinline__ float FastExp(float x) { return __expf(x); }
__device__ __forceinline__ double FastExp(double x) { return exp(x); }
__device__ __forceinline__ void Unpack(float4 v, float *o) { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
__device__ __forceinline__ void Unpack(double2 v, double *o) { o[0] = v.x; o[1] = v.y; }
__device__ __forceinline__ float4 Pack(const float *o) { return make_float4(o[0], o[1], o[2], o[3]); }
__device__ __forceinline__ double2 Pack(const double *o) { return make_double2(o[0], o[1]); }

constexpr int kMaxVecs = 4;  // vectors a lane keeps in registers: rows of up to 64 * 4 * 16 bytes

// Rows whose length is a multiple of the vector width start 16-byte aligned (the tensor does),
// so a lane reads them 16 bytes at a time.
template <typename T>
__device__ __forceinline__ bool RowIsVectorisable(int C) {
  return C % Vec16<T>::kN == 0 && C / Vec16<T>::kN <= kWave * kMaxVecs;
}

// logsumexp of one vectorisable row held in registers; same semantics as RowLogSumExp below
template <typename T>
__device__ __forceinline__ T RowLogSumExpVec(const T *__restrict__ x, int C, int lane,
                                             bool skip_first) {
  typedef typename Vec16<T>::type V;
  constexpr int kN = Vec16<T>::kN;
  const int nv = C / kN;
  const V *xv = reinterpret_cast<const V *>(x);
  T v[kMaxVecs][kN];
  T m = Real<T>::NegInf();
#pragma unroll
  for (int i = 0; i < kMaxVecs; ++i) {
    const int q = lane + i * kWave;
    if (q < nv) {
      Unpack(xv[q], v[i]);
    } else {
#pragma unroll
      for (int e = 0; e < kN; ++e) v[i][e] = Real<T>::NegInf();
    }
    if (i == 0 && skip_first && lane == 0) v[0][0] = Real<T>::NegInf();  // column 0 left out
#pragma unroll
    for (int e = 0; e < kN; ++e) m = max(m, v[i][e]);
  }
  m = WaveMax(m);
  if (m - m != 0) m = 0;  // +-inf (or NaN) maximum
  T sum = 0;
#pragma unroll
  for (int i = 0; i < kMaxVecs; ++i)
#pragma unroll
    for (int e = 0; e < kN; ++e) sum += FastExp(v[i][e] - m);
  sum = WaveSum(sum);
  return Real<T>::Log(sum) + m;
}

// logsumexp of one row, torch semantics (an infinite maximum is replaced by 0 before the
// subtraction, so an all -inf row yields -inf rather than NaN).
template <typename T>
__device__ __forceinline__ T RowLogSumExp(const T *__restrict__ x, int C, int lane,
                                          bool skip_first) {
  T m = Real<T>::NegInf();
  T sum = 0;
  const int first = skip_first ? 1 : 0;
  if (C <= kWave * kMaxRegs) {
    T v[kMaxRegs];
#pragma unroll
    for (int i = 0; i < kMaxRegs; ++i) {
      const int c = lane + i * kWave;
      v[i] = (c < C && c >= first) ? x[c] : Real<T>::NegInf();
      m = max(m, v[i]);
    }
    m = WaveMax(m);
    if (m - m != 0) m = 0;  // +-inf (or NaN) maximum
#pragma unroll
    for (int i = 0; i < kMaxRegs; ++i) sum += Real<T>::Exp(v[i] - m);
  } else {
    for (int c = lane + first; c < C; c += kWave) m = max(m, x[c]);
    m = WaveMax(m);
    if (m - m != 0) m = 0;
    for (int c = lane + first; c < C; c += kWave) sum += Real<T>::Exp(x[c] - m);
  }
  sum = WaveSum(sum);
  return Real<T>::Log(sum) + m;
}

struct RowGeom {
  int B, S, Tn, K, C;  // K rows per frame: S+1 (joint) or R (pruned)
  int blank, rnnt_type;
  int hat;  // 1: hybrid autoregressive transducer, column 0 is the blank and has its own sigmoid
};

// log sigmoid(x) = min(x, 0) - log1p(exp(-|x|)), and sigmoid(x) without overflow
template <typename T>
__device__ __forceinline__ T LogSigmoid(T x) {
  return min(x, T(0)) - Real<T>::Log1p(Real<T>::Exp(-fabs(x)));
}
template <typename T>
__device__ __forceinline__ T Sigmoid(T x) {
  const T e = Real<T>::Exp(-fabs(x));
  return (x >= 0 ? T(1) : e) / (T(1) + e);
}

// Maps row (b,t,k) to its lattice row s and to the symbol whose log-prob goes to px.
template <bool kPruned>
__device__ __forceinline__ void RowTarget(const RowGeom &g, const int64_t *__restrict__ symbols,
                                          const int64_t *__restrict__ ranges, int b, int t, int k,
                                          int *s, int *sym) {
  if (kPruned) {
    const int64_t *r = ranges + ((size_t)b * g.Tn + t) * g.K;
    int64_t shift = r[0], src = r[k];
    int S1 = g.S + 1;
    int ss = (int)((k + shift) % S1);
    if (ss < 0) ss += S1;
    *s = ss;
    // the symbol is looked up at ranges[b,t,k] in `symbols` extended by the termination symbol
    if (src >= 0 && src < g.S) *sym = (int)symbols[(size_t)b * g.S + src];
    else if (src == g.S) *sym = g.blank;
    else *sym = -1;
  } else {
    *s = k;
    *sym = k < g.S ? (int)symbols[(size_t)b * g.S + k] : -1;
  }
}

// Forward, pass 1: one wavefront per row streams the row and leaves its log-sum-exp in
// `normalizers`.  Nothing else: the look-ups that decide where a row's two log-probs go are a
// chain of dependent memory round trips, and paying that chain once per WAVEFRONT (one row)
// rather than once per LANE (64 rows, pass 2) cost a third of this kernel's time.
// The launch also carries the -inf fills that px / py need before pass 2 writes into them (work
// that is independent of the normalisers): workgroups past the first `norm_blocks` set
// a[i * stride_a] (i < na) and b[i] (i < nb) to -inf.  Pruned builder: all of px and py (everything
// outside the band stays -inf); joint builder, regular lattice: the column px[b,s,T]
// (k2/python/k2/rnnt_loss.py:193-205).
template <typename T>
struct NegInfFill {
  T *a, *b;
  size_t na, nb;
  int stride_a;
};

template <typename T>
__global__ __launch_bounds__(kRowsPerBlock *kWave) void RowNormKernel(
    const T *__restrict__ logits, T *__restrict__ normalizers, long long rows, int C,
    bool skip_first, unsigned norm_blocks, NegInfFill<T> fill) {
  if (blockIdx.x >= norm_blocks) {
    const size_t first = (size_t)(blockIdx.x - norm_blocks) * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)(gridDim.x - norm_blocks) * blockDim.x;
    for (size_t i = first; i < fill.na; i += stride) fill.a[i * fill.stride_a] = Real<T>::NegInf();
    for (size_t i = first; i < fill.nb; i += stride) fill.b[i] = Real<T>::NegInf();
    return;
  }
  const int lane = threadIdx.x & (kWave - 1);
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T *x = logits + (size_t)row * C;
  const T norm = RowIsVectorisable<T>(C) ? RowLogSumExpVec<T>(x, C, lane, skip_first)
                                         : RowLogSumExp<T>(x, C, lane, skip_first);
  if (lane == 0) normalizers[row] = norm;
}

// Forward, pass 2: one thread per row looks up where the row lands and writes
//   px[b,s,t] = logits[row, sym] - norm,   py[b,s,t] = logits[row, blank] - norm,
// or, for the hybrid autoregressive transducer (norm then covers columns 1..C-1 only),
//   py = log sigmoid(logits[row, 0]),  px = logits[row, sym] - norm + (py - logits[row, 0]).
template <typename T, bool kPruned>
__global__ void RowEmitKernel(const T *__restrict__ logits, const T *__restrict__ normalizers,
                              const int64_t *__restrict__ symbols, const int64_t *__restrict__ ranges,
                              const int64_t *__restrict__ boundary, T *__restrict__ px,
                              T *__restrict__ py, RowGeom g) {
  const long long rows = (long long)g.B * g.Tn * g.K;
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  const int k = (int)(row % g.K);
  const int t = (int)((row / g.K) % g.Tn);
  const int b = (int)(row / ((long long)g.K * g.Tn));
  const T *x = logits + (size_t)row * g.C;
  int s, sym;
  RowTarget<kPruned>(g, symbols, ranges, b, t, k, &s, &sym);
  const T norm = normalizers[row];
  const int T1 = g.rnnt_type == K2AMD_REGULAR ? g.Tn + 1 : g.Tn;
  T shift = 0, yv;
  if (g.hat) {
    const T x0 = x[0];
    yv = LogSigmoid(x0);
    shift = yv - x0;  // log(1 - sigmoid(x0))
  } else {
    yv = x[g.blank] - norm;
  }
  if (s < g.S) {
    T v = (sym >= 0 && sym < g.C) ? (x[sym] - norm) + shift : Real<T>::NegInf();
    if (g.rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t)
      v = Real<T>::NegInf();
    px[((size_t)b * g.S + s) * T1 + t] = v;
  }
  py[((size_t)b * (g.S + 1) + s) * g.Tn + t] = yv;
}

// px[b,s,t] += py[b,s+1,t] (k2/python/k2/rnnt_loss.py:222-223); T1 == Tn here.
template <typename T>
__global__ void ConstrainedKernel(T *__restrict__ px, const T *__restrict__ py, int B, int S,
                                  int Tn) {
  const size_t n = (size_t)B * S * Tn;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t b = i / ((size_t)S * Tn), rem = i - b * (size_t)S * Tn;
    px[i] += py[b * (size_t)(S + 1) * Tn + Tn + rem];
  }
}

// d loss / d logits[row, c] = -softmax(row)[c] * (gx + gy) + gx [c == sym] + gy [c == blank], with
// gx, gy the gradients that reach the row's px and py values.
//
// Backward, pass 1: one thread per row gathers what the row's gradient depends on (the look-up
// chain again, 64 rows per wavefront) and parks it in the first four elements of the row's own
// slot of logits_grad: {gx, gy, symbol, normaliser}.  Rows therefore need at least four columns.
template <typename T, bool kPruned>
__global__ void RowGradPrepKernel(const T *__restrict__ normalizers, const T *__restrict__ px_grad,
                                  const T *__restrict__ py_grad, const T *__restrict__ seq_scale,
                                  const int64_t *__restrict__ symbols,
                                  const int64_t *__restrict__ ranges,
                                  const int64_t *__restrict__ boundary, T *__restrict__ logits_grad,
                                  RowGeom g) {
  const long long rows = (long long)g.B * g.Tn * g.K;
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  const int k = (int)(row % g.K);
  const int t = (int)((row / g.K) % g.Tn);
  const int b = (int)(row / ((long long)g.K * g.Tn));
  int s, sym;
  RowTarget<kPruned>(g, symbols, ranges, b, t, k, &s, &sym);
  const int T1 = g.rnnt_type == K2AMD_REGULAR ? g.Tn + 1 : g.Tn;
  const T scale = seq_scale != nullptr ? seq_scale[b] : T(1);  // what reaches the sequence's score
  T gx = 0;
  if (s < g.S && sym >= 0 && sym < g.C) {
    const bool cut =
        g.rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t;
    if (!cut) gx = MulRounded(px_grad[((size_t)b * g.S + s) * T1 + t], scale);
  } else {
    sym = -1;
  }
  T gy = MulRounded(py_grad[((size_t)b * (g.S + 1) + s) * g.Tn + t], scale);
  if (g.rnnt_type == K2AMD_CONSTRAINED && s >= 1)
    gy += MulRounded(px_grad[((size_t)b * g.S + (s - 1)) * T1 + t], scale);  // px += py[:, 1:]
  T *rec = logits_grad + (size_t)row * g.C;
  rec[0] = gx;
  rec[1] = gy;
  rec[2] = (T)sym;  // exact: |sym| < 2^24
  rec[3] = normalizers[row];
}

// What one row's gradient is made of.  Softmax rows:
//   d/d logits[c] = -softmax[c] (gx + gy) + gx [c == sym] + gy [c == blank].
// Hybrid autoregressive transducer rows (norm covers columns 1..C-1, sg = sigmoid(logits[0])):
//   d/d logits[c >= 1] = gx ([c == sym] - exp(logits[c] - norm)),
//   d/d logits[0]      = gy (1 - sg) - gx sg + gx [sym == 0].
template <typename T, bool kHat>
struct RowGradTerms {
  T gx, gy, norm, sg;
  int sym, blank;
  template <bool kFast>
  __device__ __forceinline__ T At(T x, int c) const {
    const T p = kFast ? FastExp(x - norm) : Real<T>::Exp(x - norm);
    T v;
    if (kHat) {
      v = c == 0 ? gy * (T(1) - sg) - gx * sg : -p * gx;
    } else {
      v = -p * (gx + gy);
      if (c == blank) v += gy;
    }
    if (c == sym) v += gx;
    return v;
  }
};

// Backward, pass 2: one wavefront per row reads the row and its parked record, and writes the
// gradient over the whole slot (record included; every lane has read it by then).
template <typename T, bool kHat>
__global__ __launch_bounds__(kRowsPerBlock *kWave) void RowGradKernel(
    const T *__restrict__ logits, T *__restrict__ logits_grad, long long rows, int C, int blank) {
  const int lane = threadIdx.x & (kWave - 1);
  // Last row first: the forward pass read the rows in ascending order, so of a tensor larger than
  // the 256 MB memory-side cache it is the tail that is still there.
  const long long row = rows - 1 - ((long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6));
  if (row < 0) return;
  const T *x = logits + (size_t)row * C;
  T *dx = logits_grad + (size_t)row * C;
  typedef typename Vec16<T>::type V;
  constexpr int kN = Vec16<T>::kN;
  const bool vectorised = RowIsVectorisable<T>(C);
  const int nv = C / kN;
  V in[kMaxVecs];
  if (vectorised) {
    const V *xv = reinterpret_cast<const V *>(x);
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
      const int q = lane + i * kWave;
      if (q < nv) in[i] = xv[q];
    }
  }
  RowGradTerms<T, kHat> terms;
  terms.gx = dx[0];
  terms.gy = dx[1];
  terms.sym = (int)dx[2];
  terms.norm = dx[3];
  terms.blank = blank;
  terms.sg = kHat ? Sigmoid(x[0]) : T(0);
  // every lane has the record before any lane's store below overwrites it: a wavefront's lanes
  // run in lockstep, so this emits no instruction; it states the dependence
  __builtin_amdgcn_wave_barrier();
  if (vectorised) {
    V *dv = reinterpret_cast<V *>(dx);
    V outv[kMaxVecs];
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
      const int q = lane + i * kWave;
      if (q < nv) {
        T e[kN];
        Unpack(in[i], e);
#pragma unroll
        for (int k2 = 0; k2 < kN; ++k2) e[k2] = terms.template At<true>(e[k2], q * kN + k2);
        outv[i] = Pack(e);
      }
    }
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
      const int q = lane + i * kWave;
      if (q < nv) dv[q] = outv[i];
    }
    return;
  }
  // rows that are not read as vectors
  for (int c = lane; c < C; c += kWave) dx[c] = terms.template At<false>(x[c], c);
}

// The same in one pass, for rows too short to park a record in (C < 4).
template <typename T, bool kPruned, bool kHat>
__global__ __launch_bounds__(kRowsPerBlock *kWave) void RowBackwardKernel(
    const T *__restrict__ logits, const T *__restrict__ normalizers,
    const T *__restrict__ px_grad, const T *__restrict__ py_grad, const T *__restrict__ seq_scale,
    const int64_t *__restrict__ symbols, const int64_t *__restrict__ ranges,
    const int64_t *__restrict__ boundary, T *__restrict__ logits_grad, RowGeom g) {
  const int lane = threadIdx.x & (kWave - 1);
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  const long long rows = (long long)g.B * g.Tn * g.K;
  if (row >= rows) return;
  const int k = (int)(row % g.K);
  const int t = (int)((row / g.K) % g.Tn);
  const int b = (int)(row / ((long long)g.K * g.Tn));
  int s, sym;
  RowTarget<kPruned>(g, symbols, ranges, b, t, k, &s, &sym);
  const int T1 = g.rnnt_type == K2AMD_REGULAR ? g.Tn + 1 : g.Tn;
  // gradient reaching this row's px value and py value
  const T scale = seq_scale != nullptr ? seq_scale[b] : T(1);
  T gx = 0;
  if (s < g.S && sym >= 0 && sym < g.C) {
    const bool cut =
        g.rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t;
    if (!cut) gx = MulRounded(px_grad[((size_t)b * g.S + s) * T1 + t], scale);
  } else {
    sym = -1;
  }
  T gy = MulRounded(py_grad[((size_t)b * (g.S + 1) + s) * g.Tn + t], scale);
  if (g.rnnt_type == K2AMD_CONSTRAINED && s >= 1)
    gy += MulRounded(px_grad[((size_t)b * g.S + (s - 1)) * T1 + t], scale);  // px += py[:, 1:]
  const T *x = logits + (size_t)row * g.C;
  T *dx = logits_grad + (size_t)row * g.C;
  RowGradTerms<T, kHat> terms;
  terms.gx = gx;
  terms.gy = gy;
  terms.sym = sym;
  terms.norm = normalizers[row];
  terms.blank = g.blank;
  terms.sg = kHat ? Sigmoid(x[0]) : T(0);
  for (int c = lane; c < g.C; c += kWave) dx[c] = terms.template At<false>(x[c], c);
}

template <typename T, bool kPruned>
int RowForward(const T *logits, const int64_t *symbols, const int64_t *ranges,
               const int64_t *boundary, T *px, T *py, T *normalizers, RowGeom g,
               hipStream_t stream) {
  const int T1 = g.rnnt_type == K2AMD_REGULAR ? g.Tn + 1 : g.Tn;
  const size_t n_px = (size_t)g.B * g.S * T1, n_py = (size_t)g.B * (g.S + 1) * g.Tn;
  NegInfFill<T> fill{px, py, 0, 0, 1};
  if (kPruned) {
    fill.na = n_px;
    fill.nb = n_py;
  } else if (g.rnnt_type == K2AMD_REGULAR) {
    fill.a = px + (T1 - 1);
    fill.na = (size_t)g.B * g.S;
    fill.stride_a = T1;
  }
  const size_t fill_items = fill.na + fill.nb;
  const unsigned fill_blocks = (unsigned)((fill_items + 4095) / 4096 > 1024 ? 1024 : (fill_items + 4095) / 4096);
  const long long rows = (long long)g.B * g.Tn * g.K;
  const long long blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks + fill_blocks > 0)
    hipLaunchKernelGGL((RowNormKernel<T>), dim3((unsigned)blocks + fill_blocks), dim3(kRowsPerBlock * kWave), 0, stream,
                       logits, normalizers, rows, g.C, g.hat != 0, (unsigned)blocks, fill);
  if (rows > 0)
    hipLaunchKernelGGL((RowEmitKernel<T, kPruned>), dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream,
                       logits, (const T *)normalizers, symbols, ranges, boundary, px, py, g);
  if (g.rnnt_type == K2AMD_CONSTRAINED && n_px > 0)
    hipLaunchKernelGGL(ConstrainedKernel<T>, dim3(1024), dim3(256), 0, stream, px, py, g.B, g.S, g.Tn);
  return LaunchStatus();
}

template <typename T, bool kPruned, bool kHat>
int RowBackward(const T *logits, const T *normalizers, const T *px_grad, const T *py_grad,
                const T *seq_scale, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary,
                T *logits_grad, RowGeom g, hipStream_t stream) {
  const long long rows = (long long)g.B * g.Tn * g.K;
  if (rows > 0) {
    const long long blocks = (rows + kRowsPerBlock - 1) / kRowsPerBlock;
    if (g.C >= 4 && g.C <= (1 << 24)) {  // the record holds the symbol as a float: exact up to 2^24
      hipLaunchKernelGGL((RowGradPrepKernel<T, kPruned>), dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream,
                         normalizers, px_grad, py_grad, seq_scale, symbols, ranges, boundary, logits_grad, g);
      hipLaunchKernelGGL((RowGradKernel<T, kHat>), dim3((unsigned)blocks), dim3(kRowsPerBlock * kWave), 0, stream,
                         logits, logits_grad, rows, g.C, g.blank);
    } else {
      hipLaunchKernelGGL((RowBackwardKernel<T, kPruned, kHat>), dim3((unsigned)blocks), dim3(kRowsPerBlock * kWave), 0, stream,
                         logits, normalizers, px_grad, py_grad, seq_scale, symbols, ranges, boundary,
                         logits_grad, g);
    }
  }
  return LaunchStatus();
}

bool GeomOk(int B, int S, int T, int K, int C, int blank, int rnnt_type, int dtype) {
  if (B < 0 || S < 0 || T < 0 || K < 0 || C <= 0 || blank < 0 || blank >= C) return false;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return false;
  if (dtype != K2AMD_F32 && dtype != K2AMD_F64) return false;
  return (long long)B * T * K < (1ll << 31) * kRowsPerBlock;
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

int k2amd_rnnt_logprobs_joint_forward(const void *logits, const int64_t *symbols,
                                      const int64_t *boundary, void *px, void *py,
                                      void *normalizers, int B, int S, int T, int C,
                                      int termination_symbol, int rnnt_type, int dtype,
                                      void *stream) {
  if (!GeomOk(B, S, T, S + 1, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  RowGeom g{B, S, T, S + 1, C, termination_symbol, rnnt_type, 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return RowForward<float, false>((const float *)logits, symbols, nullptr, boundary, (float *)px, (float *)py, (float *)normalizers, g, st);
  return RowForward<double, false>((const double *)logits, symbols, nullptr, boundary, (double *)px, (double *)py, (double *)normalizers, g, st);
}

int k2amd_rnnt_logprobs_joint_backward(const void *logits, const void *normalizers,
                                       const void *px_grad, const void *py_grad,
                                       const void *seq_scale, const int64_t *symbols, const int64_t *boundary,
                                       void *logits_grad, int B, int S, int T, int C,
                                       int termination_symbol, int rnnt_type, int dtype,
                                       void *stream) {
  if (!GeomOk(B, S, T, S + 1, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  RowGeom g{B, S, T, S + 1, C, termination_symbol, rnnt_type, 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return RowBackward<float, false, false>((const float *)logits, (const float *)normalizers, (const float *)px_grad, (const float *)py_grad, (const float *)seq_scale, symbols, nullptr, boundary, (float *)logits_grad, g, st);
  return RowBackward<double, false, false>((const double *)logits, (const double *)normalizers, (const double *)px_grad, (const double *)py_grad, (const double *)seq_scale, symbols, nullptr, boundary, (double *)logits_grad, g, st);
}

int k2amd_rnnt_logprobs_pruned_forward(const void *logits, const int64_t *symbols,
                                       const int64_t *ranges, const int64_t *boundary, void *px,
                                       void *py, void *normalizers, int B, int S, int T, int R,
                                       int C, int termination_symbol, int rnnt_type, int dtype,
                                       void *stream) {
  if (!GeomOk(B, S, T, R, C, termination_symbol, rnnt_type, dtype) || R < 1 || R > S + 1) return K2AMD_ERR_INVALID_ARGUMENT;
  RowGeom g{B, S, T, R, C, termination_symbol, rnnt_type, 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return RowForward<float, true>((const float *)logits, symbols, ranges, boundary, (float *)px, (float *)py, (float *)normalizers, g, st);
  return RowForward<double, true>((const double *)logits, symbols, ranges, boundary, (double *)px, (double *)py, (double *)normalizers, g, st);
}

int k2amd_rnnt_logprobs_pruned_backward(const void *logits, const void *normalizers,
                                        const void *px_grad, const void *py_grad,
                                        const void *seq_scale, const int64_t *symbols, const int64_t *ranges,
                                        const int64_t *boundary, void *logits_grad, int B, int S,
                                        int T, int R, int C, int termination_symbol, int rnnt_type,
                                        int dtype, void *stream) {
  if (!GeomOk(B, S, T, R, C, termination_symbol, rnnt_type, dtype) || R < 1 || R > S + 1) return K2AMD_ERR_INVALID_ARGUMENT;
  RowGeom g{B, S, T, R, C, termination_symbol, rnnt_type, 0};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return RowBackward<float, true, false>((const float *)logits, (const float *)normalizers, (const float *)px_grad, (const float *)py_grad, (const float *)seq_scale, symbols, ranges, boundary, (float *)logits_grad, g, st);
  return RowBackward<double, true, false>((const double *)logits, (const double *)normalizers, (const double *)px_grad, (const double *)py_grad, (const double *)seq_scale, symbols, ranges, boundary, (double *)logits_grad, g, st);
}

int k2amd_rnnt_hat_logprobs_pruned_forward(const void *logits, const int64_t *symbols,
                                           const int64_t *ranges, const int64_t *boundary,
                                           void *px, void *py, void *normalizers, int B, int S,
                                           int T, int R, int C, int rnnt_type, int dtype,
                                           void *stream) {
  if (!GeomOk(B, S, T, R, C, 0, rnnt_type, dtype) || R < 1 || R > S + 1) return K2AMD_ERR_INVALID_ARGUMENT;
  RowGeom g{B, S, T, R, C, 0, rnnt_type, 1};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return RowForward<float, true>((const float *)logits, symbols, ranges, boundary, (float *)px, (float *)py, (float *)normalizers, g, st);
  return RowForward<double, true>((const double *)logits, symbols, ranges, boundary, (double *)px, (double *)py, (double *)normalizers, g, st);
}

int k2amd_rnnt_hat_logprobs_pruned_backward(const void *logits, const void *normalizers,
                                            const void *px_grad, const void *py_grad,
                                            const void *seq_scale, const int64_t *symbols, const int64_t *ranges,
                                            const int64_t *boundary, void *logits_grad, int B,
                                            int S, int T, int R, int C, int rnnt_type, int dtype,
                                            void *stream) {
  if (!GeomOk(B, S, T, R, C, 0, rnnt_type, dtype) || R < 1 || R > S + 1) return K2AMD_ERR_INVALID_ARGUMENT;
  RowGeom g{B, S, T, R, C, 0, rnnt_type, 1};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return RowBackward<float, true, true>((const float *)logits, (const float *)normalizers, (const float *)px_grad, (const float *)py_grad, (const float *)seq_scale, symbols, ranges, boundary, (float *)logits_grad, g, st);
  return RowBackward<double, true, true>((const double *)logits, (const double *)normalizers, (const double *)px_grad, (const double *)py_grad, (const double *)seq_scale, symbols, ranges, boundary, (double *)logits_grad, g, st);
}

}  // extern "C"
