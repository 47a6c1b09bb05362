// The terms get_rnnt_logprobs_smoothed adds to get_rnnt_logprobs (k2/python/k2/rnnt_loss.py:1471-1704):
// every lattice edge carries
//     joint_scale * log softmax(lm_s + am_t)[k]  +  lm_only_scale * log softmax(lm_s)[k]
//                                                +  am_only_scale * log softmax(am_t + log unigram)[k],
// unigram = mean over all B (S+1) rows of softmax(lm) + tiny, k the edge's symbol.  The joint term
// is the simple builder's output (k2amd_rnnt_logprobs_simple_forward on a regular or modified
// lattice without a boundary); this file turns its saved exponentials into the two marginal
// terms, mixes the three, applies what the reference applies after the mix (the -inf column at
// the last frame of a regular lattice, the "constrained" addition), and carries gradients back
// through the marginal terms.  The joint term's gradient is the simple builder's backward with
// the lattice's gradients scaled by joint_scale.
//
// Every sum here is added in an order that the launch fixes: rows by one wavefront each, columns
// over rows first inside a single-wavefront workgroup (lane c % 64 owns column c and nothing
// else touches it), then over the workgroups in their order.  Results do not depend on scheduling.
//
// The kernels keep to portable HIP (wavefront shuffles, LDS, no inline assembly), so that the
// same source also runs on host threads for tests.
#include "common.h"

namespace k2amd {
namespace {

// rows (of lm forward, of am backward) one single-wavefront workgroup adds up into its partial
// column sums before it writes them
constexpr int kRowsPerGroup = 16;

template <typename T>
__device__ __forceinline__ T WaveTotal(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

template <typename T>
struct SmallestNormal {
  static constexpr T v = std::numeric_limits<T>::min();  // torch.finfo(dtype).tiny
};

inline long long Groups(long long rows) { return (rows + kRowsPerGroup - 1) / kRowsPerGroup; }

// lm_norm[row] = log sum_c exp(lm[row][c]), and partial[group][c] = the group's sum over its rows
// of softmax(lm[row])[c].
template <typename T>
__global__ __launch_bounds__(64) void LmOnlyKernel(const T *__restrict__ lm_probs,
                                                   const T *__restrict__ lm_max,
                                                   T *__restrict__ lm_norm, T *__restrict__ partial,
                                                   long long rows, int C) {
  HIP_DYNAMIC_SHARED(double, lds_words)
  T *acc = reinterpret_cast<T *>(lds_words);  // [C]
  const int lane = threadIdx.x;
  for (int c = lane; c < C; c += kWave) acc[c] = T(0);
  const long long row0 = (long long)blockIdx.x * kRowsPerGroup;
  for (int r = 0; r < kRowsPerGroup && row0 + r < rows; ++r) {
    const long long row = row0 + r;
    const T *p = lm_probs + (size_t)row * C;
    T sum = 0;
    for (int c = lane; c < C; c += kWave) sum += p[c];
    sum = WaveTotal(sum);
    if (lane == 0) lm_norm[row] = Real<T>::Log(sum) + lm_max[row];
    for (int c = lane; c < C; c += kWave) acc[c] += p[c] / sum;
  }
  for (int c = lane; c < C; c += kWave) partial[(size_t)blockIdx.x * C + c] = acc[c];
}

// unigram[c] = sum of the groups' partial sums / rows + tiny;  unigram[C + c] = its log
template <typename T>
__global__ void UnigramKernel(const T *__restrict__ partial, T *__restrict__ unigram, long long groups,
                              long long rows, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  T sum = 0;
  for (long long g = 0; g < groups; ++g) sum += partial[(size_t)g * C + c];
  const T u = sum / T(rows) + SmallestNormal<T>::v;
  unigram[c] = u;
  unigram[(size_t)C + c] = Real<T>::Log(u);
}

// am_norm[row] = log sum_c exp(am[row][c]) unigram[c]; one wavefront per row
template <typename T>
__global__ __launch_bounds__(256) void AmOnlyKernel(const T *__restrict__ am_probs,
                                                    const T *__restrict__ am_max,
                                                    const T *__restrict__ unigram,
                                                    T *__restrict__ am_norm, long long rows, int C) {
  const int lane = threadIdx.x & (kWave - 1);
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;  // the whole wavefront
  const T *p = am_probs + (size_t)row * C;
  T sum = 0;
  for (int c = lane; c < C; c += kWave) sum += p[c] * unigram[c];
  sum = WaveTotal(sum);
  if (lane == 0) am_norm[row] = Real<T>::Log(sum) + am_max[row];
}

template <typename T>
struct MixArgs {
  const T *lm, *am;
  const int64_t *symbols, *boundary;
  const T *lm_norm, *am_norm, *log_unigram;
  const T *px_joint, *py_joint;
  T *px, *py;
  T joint_scale, lm_scale, am_scale;
  int B, S, Tn, C, blank, rnnt_type;
};

// One thread per (b, s, t), s in [0, S]: writes py[b][s][t] and, for s < S, px[b][s][t].
template <typename T>
__global__ __launch_bounds__(256) void MixKernel(const MixArgs<T> a) {
  const int S = a.S, Tn = a.Tn, C = a.C;
  const int T1 = a.rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
  const size_t per_b = (size_t)(S + 1) * Tn, n = (size_t)a.B * per_b;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const int b = (int)(i / per_b);
    const size_t rem = i - (size_t)b * per_b;
    const int s = (int)(rem / Tn), t = (int)(rem - (size_t)s * Tn);
    const size_t lm_row = (size_t)b * (S + 1) + s, am_row = (size_t)b * Tn + t;
    const T *lmr = a.lm + lm_row * C, *amr = a.am + am_row * C;
    const T am_norm = a.am_norm[am_row];
    const T py_am_only = (amr[a.blank] + a.log_unigram[a.blank]) - am_norm;
    const T py_mix = a.py_joint[i] * a.joint_scale + (lmr[a.blank] - a.lm_norm[lm_row]) * a.lm_scale +
                     py_am_only * a.am_scale;
    a.py[i] = py_mix;
    if (s == S) continue;
    T *pxr = a.px + ((size_t)b * S + s) * T1;
    if (a.rnnt_type == K2AMD_REGULAR && t == Tn - 1) pxr[Tn] = Real<T>::NegInf();
    const int64_t sym = a.symbols[(size_t)b * S + s];
    T px_mix = Real<T>::NegInf();
    if (sym >= 0 && sym < C) {
      px_mix = a.px_joint[((size_t)b * S + s) * T1 + t] * a.joint_scale +
               (lmr[sym] - a.lm_norm[lm_row]) * a.lm_scale +
               ((amr[sym] + a.log_unigram[sym]) - am_norm) * a.am_scale;
      if (a.rnnt_type == K2AMD_REGULAR && a.boundary != nullptr && a.boundary[4 * b + 3] == t)
        px_mix = Real<T>::NegInf();
      if (a.rnnt_type == K2AMD_CONSTRAINED)  // + py of the row above, mixed the same way
        px_mix += a.py_joint[i + Tn] * a.joint_scale +
                  (lmr[(size_t)C + a.blank] - a.lm_norm[lm_row + 1]) * a.lm_scale + py_am_only * a.am_scale;
    }
    pxr[t] = px_mix;
  }
}

template <typename T>
__global__ void FillKernel(T *__restrict__ dst, size_t n, T v) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = v;
}

// What reaches the mixed px / py of sequence b, as the two marginal terms see it: the "cut" of a
// regular lattice (px[b][:][boundary[b][3]] was overwritten with -inf: nothing flows back) and
// the "constrained" addition (py[b][s][t] also fed px[b][s-1][t]).
template <typename T>
struct LatticeGrads {
  const T *px_grad, *py_grad;
  const T *seq_scale;  // what reaches sequence b's score multiplies its gradients (null: 1)
  const int64_t *boundary;
  int S, Tn, rnnt_type;
  __device__ __forceinline__ T Scale(int b) const { return seq_scale != nullptr ? seq_scale[b] : T(1); }
  __device__ __forceinline__ T Gx(int b, int s, int t) const {
    if (s >= S) return T(0);
    if (rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t) return T(0);
    const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
    return px_grad[((size_t)b * S + s) * T1 + t] * Scale(b);
  }
  __device__ __forceinline__ T Gy(int b, int s, int t) const {
    T g = py_grad[((size_t)b * (S + 1) + s) * Tn + t] * Scale(b);
    if (rnnt_type == K2AMD_CONSTRAINED && s >= 1) g += Gx(b, s - 1, t);
    return g;
  }
};

// The am-only term's gradient.  With z = am[b][t] + log unigram, vx / vy the sums over s of
// Gx / Gy at frame t, and p = softmax(z) = am_probs unigram exp(am_max - am_norm):
//     dz[c] = am_scale * ( sum over s with symbols[b][s] == c of Gx(b,s,t)  +  (c == blank) vy
//                          - p[c] (vx + vy) )
// is added to am_grad[b][t], and the group's sum of dz over its rows is written to partial[group]
// (the gradient that reaches log unigram).
// The symbols' terms: positions that carry the same symbol are chained once per sequence
// (lead_of[s] = the symbol if s is its first position, else -1; next_of[s] = the next position
// with the same symbol, or -1), so that per row the first position's lane adds up its chain in
// ascending s and writes one column: a fixed order, no two lanes on one column, and a cost per row
// of the longest chain rather than of S.
// LDS: the row being built [C], the group's sums [C], Gx of the row's frame [S]; then as ints the
// sequence's symbols [S], lead_of [S], next_of [S].
template <typename T>
__global__ __launch_bounds__(64) void AmOnlyGradKernel(LatticeGrads<T> g, const int64_t *__restrict__ symbols,
                                                       const T *__restrict__ am_probs,
                                                       const T *__restrict__ am_max,
                                                       const T *__restrict__ am_norm,
                                                       const T *__restrict__ unigram,
                                                       T *__restrict__ am_grad, T *__restrict__ partial,
                                                       long long rows, int C, int blank, T am_scale) {
  HIP_DYNAMIC_SHARED(double, lds_words)
  T *dz = reinterpret_cast<T *>(lds_words);  // [C]
  T *acc = dz + C;                           // [C]
  T *gx_of = acc + C;                        // [S]
  const int lane = threadIdx.x, S = g.S, Tn = g.Tn;
  int *sym_of = reinterpret_cast<int *>(gx_of + S);  // [S]
  int *lead_of = sym_of + S;                         // [S]
  int *next_of = lead_of + S;                        // [S]
  for (int c = lane; c < C; c += kWave) acc[c] = T(0);
  const long long row0 = (long long)blockIdx.x * kRowsPerGroup;
  int chained_b = -1;  // the sequence whose chains the LDS arrays hold
  for (int r = 0; r < kRowsPerGroup && row0 + r < rows; ++r) {
    const long long row = row0 + r;
    const int b = (int)(row / Tn), t = (int)(row - (long long)b * Tn);
    if (b != chained_b) {  // the same for every lane
      chained_b = b;
      const int64_t *sym = symbols + (size_t)b * S;
      for (int s = lane; s < S; s += kWave) sym_of[s] = sym[s] >= 0 && sym[s] < C ? (int)sym[s] : -1;
      __syncthreads();
      for (int s = lane; s < S; s += kWave) {
        const int mine = sym_of[s];
        bool first = mine >= 0;
        int next = -1;
        if (mine >= 0) {
          for (int k = 0; k < s && first; ++k) first = sym_of[k] != mine;
          for (int k = s + 1; k < S && next < 0; ++k)
            if (sym_of[k] == mine) next = k;
        }
        lead_of[s] = first ? mine : -1;
        next_of[s] = next;
      }
    }
    T vx = 0, vy = 0;
    for (int s = lane; s <= S; s += kWave) {
      const T gx = g.Gx(b, s, t);
      if (s < S) gx_of[s] = gx;
      vx += gx;
      vy += g.Gy(b, s, t);
    }
    vx = WaveTotal(vx);
    vy = WaveTotal(vy);
    const T inv_sum = Real<T>::Exp(am_max[row] - am_norm[row]);
    const T *p = am_probs + (size_t)row * C;
    for (int c = lane; c < C; c += kWave)
      dz[c] = am_scale * ((c == blank ? vy : T(0)) - p[c] * unigram[c] * inv_sum * (vx + vy));
    __syncthreads();  // dz, gx_of and the chains are read by other lanes than the ones that wrote them
    for (int s = lane; s < S; s += kWave) {
      const int c = lead_of[s];
      if (c < 0) continue;
      T v = gx_of[s];
      for (int k = next_of[s]; k >= 0; k = next_of[k]) v += gx_of[k];
      dz[c] += am_scale * v;
    }
    __syncthreads();
    T *out = am_grad + (size_t)row * C;
    for (int c = lane; c < C; c += kWave) {
      const T v = dz[c];
      out[c] += v;
      acc[c] += v;
    }
    __syncthreads();  // before the next row overwrites dz and gx_of
  }
  for (int c = lane; c < C; c += kWave) partial[(size_t)blockIdx.x * C + c] = acc[c];
}

// d_unigram[c] = sum of the groups' partial sums / unigram[c] / lm_rows: what one row's
// softmax(lm)[c] receives through the unigram (log unigram = log(mean + tiny)).
template <typename T>
__global__ void UnigramGradKernel(const T *__restrict__ partial, const T *__restrict__ unigram,
                                  T *__restrict__ d_unigram, long long groups, long long lm_rows, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  T sum = 0;
  for (long long k = 0; k < groups; ++k) sum += partial[(size_t)k * C + c];
  d_unigram[c] = sum / unigram[c] / T(lm_rows);
}

// The lm-only term's gradient and the unigram's, one wavefront per row (b, s) of lm.  With
// p = softmax(lm[b][s]) = lm_probs exp(lm_max - lm_norm), wx / wy the sums over t of Gx / Gy:
//     lm_grad[b][s][c] += lm_scale * ( (c == symbols[b][s]) wx + (c == blank) wy - p[c] (wx + wy) )
//                         + p[c] ( d_unigram[c] - sum_k p[k] d_unigram[k] )
template <typename T>
__global__ __launch_bounds__(256) void LmOnlyGradKernel(LatticeGrads<T> g, const int64_t *__restrict__ symbols,
                                                        const T *__restrict__ lm_probs,
                                                        const T *__restrict__ lm_max,
                                                        const T *__restrict__ lm_norm,
                                                        const T *__restrict__ d_unigram,
                                                        T *__restrict__ lm_grad, long long rows, int C,
                                                        int blank, T lm_scale) {
  const int lane = threadIdx.x & (kWave - 1), S = g.S, Tn = g.Tn;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;  // the whole wavefront
  const int b = (int)(row / (S + 1)), s = (int)(row - (long long)b * (S + 1));
  T wx = 0, wy = 0;
  for (int t = lane; t < Tn; t += kWave) {
    wx += g.Gx(b, s, t);
    wy += g.Gy(b, s, t);
  }
  wx = WaveTotal(wx);
  wy = WaveTotal(wy);
  const T inv_sum = Real<T>::Exp(lm_max[row] - lm_norm[row]);
  const T *p = lm_probs + (size_t)row * C;
  T dot = 0;
  for (int c = lane; c < C; c += kWave) dot += p[c] * inv_sum * d_unigram[c];
  dot = WaveTotal(dot);
  const int64_t sym = s < S ? symbols[(size_t)b * S + s] : -1;
  T *out = lm_grad + (size_t)row * C;
  for (int c = lane; c < C; c += kWave) {
    const T pc = p[c] * inv_sum;
    T v = lm_scale * ((c == blank ? wy : T(0)) - pc * (wx + wy)) + pc * (d_unigram[c] - dot);
    if (c == sym) v += lm_scale * wx;
    out[c] += v;
  }
}

constexpr size_t kLdsLimit = 64 * 1024;  // what a launch may ask for without a function attribute

// AmOnlyGradKernel's arrays: 2 C + S elements, then 3 S ints
inline size_t BackwardLdsBytes(int S, int C, size_t elem) { return ((size_t)2 * C + S) * elem + (size_t)3 * S * 4; }

bool ArgsOk(int B, int S, int T, int C, int blank, int rnnt_type, int dtype) {
  if (B < 0 || S < 0 || T < 0 || C <= 0 || blank < 0 || blank >= C) return false;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return false;
  return dtype == K2AMD_F32 || dtype == K2AMD_F64;
}

// The vocabulary has to fit the workgroups' LDS arrays, and grid sizes 32 bits.
bool Served(int B, int S, int T, int C, int dtype) {
  if (BackwardLdsBytes(S, C, dtype == K2AMD_F64 ? 8 : 4) > kLdsLimit) return false;
  const long long lim = 1ll << 30;
  return (long long)B * (S + 1) < lim && (long long)B * T < lim;
}

inline unsigned GridFor(size_t n) { return (unsigned)std::min<size_t>((n + 255) / 256, 8192); }

template <typename T>
int SmoothedForward(const T *lm, const T *am, const int64_t *symbols, const int64_t *boundary,
                    const T *lm_probs, const T *am_probs, const T *lm_max, const T *am_max,
                    const T *px_joint, const T *py_joint, T *px, T *py, T *lm_norm, T *am_norm,
                    T *unigram, T *scratch, double lm_only_scale, double am_only_scale, int B, int S,
                    int Tn, int C, int blank, int rnnt_type, hipStream_t st) {
  const long long lm_rows = (long long)B * (S + 1), am_rows = (long long)B * Tn;
  const long long groups = Groups(lm_rows);
  hipLaunchKernelGGL(LmOnlyKernel<T>, dim3((unsigned)groups), dim3(64), (size_t)C * sizeof(T), st, lm_probs,
                     lm_max, lm_norm, scratch, lm_rows, C);
  hipLaunchKernelGGL(UnigramKernel<T>, dim3((C + 255) / 256), dim3(256), 0, st, (const T *)scratch, unigram,
                     groups, lm_rows, C);
  if (Tn == 0) {  // no frames: py is empty, px is its one -inf column where the lattice is regular
    if (rnnt_type == K2AMD_REGULAR && S > 0)
      hipLaunchKernelGGL(FillKernel<T>, dim3(GridFor((size_t)B * S)), dim3(256), 0, st, px, (size_t)B * S,
                         Real<T>::NegInf());
    return LaunchStatus();
  }
  hipLaunchKernelGGL(AmOnlyKernel<T>, dim3((unsigned)((am_rows + 3) / 4)), dim3(256), 0, st, am_probs, am_max,
                     (const T *)unigram, am_norm, am_rows, C);
  const double joint_scale = 1.0 - lm_only_scale - am_only_scale;
  // exact zeros would turn an infinite term into a NaN (k2/python/k2/rnnt_loss.py:1677-1682)
  if (lm_only_scale == 0.0) lm_only_scale = 1.0e-20;
  if (am_only_scale == 0.0) am_only_scale = 1.0e-20;
  MixArgs<T> a{lm, am, symbols, boundary, lm_norm, am_norm, unigram + C, px_joint, py_joint, px, py,
               (T)joint_scale, (T)lm_only_scale, (T)am_only_scale, B, S, Tn, C, blank, rnnt_type};
  hipLaunchKernelGGL(MixKernel<T>, dim3(GridFor((size_t)lm_rows * Tn)), dim3(256), 0, st, a);
  return LaunchStatus();
}

template <typename T>
int SmoothedBackward(const T *px_grad, const T *py_grad, const T *seq_scale, const int64_t *symbols,
                     const int64_t *boundary, const T *lm_probs, const T *am_probs, const T *lm_max,
                     const T *am_max, const T *lm_norm, const T *am_norm, const T *unigram, T *lm_grad,
                     T *am_grad, T *scratch, double lm_only_scale, double am_only_scale, int B, int S,
                     int Tn, int C, int blank, int rnnt_type, hipStream_t st) {
  const long long lm_rows = (long long)B * (S + 1), am_rows = (long long)B * Tn;
  const long long groups = Groups(am_rows);
  if (lm_only_scale == 0.0) lm_only_scale = 1.0e-20;
  if (am_only_scale == 0.0) am_only_scale = 1.0e-20;
  LatticeGrads<T> g{px_grad, py_grad, seq_scale, boundary, S, Tn, rnnt_type};
  T *d_unigram = scratch, *partial = scratch + C;
  if (groups > 0)
    hipLaunchKernelGGL(AmOnlyGradKernel<T>, dim3((unsigned)groups), dim3(64), BackwardLdsBytes(S, C, sizeof(T)), st, g,
                       symbols, am_probs, am_max, am_norm, unigram, am_grad, partial, am_rows, C, blank,
                       (T)am_only_scale);
  hipLaunchKernelGGL(UnigramGradKernel<T>, dim3((C + 255) / 256), dim3(256), 0, st, (const T *)partial, unigram,
                     d_unigram, groups, lm_rows, C);
  hipLaunchKernelGGL(LmOnlyGradKernel<T>, dim3((unsigned)((lm_rows + 3) / 4)), dim3(256), 0, st, g, symbols,
                     lm_probs, lm_max, lm_norm, (const T *)d_unigram, lm_grad, lm_rows, C, blank,
                     (T)lm_only_scale);
  return LaunchStatus();
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

size_t k2amd_rnnt_smoothed_scratch_elements(int B, int S, int T, int C) {
  if (B <= 0 || S < 0 || T < 0 || C <= 0) return 0;
  const size_t forward = (size_t)Groups((long long)B * (S + 1)) * C;
  const size_t backward = (size_t)C + (size_t)Groups((long long)B * T) * C;
  return std::max(forward, backward);
}

int k2amd_rnnt_smoothed_supported(int B, int S, int T, int C, int dtype) {
  return B >= 0 && S >= 0 && T >= 0 && C > 0 && (dtype == K2AMD_F32 || dtype == K2AMD_F64) &&
         Served(B, S, T, C, dtype);
}

int k2amd_rnnt_smoothed_forward(const void *lm, const void *am, const int64_t *symbols, const int64_t *boundary,
                                const void *lm_probs, const void *am_probs, const void *lm_max,
                                const void *am_max, const void *px_joint, const void *py_joint, void *px,
                                void *py, void *lm_norm, void *am_norm, void *unigram, void *scratch,
                                size_t scratch_elements, double lm_only_scale, double am_only_scale, int B,
                                int S, int T, int C, int termination_symbol, int rnnt_type, int dtype,
                                void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (!Served(B, S, T, C, dtype)) return K2AMD_ERR_UNSUPPORTED;
  if (B == 0) return K2AMD_OK;
  if (!lm || !lm_probs || !lm_max || !lm_norm || !unigram || (!symbols && S > 0) || (!px && S > 0))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (T > 0 && (!am || !am_probs || !am_max || !am_norm || !py || !py_joint || (!px_joint && S > 0)))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (!scratch || scratch_elements < k2amd_rnnt_smoothed_scratch_elements(B, S, T, C)) return K2AMD_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SmoothedForward<float>((const float *)lm, (const float *)am, symbols, boundary, (const float *)lm_probs, (const float *)am_probs, (const float *)lm_max, (const float *)am_max, (const float *)px_joint, (const float *)py_joint, (float *)px, (float *)py, (float *)lm_norm, (float *)am_norm, (float *)unigram, (float *)scratch, lm_only_scale, am_only_scale, B, S, T, C, termination_symbol, rnnt_type, st);
  return SmoothedForward<double>((const double *)lm, (const double *)am, symbols, boundary, (const double *)lm_probs, (const double *)am_probs, (const double *)lm_max, (const double *)am_max, (const double *)px_joint, (const double *)py_joint, (double *)px, (double *)py, (double *)lm_norm, (double *)am_norm, (double *)unigram, (double *)scratch, lm_only_scale, am_only_scale, B, S, T, C, termination_symbol, rnnt_type, st);
}

int k2amd_rnnt_smoothed_backward(const void *px_grad, const void *py_grad, const void *seq_scale,
                                 const int64_t *symbols, const int64_t *boundary, const void *lm_probs,
                                 const void *am_probs, const void *lm_max, const void *am_max,
                                 const void *lm_norm, const void *am_norm, const void *unigram, void *lm_grad,
                                 void *am_grad, void *scratch, size_t scratch_elements, double lm_only_scale,
                                 double am_only_scale, int B, int S, int T, int C, int termination_symbol,
                                 int rnnt_type, int dtype, void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (!Served(B, S, T, C, dtype)) return K2AMD_ERR_UNSUPPORTED;
  if (B == 0) return K2AMD_OK;
  if (!lm_probs || !lm_max || !lm_norm || !unigram || !lm_grad || (!symbols && S > 0))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (T > 0 && (!py_grad || (!px_grad && S > 0) || !am_probs || !am_max || !am_norm || !am_grad))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (!scratch || scratch_elements < k2amd_rnnt_smoothed_scratch_elements(B, S, T, C)) return K2AMD_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SmoothedBackward<float>((const float *)px_grad, (const float *)py_grad, (const float *)seq_scale, symbols, boundary, (const float *)lm_probs, (const float *)am_probs, (const float *)lm_max, (const float *)am_max, (const float *)lm_norm, (const float *)am_norm, (const float *)unigram, (float *)lm_grad, (float *)am_grad, (float *)scratch, lm_only_scale, am_only_scale, B, S, T, C, termination_symbol, rnnt_type, st);
  return SmoothedBackward<double>((const double *)px_grad, (const double *)py_grad, (const double *)seq_scale, symbols, boundary, (const double *)lm_probs, (const double *)am_probs, (const double *)lm_max, (const double *)am_max, (const double *)lm_norm, (const double *)am_norm, (const double *)unigram, (double *)lm_grad, (double *)am_grad, (double *)scratch, lm_only_scale, am_only_scale, B, S, T, C, termination_symbol, rnnt_type, st);
}

}  // extern "C"
