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
// Everything is row work over [B][S+1][C], [B][T][C] and the lattice, one wavefront per row, plus
// sums down the columns of those tensors (over all rows of the batch: the unigram and its
// gradient), which take two steps: 64 columns x a chunk of rows per workgroup, four wavefronts
// adding every fourth row of the chunk, then the chunks added in order by the kernel that
// consumes them.  Every sum is added in an order that the launch fixes; results do not depend on
// scheduling.  No vocabulary limit: nothing holds a row in LDS.
//
// The kernels keep to portable HIP (wavefront shuffles, LDS, no inline assembly), so that the
// same source also runs on host threads for tests.
#include "common.h"

namespace k2amd {
namespace {

constexpr int kRowsPerBlock = 4;  // one wavefront per row, 256 threads per workgroup
constexpr int kMaxChunks = 64;    // chunks of rows of a column sum

template <typename T>
__device__ __forceinline__ T WaveTotal(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ int WaveLowest(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = min(v, __shfl_xor(v, off, kWave));
  return v;
}

template <typename T>
struct SmallestNormal {
  static constexpr T v = std::numeric_limits<T>::min();  // torch.finfo(dtype).tiny
};

// chunks a column sum over `rows` rows is split into, and the rows of each
inline int Chunks(long long rows) { return (int)std::min<long long>(kMaxChunks, std::max<long long>(1, (rows + 63) / 64)); }
inline int RowsPerChunk(long long rows) { return (int)((rows + Chunks(rows) - 1) / Chunks(rows)); }
inline unsigned RowBlocks(long long rows) { return (unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock); }

// lm_norm[row] = log sum_c exp(lm[row][c]);  inv_sum[row] = 1 / sum_c exp(lm[row][c] - max)
template <typename T>
__global__ __launch_bounds__(256) void LmRowKernel(const T *__restrict__ lm_probs, const T *__restrict__ lm_max,
                                                   T *__restrict__ lm_norm, T *__restrict__ inv_sum,
                                                   long long rows, int C) {
  const int lane = threadIdx.x & (kWave - 1);
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;  // the whole wavefront
  const T *p = lm_probs + (size_t)row * C;
  T sum = 0;
  for (int c = lane; c < C; c += kWave) sum += p[c];
  sum = WaveTotal(sum);
  if (lane == 0) {
    lm_norm[row] = Real<T>::Log(sum) + lm_max[row];
    inv_sum[row] = T(1) / sum;
  }
}

// Two column sums in one launch (blockIdx.z picks; grid.z = 1 runs the first alone):
//   z = 0:  partial[chunk][c]  = sum over the chunk's rows r of x[r][c] * weight[r]
//   z = 1:  partial2[chunk][c] = sum over the chunk's rows (b, s) of lm of
//                                (c == symbols[b][s]) wx(b,s) + (c == blank) wy(b,s),
//           wx, wy = row_info[row][0], [1]
// Workgroup = 64 columns x one chunk; wavefront w adds rows first + w, first + w + 4, ...
template <typename T>
struct ColumnSumArgs {
  const T *x, *weight;
  T *partial;
  long long rows;
  int rows_per_chunk, chunks;
  const T *row_info;
  const int64_t *symbols;
  T *partial2;
  long long rows2;
  int rows_per_chunk2, chunks2, S, blank;
};

template <typename T>
__global__ __launch_bounds__(256) void ColumnSumsKernel(const ColumnSumArgs<T> a, int C) {
  __shared__ T part[4][kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int c = blockIdx.x * kWave + lane, chunk = blockIdx.y;
  const bool second = blockIdx.z == 1;
  const int chunks = second ? a.chunks2 : a.chunks;
  T acc = 0;
  if (chunk < chunks && c < C) {  // (the two sums may have different numbers of chunks)
    const int per = second ? a.rows_per_chunk2 : a.rows_per_chunk;
    const long long rows = second ? a.rows2 : a.rows;
    const long long first = (long long)chunk * per, last = min(rows, first + per);
    if (!second) {
      for (long long r = first + wave; r < last; r += 4) acc += a.x[(size_t)r * C + c] * a.weight[r];
    } else {
      for (long long r = first + wave; r < last; r += 4) {
        const int b = (int)(r / (a.S + 1)), s = (int)(r - (long long)b * (a.S + 1));
        if (s < a.S && a.symbols[(size_t)b * a.S + s] == c) acc += a.row_info[4 * r];
        if (c == a.blank) acc += a.row_info[4 * r + 1];
      }
    }
  }
  part[wave][lane] = acc;
  __syncthreads();
  if (wave == 0 && chunk < chunks && c < C)
    (second ? a.partial2 : a.partial)[(size_t)chunk * C + c] =
        (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}

// unigram[c] = sum of the chunks' partial sums / rows + tiny;  unigram[C + c] = its log
template <typename T>
__global__ void UnigramKernel(const T *__restrict__ partial, T *__restrict__ unigram, int chunks,
                              long long rows, int C) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  T sum = 0;
  for (int k = 0; k < chunks; ++k) sum += partial[(size_t)k * C + c];
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
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
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

// Backward, first pass: what every later kernel needs of the lattice's gradients, one wavefront
// per row of lm, then per row of am.
//   row (b, s) of lm:  row_info[row] = { wx, wy, lead, next }: wx / wy the sums over t of
//       Gx / Gy; lead = 1 if s is the first position of sequence b that carries its symbol (and
//       the symbol is inside the vocabulary), else 0; next = the next position with the same
//       symbol, or -1 (small integers, exact in the element type).  The chains let a row of am
//       add the terms of a repeated symbol in ascending s, one lane per distinct symbol.
//   row (b, t) of am:  col_info[row] = { vx + vy, vy }, the sums over s of Gx / Gy at frame t,
//       and am_weight[row] = (vx + vy) exp(am_max - am_norm): softmax(am + log unigram)[c]
//       (vx + vy) = am_probs[c] unigram[c] am_weight.
template <typename T>
__global__ __launch_bounds__(256) void LatticeSumsKernel(LatticeGrads<T> g, const int64_t *__restrict__ symbols,
                                                         const T *__restrict__ am_max,
                                                         const T *__restrict__ am_norm,
                                                         T *__restrict__ row_info, T *__restrict__ col_info,
                                                         T *__restrict__ am_weight, long long lm_rows,
                                                         long long am_rows, int C) {
  const int lane = threadIdx.x & (kWave - 1), S = g.S, Tn = g.Tn;
  long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row < lm_rows) {
    const int b = (int)(row / (S + 1)), s = (int)(row - (long long)b * (S + 1));
    T wx = 0, wy = 0;
    for (int t = lane; t < Tn; t += kWave) {
      wx += g.Gx(b, s, t);
      wy += g.Gy(b, s, t);
    }
    wx = WaveTotal(wx);
    wy = WaveTotal(wy);
    const int64_t *sym = symbols + (size_t)b * S;
    const int64_t mine = s < S ? sym[s] : -1;
    const bool valid = mine >= 0 && mine < C;
    int earlier = 0, next = S;  // S: none
    if (valid)
      for (int k = lane; k < S; k += kWave)
        if (sym[k] == mine) {
          if (k < s) earlier = 1;
          if (k > s) next = min(next, k);
        }
    earlier = -WaveLowest(-earlier);  // 1 if any lane saw one
    next = WaveLowest(next);
    if (lane == 0) {
      T *info = row_info + 4 * (size_t)row;
      info[0] = wx;
      info[1] = wy;
      info[2] = T(valid && !earlier ? 1 : 0);
      info[3] = T(next < S ? next : -1);
    }
    return;
  }
  row -= lm_rows;
  if (row >= am_rows) return;
  const int b = (int)(row / Tn), t = (int)(row - (long long)b * Tn);
  T vx = 0, vy = 0;
  for (int s = lane; s <= S; s += kWave) {
    vx += g.Gx(b, s, t);
    vy += g.Gy(b, s, t);
  }
  vx = WaveTotal(vx);
  vy = WaveTotal(vy);
  if (lane == 0) {
    col_info[2 * (size_t)row] = vx + vy;
    col_info[2 * (size_t)row + 1] = vy;
    am_weight[row] = (vx + vy) * Real<T>::Exp(am_max[row] - am_norm[row]);
  }
}

// The am-only term's gradient, one wavefront per row (b, t) of am.  With z = am[b][t] + log
// unigram and p = softmax(z):
//     dz[c] = am_scale * ( sum over s with symbols[b][s] == c of Gx(b,s,t)  +  (c == blank) vy
//                          - p[c] (vx + vy) )
// is added to am_grad[b][t]: the dense part by every lane over its columns, then, once those
// stores have completed, the symbols' terms by the lanes that hold a chain's first position.
template <typename T>
__global__ __launch_bounds__(256) void AmOnlyGradKernel(LatticeGrads<T> g, const int64_t *__restrict__ symbols,
                                                        const T *__restrict__ am_probs,
                                                        const T *__restrict__ unigram,
                                                        const T *__restrict__ row_info,
                                                        const T *__restrict__ col_info,
                                                        const T *__restrict__ am_weight,
                                                        T *__restrict__ am_grad, long long rows, int C,
                                                        int blank, T am_scale) {
  const int lane = threadIdx.x & (kWave - 1), S = g.S, Tn = g.Tn;
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  const bool live = row < rows;  // (no early exit: the barrier below is for all wavefronts)
  const long long r = live ? row : 0;
  const int b = (int)(r / Tn), t = (int)(r - (long long)b * Tn);
  T *out = am_grad + (size_t)r * C;
  if (live) {
    const T vy = col_info[2 * (size_t)r + 1], weight = am_weight[r];
    const T *p = am_probs + (size_t)r * C;
    for (int c = lane; c < C; c += kWave)
      out[c] += am_scale * ((c == blank ? vy : T(0)) - p[c] * unigram[c] * weight);
  }
  __syncthreads();  // the stores above, before other lanes add to the same elements
  if (!live) return;
  const T *info = row_info + 4 * (size_t)b * (S + 1);
  const int64_t *sym = symbols + (size_t)b * S;
  for (int s = lane; s < S; s += kWave) {
    if (info[4 * s + 2] == T(0)) continue;  // not the first position of its symbol
    T v = g.Gx(b, s, t);
    for (int k = (int)info[4 * s + 3]; k >= 0; k = (int)info[4 * k + 3]) v += g.Gx(b, k, t);
    out[sym[s]] += am_scale * v;
  }
}

// d_unigram[c]: what one row's softmax(lm)[c] receives through the unigram.  The gradient that
// reaches log unigram[c] is the sum over all rows of am of dz[c]:
//     am_scale * ( partial2 summed over its chunks  -  unigram[c] * partial summed over its chunks ),
// and log unigram = log(mean + tiny), the mean over lm_rows rows.
template <typename T>
__global__ void UnigramGradKernel(const T *__restrict__ partial, int chunks, const T *__restrict__ partial2,
                                  int chunks2, const T *__restrict__ unigram, T *__restrict__ d_unigram,
                                  long long lm_rows, int C, T am_scale) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  T dense = 0, sparse = 0;
  for (int k = 0; k < chunks; ++k) dense += partial[(size_t)k * C + c];
  for (int k = 0; k < chunks2; ++k) sparse += partial2[(size_t)k * C + c];
  d_unigram[c] = am_scale * (sparse - unigram[c] * dense) / unigram[c] / T(lm_rows);
}

// The lm-only term's gradient and the unigram's, one wavefront per row (b, s) of lm.  With
// p = softmax(lm[b][s]) = lm_probs exp(lm_max - lm_norm), wx / wy the sums over t of Gx / Gy:
//     lm_grad[b][s][c] += lm_scale * ( (c == symbols[b][s]) wx + (c == blank) wy - p[c] (wx + wy) )
//                         + p[c] ( d_unigram[c] - sum_k p[k] d_unigram[k] )
template <typename T>
__global__ __launch_bounds__(256) void LmOnlyGradKernel(const int64_t *__restrict__ symbols,
                                                        const T *__restrict__ lm_probs,
                                                        const T *__restrict__ lm_max,
                                                        const T *__restrict__ lm_norm,
                                                        const T *__restrict__ row_info,
                                                        const T *__restrict__ d_unigram,
                                                        T *__restrict__ lm_grad, long long rows, int S, int C,
                                                        int blank, T lm_scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const long long row = (long long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;  // the whole wavefront
  const int b = (int)(row / (S + 1)), s = (int)(row - (long long)b * (S + 1));
  const T wx = row_info[4 * (size_t)row], wy = row_info[4 * (size_t)row + 1];
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

bool ArgsOk(int B, int S, int T, int C, int blank, int rnnt_type, int dtype) {
  if (B < 0 || S < 0 || T < 0 || C <= 0 || blank < 0 || blank >= C) return false;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return false;
  return dtype == K2AMD_F32 || dtype == K2AMD_F64;
}

// Grid sizes and row numbers are 32 bits.
bool Served(int B, int S, int T, int C) {
  const long long lim = 1ll << 30;
  return (long long)B * (S + 1) + (long long)B * T < lim && C < (1 << 26);
}

inline unsigned GridFor(size_t n) { return (unsigned)std::min<size_t>((n + 255) / 256, 8192); }

// scratch of the forward: inv_sum [lm_rows], partial [chunks][C]
size_t ForwardScratch(long long lm_rows, int C) { return (size_t)lm_rows + (size_t)Chunks(lm_rows) * C; }
// of the backward: row_info [lm_rows][4], col_info [am_rows][2], am_weight [am_rows],
// partial [chunks of am rows][C], partial2 [chunks of lm rows][C], d_unigram [C]
size_t BackwardScratch(long long lm_rows, long long am_rows, int C) {
  return 4 * (size_t)lm_rows + 3 * (size_t)am_rows +
         ((size_t)Chunks(am_rows) + (size_t)Chunks(lm_rows) + 1) * C;
}

template <typename T>
int SmoothedForward(const T *lm, const T *am, const int64_t *symbols, const int64_t *boundary,
                    const T *lm_probs, const T *am_probs, const T *lm_max, const T *am_max,
                    const T *px_joint, const T *py_joint, T *px, T *py, T *lm_norm, T *am_norm,
                    T *unigram, T *scratch, double lm_only_scale, double am_only_scale, int B, int S,
                    int Tn, int C, int blank, int rnnt_type, hipStream_t st) {
  const long long lm_rows = (long long)B * (S + 1), am_rows = (long long)B * Tn;
  T *inv_sum = scratch, *partial = scratch + lm_rows;
  const int chunks = Chunks(lm_rows);
  hipLaunchKernelGGL(LmRowKernel<T>, dim3(RowBlocks(lm_rows)), dim3(256), 0, st, lm_probs, lm_max, lm_norm, inv_sum,
                     lm_rows, C);
  ColumnSumArgs<T> sums{lm_probs, inv_sum, partial, lm_rows, RowsPerChunk(lm_rows), chunks,
                        nullptr, nullptr, nullptr, 0, 0, 0, S, blank};
  hipLaunchKernelGGL(ColumnSumsKernel<T>, dim3((C + kWave - 1) / kWave, chunks, 1), dim3(256), 0, st, sums, C);
  hipLaunchKernelGGL(UnigramKernel<T>, dim3((C + 255) / 256), dim3(256), 0, st, (const T *)partial, unigram,
                     chunks, lm_rows, C);
  if (Tn == 0) {  // no frames: py is empty, px is its one -inf column where the lattice is regular
    if (rnnt_type == K2AMD_REGULAR && S > 0)
      hipLaunchKernelGGL(FillKernel<T>, dim3(GridFor((size_t)B * S)), dim3(256), 0, st, px, (size_t)B * S,
                         Real<T>::NegInf());
    return LaunchStatus();
  }
  hipLaunchKernelGGL(AmOnlyKernel<T>, dim3(RowBlocks(am_rows)), dim3(256), 0, st, am_probs, am_max,
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
  if (lm_only_scale == 0.0) lm_only_scale = 1.0e-20;
  if (am_only_scale == 0.0) am_only_scale = 1.0e-20;
  LatticeGrads<T> g{px_grad, py_grad, seq_scale, boundary, S, Tn, rnnt_type};
  const int chunks_am = Chunks(am_rows), chunks_lm = Chunks(lm_rows);
  T *row_info = scratch, *col_info = row_info + 4 * lm_rows, *am_weight = col_info + 2 * am_rows;
  T *partial = am_weight + am_rows, *partial2 = partial + (size_t)chunks_am * C;
  T *d_unigram = partial2 + (size_t)chunks_lm * C;
  hipLaunchKernelGGL(LatticeSumsKernel<T>, dim3(RowBlocks(lm_rows) + RowBlocks(am_rows) + 1), dim3(256), 0, st, g,
                     symbols, am_max, am_norm, row_info, col_info, am_weight, lm_rows, am_rows, C);
  if (am_rows > 0)
    hipLaunchKernelGGL(AmOnlyGradKernel<T>, dim3(RowBlocks(am_rows)), dim3(256), 0, st, g, symbols, am_probs,
                       unigram, (const T *)row_info, (const T *)col_info, (const T *)am_weight, am_grad, am_rows, C,
                       blank, (T)am_only_scale);
  ColumnSumArgs<T> sums{am_probs, am_weight, partial, am_rows, RowsPerChunk(std::max<long long>(am_rows, 1)),
                        am_rows > 0 ? chunks_am : 0, row_info, symbols, partial2, lm_rows, RowsPerChunk(lm_rows),
                        chunks_lm, S, blank};
  hipLaunchKernelGGL(ColumnSumsKernel<T>, dim3((C + kWave - 1) / kWave, std::max(chunks_am, chunks_lm), 2),
                     dim3(256), 0, st, sums, C);
  hipLaunchKernelGGL(UnigramGradKernel<T>, dim3((C + 255) / 256), dim3(256), 0, st, (const T *)partial,
                     am_rows > 0 ? chunks_am : 0, (const T *)partial2, chunks_lm, unigram, d_unigram, lm_rows, C,
                     (T)am_only_scale);
  hipLaunchKernelGGL(LmOnlyGradKernel<T>, dim3(RowBlocks(lm_rows)), dim3(256), 0, st, symbols, lm_probs, lm_max,
                     lm_norm, (const T *)row_info, (const T *)d_unigram, lm_grad, lm_rows, S, C, blank,
                     (T)lm_only_scale);
  return LaunchStatus();
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

size_t k2amd_rnnt_smoothed_scratch_elements(int B, int S, int T, int C) {
  if (B <= 0 || S < 0 || T < 0 || C <= 0) return 0;
  const long long lm_rows = (long long)B * (S + 1), am_rows = (long long)B * T;
  return std::max(ForwardScratch(lm_rows, C), BackwardScratch(lm_rows, am_rows, C));
}

int k2amd_rnnt_smoothed_supported(int B, int S, int T, int C, int dtype) {
  return B >= 0 && S >= 0 && T >= 0 && C > 0 && (dtype == K2AMD_F32 || dtype == K2AMD_F64) && Served(B, S, T, C);
}

int k2amd_rnnt_smoothed_forward(const void *lm, const void *am, const int64_t *symbols, const int64_t *boundary,
                                const void *lm_probs, const void *am_probs, const void *lm_max,
                                const void *am_max, const void *px_joint, const void *py_joint, void *px,
                                void *py, void *lm_norm, void *am_norm, void *unigram, void *scratch,
                                size_t scratch_elements, double lm_only_scale, double am_only_scale, int B,
                                int S, int T, int C, int termination_symbol, int rnnt_type, int dtype,
                                void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (!Served(B, S, T, C)) return K2AMD_ERR_UNSUPPORTED;
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
  if (!Served(B, S, T, C)) return K2AMD_ERR_UNSUPPORTED;
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
