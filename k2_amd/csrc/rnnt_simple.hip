// get_rnnt_logprobs for the "simple" joiner (am + lm), forward and backward
// (k2/python/k2/rnnt_loss.py:65-225).
//
// Forward:  row maxima + exponentials of am and lm (one wavefront per row), then a batched
// [S+1 x C] * [C x T] product (LDS-tiled 64x64, fp32 on the matrix cores) whose epilogue takes
// the log, adds the maxima back and emits
// px / py directly, so the normaliser never makes a round trip through HBM as a separate tensor
// apart from the `denom` buffer kept for the backward.
// Backward: one pass over dpx, dpy writes Q = (dpx + dpy) / denom and their sums along s and t;
// two more batched products (Q * am_probs, Q^T * lm_probs) scaled by the saved exponentials,
// whose epilogues add the gathered terms (symbol and termination columns) from those sums.
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

// probs[row][c] = exp(x[row][c] - max_c x[row][c]); one wavefront per row.  Rows of lm first, then
// rows of am, in one launch.
template <typename T>
__global__ __launch_bounds__(256) void RowMaxExpKernel(const T *__restrict__ lm,
                                                       T *__restrict__ lm_probs,
                                                       T *__restrict__ lm_max, long long lm_rows,
                                                       const T *__restrict__ am,
                                                       T *__restrict__ am_probs,
                                                       T *__restrict__ am_max, long long am_rows,
                                                       int C) {
  const int lane = threadIdx.x & (kWave - 1);
  long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const T *x = lm;
  T *probs = lm_probs, *row_max = lm_max;
  if (row >= lm_rows) {
    row -= lm_rows;
    if (row >= am_rows) return;
    x = am; probs = am_probs; row_max = am_max;
  }
  const T *xr = x + (size_t)row * C;
  T *pr = probs + (size_t)row * C;
  constexpr int kRegs = 8;
  if (C <= kWave * kRegs) {  // the row stays in registers between the two passes
    T v[kRegs];
    T m = Real<T>::NegInf();
#pragma unroll
    for (int i = 0; i < kRegs; ++i) {
      const int c = lane + i * kWave;
      v[i] = c < C ? xr[c] : Real<T>::NegInf();
      m = max(m, v[i]);
    }
    m = WaveMaxS(m);
    if (lane == 0) row_max[row] = m;
#pragma unroll
    for (int i = 0; i < kRegs; ++i) {
      const int c = lane + i * kWave;
      if (c < C) pr[c] = Real<T>::Exp(v[i] - m);
    }
    return;
  }
  T m = Real<T>::NegInf();
  for (int c = lane; c < C; c += kWave) m = max(m, xr[c]);
  m = WaveMaxS(m);
  if (lane == 0) row_max[row] = m;
  for (int c = lane; c < C; c += kWave) pr[c] = Real<T>::Exp(xr[c] - m);
}

// ---- batched product  acc[b][m][n] = sum_k A[b](m,k) * Bm[b](k,n)  with element strides --------
struct MatView {
  size_t batch;  // elements between consecutive b
  int row, col;  // strides of the (m or k) and (k or n) index
};

constexpr int kTile = 64, kTileK = 16, kPad = 4;
// LDS scratch an epilogue may ask for (see AmGradEpilogue): per tile column a count and up to
// kMaxHits entries
constexpr int kStageColumns = 64, kMaxHits = 4;
constexpr int kStageInts = kStageColumns * (1 + kMaxHits);

// What an epilogue loads for a thread's elements (all in one column n, rows `rows`, clamped into
// the matrix by the caller), in rounds so that the loads of one round are in flight together: the
// compiler cannot move a load across a store that might alias it or out of a branch, and one
// dependent round trip per element is what a tile's epilogue would otherwise cost.
//   pre[r] = epi.Prepare(b, m, n, column)            what every element loads
//   for k < Epilogue::kLevels: if any element of the wavefront has epi.Wants(k, column, pre[r]):
//       epi.Extra(k, b, m, n, column, pre[r])         for every element; loads without branches
//                                                    (from clamped addresses), values by select
template <typename Epilogue, int R>
__device__ __forceinline__ void PrepareElements(const Epilogue &epi, int b, const int (&rows)[R],
                                                int n, const typename Epilogue::ColumnData &column,
                                                typename Epilogue::ElementData (&pre)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) pre[r] = epi.Prepare(b, rows[r], n, column);
  if constexpr (Epilogue::kLevels > 0) {
#pragma unroll
    for (int k = 0; k < Epilogue::kLevels; ++k) {
      bool wanted = false;
#pragma unroll
      for (int r = 0; r < R; ++r) wanted |= epi.Wants(k, column, pre[r]);
      if (!__any(wanted)) continue;
#pragma unroll
      for (int r = 0; r < R; ++r) epi.Extra(k, b, rows[r], n, column, pre[r]);
    }
  }
}

// fp64: one 64 x 64 output tile per workgroup, K in steps of 16 staged through LDS as As[k][m],
// Bs[k][n] (scalar, bounds-checked loads: any stride works), 16 x 16 threads with 4 x 4 outputs
// each on the vector ALUs.
//
template <typename T, typename Epilogue>
__global__ __launch_bounds__(256) void BatchedProductKernel(const T *__restrict__ A, MatView av,
                                                            const T *__restrict__ Bm, MatView bv,
                                                            int M, int N, int K, Epilogue epi) {
  __shared__ T As[kTileK][kTile + kPad];
  __shared__ T Bs[kTileK][kTile + kPad];
  __shared__ int stage[kStageInts];
  const int b = blockIdx.z;
  const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  const T *Ab = A + (size_t)b * av.batch;
  const T *Bb = Bm + (size_t)b * bv.batch;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
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
  if constexpr (Epilogue::kStaged) epi.Stage(b, n0, kTile, stage);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + tx * 4 + j;
    if (n >= N) continue;
    const auto column = epi.Column(b, n, n - n0, stage);
    typename Epilogue::ElementData pre[4];
    int rows[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) rows[i] = min(m0 + ty * 4 + i, M - 1);
    PrepareElements(epi, b, rows, n, column, pre);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + ty * 4 + i;
      if (m < M) epi.Finish(b, m, n, acc[i][j], column, pre[i]);
    }
  }
}

// fp32: the same product on the matrix cores (this batched product is the one dense contraction
// of the path: the reference's torch.matmul, k2/python/k2/rnnt_loss.py:178), full fp32 products
// and sums with v_mfma_f32_32x32x2_f32.
//
// One 32 x 32 output tile per workgroup; its four wavefronts split K into four contiguous
// ranges, multiply straight out of registers (no LDS staging, no barrier in the loop, loads
// several steps ahead of their use) and add their partial tiles through LDS at the end.  In
// step j of a 16-wide k chunk a lane feeds row (lane % 32) of A and column (lane % 32) of B at
// k = 8 (lane / 32) + j; it ends up holding column (lane % 32) of the tile at rows
// 8 (r / 4) + 4 (lane / 32) + r % 4, r = 0..15.  Rows and columns past the edge are read from a
// clamped address: what they produce stays in outputs that are never written.
typedef float Acc16 __attribute__((ext_vector_type(16)));
constexpr int kMfmaTile = 32, kChunk = 16, kAhead = 4;

// One lane's view of an operand: element (k) of its row (A) or column (B).  kWide: k is the
// contiguous axis and every row starts 16-byte aligned, so eight k's are two 16-byte loads;
// otherwise eight scalar loads kstride elements apart (coalesced across the lanes when the
// contiguous axis is m / n).
template <bool kWide>
struct LaneOperand {
  const float *p;  // row / column start
  int kstride;     // elements between consecutive k
  __device__ __forceinline__ void Full(int k, float (&r)[8]) const {  // k .. k+7 all < K
    if (kWide) {
      const float4 u = *reinterpret_cast<const float4 *>(p + k);
      const float4 v = *reinterpret_cast<const float4 *>(p + k + 4);
      r[0] = u.x; r[1] = u.y; r[2] = u.z; r[3] = u.w; r[4] = v.x; r[5] = v.y; r[6] = v.z; r[7] = v.w;
    } else {
      const float *q = p + (size_t)k * kstride;
#pragma unroll
      for (int j = 0; j < 8; ++j) r[j] = q[(size_t)j * kstride];
    }
  }
  // the last, partial chunk: addresses clamped to K-1, values past K read as zero
  __device__ __forceinline__ void Ragged(int k, int K, float (&r)[8]) const {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = p[(size_t)min(k + j, K - 1) * kstride];
      r[j] = k + j < K ? v : 0.f;
    }
  }
};

// Small products (too few 64 x 64 tiles to fill the chip): one 32 x 32 tile per workgroup, K split
// over its four wavefronts, operands straight from global memory into registers.
// Workgroups are numbered so that those resident on one XCD (dispatch is round-robin over the
// eight XCDs) work on neighbouring tiles of the same batch elements and share them in that L2.
// The loop over full chunks is free of branches: chunk c + kAhead is requested while chunk c is
// multiplied, with the chunk index clamped at the end of the range instead of tested.
template <bool kAWide, bool kBWide, typename Epilogue>
__global__ __launch_bounds__(256) void ProductSplitKKernel(const float *__restrict__ A, MatView av,
                                                         const float *__restrict__ Bm, MatView bv,
                                                         int M, int N, int K, int tiles_n,
                                                         int tiles_m, int total, Epilogue epi) {
  __shared__ float part[4][kMfmaTile][kMfmaTile + 1];
  __shared__ int stage[kStageInts];
  const int per_xcd = (total + 7) / 8;
  const int id = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (id >= total) return;
  const int b = id / (tiles_n * tiles_m);
  const int tile = id - b * tiles_n * tiles_m;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 31, half = lane >> 5;
  const int m0 = (tile / tiles_n) * kMfmaTile, n0 = (tile % tiles_n) * kMfmaTile;
  LaneOperand<kAWide> oa;
  LaneOperand<kBWide> ob;
  oa.p = A + (size_t)b * av.batch + (size_t)min(m0 + col, M - 1) * av.row;
  oa.kstride = av.col;
  ob.p = Bm + (size_t)b * bv.batch + (size_t)min(n0 + col, N - 1) * bv.col;
  ob.kstride = bv.row;
  const int full = K / kChunk;  // chunks with all 16 k's
  const int per_wave = (full + 3) / 4;
  const int c_begin = min(wave * per_wave, full);
  const int c_end = min(c_begin + per_wave, full);
  Acc16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0;
  float ra[kAhead][8], rb[kAhead][8];
  const int c_last = c_end - 1;
  if (c_begin < c_end) {
#pragma unroll
    for (int d = 0; d < kAhead; ++d) {
      const int k = min(c_begin + d, c_last) * kChunk + half * 8;
      oa.Full(k, ra[d]);
      ob.Full(k, rb[d]);
    }
  }
  // (here: what the staging waits for is covered by the operands' first loads)
  if constexpr (Epilogue::kStaged) epi.Stage(b, n0, kMfmaTile, stage);
  if (c_begin < c_end) {
    int c = c_begin;
    for (; c + kAhead <= c_end; c += kAhead) {
#pragma unroll
      for (int d = 0; d < kAhead; ++d) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[d][j], rb[d][j], acc, 0, 0, 0);
        // keep the request for chunk c + d + kAhead here, between the multiplies of two chunks
        // (left to itself the scheduler gathers all requests at the end of the loop body, which
        // leaves nothing in flight across the back edge)
        __builtin_amdgcn_sched_barrier(0);
        const int k = min(c + d + kAhead, c_last) * kChunk + half * 8;
        oa.Full(k, ra[d]);
        ob.Full(k, rb[d]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int d = 0; d < kAhead - 1; ++d) {  // what is left of the range: fewer than kAhead chunks
      if (c + d < c_end) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[d][j], rb[d][j], acc, 0, 0, 0);
      }
    }
  }
  if (full * kChunk < K && wave == 3) {  // the partial chunk at the end of K
    float ta[8], tb[8];
    const int k = full * kChunk + half * 8;
    oa.Ragged(k, K, ta);
    ob.Ragged(k, K, tb);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ta[j], tb[j], acc, 0, 0, 0);
  }
  const int n = n0 + col;
  // add the four partial tiles: wave w finishes rows 8 w .. 8 w + 7
#pragma unroll
  for (int r = 0; r < 16; ++r) part[wave][(r >> 2) * 8 + half * 4 + (r & 3)][col] = acc[r];
  __syncthreads();
  if (n >= N) return;
  const auto column = epi.Column(b, n, col, stage);
  typename Epilogue::ElementData pre[4];
  int rows[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) rows[r] = min(m0 + wave * 8 + half * 4 + r, M - 1);
  PrepareElements(epi, b, rows, n, column, pre);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = wave * 8 + half * 4 + r;
    const int m = m0 + row;
    if (m < M)
      epi.Finish(b, m, n,
                 (part[0][row][col] + part[1][row][col]) + (part[2][row][col] + part[3][row][col]),
                 column, pre[r]);
  }
}

// ---- large products: 64 x 64 tile per workgroup, operands staged through LDS -----------------
//
// K in steps of 32 through a double-buffered LDS tile As[k][m], Bs[k][n]: each element of the
// operands is read from global memory once per workgroup, as whole 128-byte lines where the
// layout allows 16-byte loads, and the requests for step c + 2 are in flight while step c is
// multiplied (the barrier below does not wait for them).  Each wavefront multiplies a 32 x 32
// quadrant; in step j of a chunk a lane feeds k = 16 (lane / 32) + j.
// Rows of 66 floats: the four k rows a wavefront parks at once, and the two halves of a wavefront
// reading rows 16 apart, then fall on different LDS banks.
constexpr int kKc = 32, kLdsRow = kTile + 2;

__device__ __forceinline__ void LdsOnlyBarrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Two groups of four consecutive elements per thread along the operand's contiguous axis
// (kKFast: that axis is k, else it is m / n).  kWide: the rows allow 16-byte loads and their
// length is a multiple of four, so a group is inside or outside as a whole.  Loads are free of
// branches: addresses are clamped into the operand, what lies outside reads as zero.
template <bool kKFast, bool kWide>
struct QuadStager {
  const float *base;      // operand of this batch element
  int lead[2], other[2];  // first index along the contiguous axis / index along the other axis
  int lead_n, other_n;    // extents
  int other_stride;       // elements between consecutive `other`
  int mn0;
  bool inside[2][4];      // of the values last fetched: which lie inside the operand
  __device__ void Init(const float *p, int mn0_, int MN, int K, int stride, int tid) {
    base = p; other_stride = stride; mn0 = mn0_;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = tid + 256 * i;
      if (kKFast) { lead[i] = (q & 7) * 4; other[i] = mn0 + (q >> 3); }
      else        { lead[i] = mn0 + (q & 15) * 4; other[i] = q >> 4; }
    }
    lead_n = kKFast ? K : MN;
    other_n = kKFast ? MN : K;
  }
  // Requests only: nothing here waits for the values (Park applies `inside`).
  __device__ __forceinline__ void Fetch(int k0, float (&r)[2][4]) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int l = lead[i] + (kKFast ? k0 : 0), o = other[i] + (kKFast ? 0 : k0);
      const float *row = base + (size_t)min(o, other_n - 1) * other_stride;
      if (kWide) {
        const float4 v = *reinterpret_cast<const float4 *>(row + min(l, lead_n - 4));
        r[i][0] = v.x; r[i][1] = v.y; r[i][2] = v.z; r[i][3] = v.w;
#pragma unroll
        for (int e = 0; e < 4; ++e) inside[i][e] = o < other_n && l < lead_n;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          r[i][e] = row[min(l + e, lead_n - 1)];
          inside[i][e] = o < other_n && l + e < lead_n;
        }
      }
    }
  }
  __device__ __forceinline__ void Park(float (*tile)[kLdsRow], const float (&r)[2][4]) const {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = inside[i][e] ? r[i][e] : 0.f;
      if (kKFast) {
#pragma unroll
        for (int e = 0; e < 4; ++e) tile[lead[i] + e][other[i] - mn0] = v[e];
      } else {
        float2 *dst = reinterpret_cast<float2 *>(&tile[other[i]][lead[i] - mn0]);  // rows are 8-byte aligned
        dst[0] = make_float2(v[0], v[1]);
        dst[1] = make_float2(v[2], v[3]);
      }
    }
  }
};

template <bool kAKFast, bool kAWide, bool kBKFast, bool kBWide, typename Epilogue>
__global__ __launch_bounds__(256) void ProductLdsKernel(const float *__restrict__ A, MatView av,
                                                        const float *__restrict__ Bm, MatView bv,
                                                        int M, int N, int K, int tiles_n,
                                                        int tiles_m, int total, Epilogue epi) {
  __shared__ __attribute__((aligned(16))) float As[2][kKc][kLdsRow];
  __shared__ __attribute__((aligned(16))) float Bs[2][kKc][kLdsRow];
  __shared__ int stage[kStageInts];
  const int per_xcd = (total + 7) / 8;
  const int id = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (id >= total) return;
  const int b = id / (tiles_n * tiles_m);
  const int tile = id - b * tiles_n * tiles_m;
  const int m0 = (tile / tiles_n) * kTile, n0 = (tile % tiles_n) * kTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 31, half = lane >> 5;
  const int qm = (wave >> 1) * kMfmaTile, qn = (wave & 1) * kMfmaTile;
  QuadStager<kAKFast, kAWide> sa;
  QuadStager<kBKFast, kBWide> sb;
  sa.Init(A + (size_t)b * av.batch, m0, M, K, kAKFast ? av.row : av.col, threadIdx.x);
  sb.Init(Bm + (size_t)b * bv.batch, n0, N, K, kBKFast ? bv.col : bv.row, threadIdx.x);
  Acc16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0;
  const int chunks = (K + kKc - 1) / kKc;
  float ra[2][4], rb[2][4];
  float fa[2][kKc / 2], fb[2][kKc / 2];  // the lane's operands of the current and the next chunk
  auto read_fragments = [&](int buf, float (&a)[kKc / 2], float (&bb)[kKc / 2]) {
#pragma unroll
    for (int j = 0; j < kKc / 2; ++j) {
      a[j] = As[buf][half * (kKc / 2) + j][qm + col];
      bb[j] = Bs[buf][half * (kKc / 2) + j][qn + col];
    }
  };
  // One chunk: its operands are in registers already.  The first multiplies cover the parking of
  // chunk c + 1 and the barrier, the rest cover the LDS reads of chunk c + 1 and the requests for
  // chunk c + 2, so the matrix pipeline only idles while wavefronts wait for one another.
  auto chunk = [&](int c, float (&a)[kKc / 2], float (&bb)[kKc / 2], float (&na)[kKc / 2],
                   float (&nb)[kKc / 2]) {
    constexpr int kEarly = 4;
#pragma unroll
    for (int j = 0; j < kEarly; ++j)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bb[j], acc, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    sa.Park(As[(c + 1) & 1], ra);  // zeros past K
    sb.Park(Bs[(c + 1) & 1], rb);
    LdsOnlyBarrier();
    __builtin_amdgcn_sched_barrier(0);
    sa.Fetch((c + 2) * kKc, ra);
    sb.Fetch((c + 2) * kKc, rb);
    read_fragments((c + 1) & 1, na, nb);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = kEarly; j < kKc / 2; ++j)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bb[j], acc, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  sa.Fetch(0, ra);
  sb.Fetch(0, rb);
  // (here: what the staging waits for is covered by the operands' first loads)
  if constexpr (Epilogue::kStaged) epi.Stage(b, n0, kTile, stage);
  sa.Park(As[0], ra);
  sb.Park(Bs[0], rb);
  sa.Fetch(kKc, ra);
  sb.Fetch(kKc, rb);
  LdsOnlyBarrier();
  read_fragments(0, fa[0], fb[0]);
  for (int c = 0; c < chunks; c += 2) {
    chunk(c, fa[0], fb[0], fa[1], fb[1]);
    if (c + 1 < chunks) chunk(c + 1, fa[1], fb[1], fa[0], fb[0]);
  }
  const int n = n0 + qn + col;
  if (n >= N) return;
  const auto column = epi.Column(b, n, qn + col, stage);
  typename Epilogue::ElementData pre[16];
  int rows[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) rows[r] = min(m0 + qm + (r >> 2) * 8 + half * 4 + (r & 3), M - 1);
  PrepareElements(epi, b, rows, n, column, pre);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + qm + (r >> 2) * 8 + half * 4 + (r & 3);
    if (m < M) epi.Finish(b, m, n, acc[r], column, pre[r]);
  }
}

// 16-byte loads along an operand's contiguous axis: rows a multiple of four long and dense,
// every batch element aligned.
inline bool WideAlongRows(const float *p, int stride, int row_len, size_t batch) {
  return stride % 4 == 0 && row_len % 4 == 0 && row_len >= 4 && batch % 4 == 0 &&
         reinterpret_cast<size_t>(p) % 16 == 0;
}

template <bool kAKFast, bool kBKFast, typename Epilogue>
void LaunchLds(const float *A, MatView av, const float *Bm, MatView bv, int M, int N, int K, int B,
               Epilogue epi, hipStream_t st) {
  const int tn = (N + kTile - 1) / kTile, tm = (M + kTile - 1) / kTile, total = tn * tm * B;
  const dim3 grid(((total + 7) / 8) * 8), block(256);
  const bool aw = WideAlongRows(A, kAKFast ? av.row : av.col, kAKFast ? K : M, av.batch);
  const bool bw = WideAlongRows(Bm, kBKFast ? bv.col : bv.row, kBKFast ? K : N, bv.batch);
#define K2AMD_LAUNCH_LDS(AW, BW)                                                                  \
  hipLaunchKernelGGL((ProductLdsKernel<kAKFast, AW, kBKFast, BW, Epilogue>), grid, block, 0, st, A, \
                     av, Bm, bv, M, N, K, tn, tm, total, epi)
  if (aw && bw) K2AMD_LAUNCH_LDS(true, true);
  else if (aw) K2AMD_LAUNCH_LDS(true, false);
  else if (bw) K2AMD_LAUNCH_LDS(false, true);
  else K2AMD_LAUNCH_LDS(false, false);
#undef K2AMD_LAUNCH_LDS
}

template <typename Epilogue>
void LaunchSplitK(const float *A, MatView av, const float *Bm, MatView bv, int M, int N, int K, int B,
                Epilogue epi, hipStream_t st) {
  const int tn = (N + kMfmaTile - 1) / kMfmaTile, tm = (M + kMfmaTile - 1) / kMfmaTile;
  const int total = tn * tm * B;
  const dim3 grid(((total + 7) / 8) * 8), block(256);
  // 16-byte loads along k: k contiguous, rows a multiple of four long, every batch element aligned
  const bool a_wide = av.col == 1 && av.row % 4 == 0 && av.batch % 4 == 0 &&
                      reinterpret_cast<size_t>(A) % 16 == 0;
  const bool b_wide = bv.row == 1 && bv.col % 4 == 0 && bv.batch % 4 == 0 &&
                      reinterpret_cast<size_t>(Bm) % 16 == 0;
  if (a_wide && b_wide)
    hipLaunchKernelGGL((ProductSplitKKernel<true, true, Epilogue>), grid, block, 0, st, A, av, Bm, bv, M, N, K, tn, tm, total, epi);
  else if (a_wide)
    hipLaunchKernelGGL((ProductSplitKKernel<true, false, Epilogue>), grid, block, 0, st, A, av, Bm, bv, M, N, K, tn, tm, total, epi);
  else if (b_wide)
    hipLaunchKernelGGL((ProductSplitKKernel<false, true, Epilogue>), grid, block, 0, st, A, av, Bm, bv, M, N, K, tn, tm, total, epi);
  else
    hipLaunchKernelGGL((ProductSplitKKernel<false, false, Epilogue>), grid, block, 0, st, A, av, Bm, bv, M, N, K, tn, tm, total, epi);
}

// Picks the kernel by element type and, for fp32, by size.  kAKFast / kBKFast: the contiguous
// axis of A(m,k) / B(k,n) is k (the caller's MatView says the same: av.col == 1 / bv.row == 1).
template <typename T, bool kAKFast, bool kBKFast, typename Epilogue>
void LaunchProduct(const T *A, MatView av, const T *Bm, MatView bv, int M, int N, int K, int B,
                   Epilogue epi, hipStream_t st) {
  if (M <= 0 || N <= 0 || B <= 0) return;
  if constexpr (sizeof(T) == 4) {
    const long long big_tiles = (long long)((N + 63) / 64) * ((M + 63) / 64) * B;
    // The 64 x 64 tiles once they give every compute unit two workgroups; four where K is short:
    // the operands then matter little and a 32 x 32 tile's epilogue is a quarter as long per thread
    // (B=16 T=250 S=50 C=500, the am gradient, K = 51: 15.4 us against 18.4 us).
    if (big_tiles >= (K <= 128 ? 1024 : 512))
      LaunchLds<kAKFast, kBKFast>(A, av, Bm, bv, M, N, K, B, epi, st);
    else
      LaunchSplitK(A, av, Bm, bv, M, N, K, B, epi, st);
  } else {
    dim3 grid((N + kTile - 1) / kTile, (M + kTile - 1) / kTile, B);
    hipLaunchKernelGGL((BatchedProductKernel<T, Epilogue>), grid, dim3(256), 0, st, A, av, Bm, bv, M, N, K, epi);
  }
}

template <typename T>
struct Tiny;
template <>
struct Tiny<float> { static constexpr float v = 1.17549435e-38f; };   // torch.finfo(float32).tiny
template <>
struct Tiny<double> { static constexpr double v = 2.2250738585072014e-308; };

// Effective gradients of the un-fixed px / py values at (b,s,t), t < T.
template <typename T>
struct GradView {
  const T *px_grad, *py_grad;
  const T *seq_scale;  // what reaches sequence b's score multiplies its gradients (null: 1)
  const int64_t *boundary;
  int S, Tn, rnnt_type;
  __device__ __forceinline__ T Scale(int b) const { return seq_scale != nullptr ? seq_scale[b] : T(1); }
  __device__ __forceinline__ T Gx(int b, int s, int t) const {
    if (s >= S) return 0;
    if (rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t) return 0;
    const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
    return MulRounded(px_grad[((size_t)b * S + s) * T1 + t], Scale(b));
  }
  __device__ __forceinline__ T Gy(int b, int s, int t) const {
    T g = MulRounded(py_grad[((size_t)b * (S + 1) + s) * Tn + t], Scale(b));
    if (rnnt_type == K2AMD_CONSTRAINED && s >= 1) g += Gx(b, s - 1, t);
    return g;
  }
};

// Epilogues work in steps so that a thread can issue the loads of all its elements before the
// first store (see PrepareElements):
//   epi.Stage(b, n0, width, scratch)          (only if Epilogue::kStaged; whole workgroup, has
//                                              barriers) what depends on the tile's columns
//   column = epi.Column(b, n, n - n0, scratch)   what depends on (b, n) only
//   PrepareElements: epi.Prepare, then epi.Wants / epi.Extra for Epilogue::kLevels rounds
//   epi.Finish(b, m, n, acc, column, pre)        arithmetic and stores

// Forward epilogue: (m, n) = (s, t).  Also writes the -inf column px[b,s,T] of a regular lattice
// (k2/python/k2/rnnt_loss.py:193-205) from the threads that hold t = T-1.
template <typename T>
struct ForwardEpilogue {
  const T *lm, *am, *lm_max, *am_max;
  const int64_t *symbols, *boundary;
  T *px, *py, *denom;
  int S, Tn, C, blank, rnnt_type;
  struct ColumnData {
    const T *amr;
    T am_max, am_blank;
    bool cut;  // regular lattice: px[b, :, t_end] = -inf (k2/python/k2/rnnt_loss.py:25-43)
  };
  struct ElementData {
    T lm_max, lm_blank, sym_sum;  // sym_sum = am[b,t,sym] + lm[b,s,sym], -inf without a symbol
  };
  static constexpr bool kStaged = false;
  static constexpr int kLevels = 0;
  __device__ __forceinline__ ColumnData Column(int b, int t, int, const int *) const {
    ColumnData c;
    c.amr = am + ((size_t)b * Tn + t) * C;
    c.am_max = am_max[(size_t)b * Tn + t];
    c.am_blank = c.amr[blank];
    c.cut = rnnt_type == K2AMD_REGULAR && boundary != nullptr && boundary[4 * b + 3] == t;
    return c;
  }
  __device__ __forceinline__ ElementData Prepare(int b, int s, int, const ColumnData &c) const {
    ElementData e;
    const size_t row = (size_t)b * (S + 1) + s;
    const T *lmr = lm + row * C;
    e.lm_max = lm_max[row];
    e.lm_blank = lmr[blank];
    e.sym_sum = Real<T>::NegInf();
    if (s < S) {
      const int64_t sym = symbols[(size_t)b * S + s];
      if (sym >= 0 && sym < C) e.sym_sum = c.amr[sym] + lmr[sym];
    }
    return e;
  }
  __device__ __forceinline__ void Finish(int b, int s, int t, T acc, const ColumnData &c,
                                         const ElementData &e) const {
    const size_t row = (size_t)b * (S + 1) + s;
    const T d = acc + Tiny<T>::v;
    denom[row * Tn + t] = d;
    const T norm = (Real<T>::Log(d) + e.lm_max) + c.am_max;
    py[row * Tn + t] = (c.am_blank + e.lm_blank) - norm;
    if (s < S) {
      const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
      T *pxr = px + ((size_t)b * S + s) * T1;
      pxr[t] = c.cut ? Real<T>::NegInf() : e.sym_sum - norm;
      if (rnnt_type == K2AMD_REGULAR && t == Tn - 1) pxr[Tn] = Real<T>::NegInf();
    }
  }
};

// Epilogue of the lm gradient, (m, n) = (s, c):
//   lm_grad[b,s,c] = -lm_probs[b,s,c] * acc + (c == symbols[b,s]) * sum_t Gx(b,s,t)
//                    + (c == blank) * sum_t Gy(b,s,t).
// The two sums come from QSumsKernel as one value per chunk of t and are added here in the order
// of the chunks.
template <typename T>
struct LmGradEpilogue {
  const T *scale;  // lm_probs
  T *out;
  const int64_t *symbols;
  const T *row_x, *row_y;  // [B][S+1][chunks]
  int S, N, chunks, blank;
  struct ColumnData {};
  struct ElementData {
    T scale, sum_x, sum_y;
    bool takes_x, takes_y;
  };
  static constexpr bool kStaged = false;
  static constexpr int kLevels = 1;
  __device__ __forceinline__ ColumnData Column(int, int, int, const int *) const { return ColumnData(); }
  __device__ __forceinline__ ElementData Prepare(int b, int s, int c, const ColumnData &) const {
    ElementData e;
    e.scale = scale[((size_t)b * (S + 1) + s) * N + c];
    e.sum_x = e.sum_y = 0;
    const int64_t sym = S > 0 ? symbols[(size_t)b * S + min(s, S - 1)] : -1;
    e.takes_x = s < S && sym == c;
    e.takes_y = c == blank;
    return e;
  }
  __device__ __forceinline__ bool Wants(int, const ColumnData &, const ElementData &e) const {
    return e.takes_x || e.takes_y;
  }
  __device__ __forceinline__ void Extra(int, int b, int s, int, const ColumnData &, ElementData &e) const {
    const size_t first = ((size_t)b * (S + 1) + s) * chunks;
    T sx = 0, sy = 0;
    for (int k = 0; k < chunks; ++k) {
      sx += row_x[first + k];
      sy += row_y[first + k];
    }
    e.sum_x = e.takes_x ? sx : T(0);
    e.sum_y = e.takes_y ? sy : T(0);
  }
  __device__ __forceinline__ void Finish(int b, int s, int c, T acc, const ColumnData &,
                                         const ElementData &e) const {
    out[((size_t)b * (S + 1) + s) * N + c] = (-e.scale * acc + e.sum_x) + e.sum_y;
  }
};

// Epilogue of the am gradient, (m, n) = (t, c):
//   am_grad[b,t,c] = -am_probs[b,t,c] * acc + sum over s with symbols[b,s] == c of Gx(b,s,t)
//                    + (c == blank) * sum over s of Gy(b,s,t)
// (the latter from QSumsKernel as one value per group of rows s, added here in the groups' order).
// Stage lists, for each of the tile's columns, the positions s whose symbol is that column (up
// to kMaxHits, sorted; longer lists are rescanned per element), so that the symbol terms cost a
// tile one pass over the sequence's symbols instead of a launch of their own.  The terms of an
// element are added in the order of s: the result does not depend on scheduling.
template <typename T>
struct AmGradEpilogue {
  static constexpr bool kStaged = true;
  const T *scale;
  T *out;
  GradView<T> gv;
  const int64_t *symbols;
  const T *col_y;  // [B][groups][Tn]
  int M, N;        // Tn, C
  int blank, groups;
  static constexpr int kLevels = kMaxHits + 1;
  struct ColumnData {
    int hits;  // positions s with symbols[b,s] == c (all of them, also beyond kMaxHits)
    int s[kMaxHits];
    T scale;          // of sequence b
    int64_t t_cut;    // regular lattice with a boundary: px_grad[b, :, t_cut] does not count
    bool is_blank;
  };
  struct ElementData { T scale, sym_sum; };
  __device__ void Stage(int b, int n0, int width, int *scratch) const {
    int *count = scratch, *hit = scratch + kStageColumns;
    for (int i = threadIdx.x; i < kStageColumns; i += blockDim.x) count[i] = 0;
    __syncthreads();
    const int64_t *sym = symbols + (size_t)b * gv.S;
    for (int s = threadIdx.x; s < gv.S; s += blockDim.x) {
      const int64_t c = sym[s] - n0;
      if (c >= 0 && c < width) {
        const int slot = atomicAdd(&count[c], 1);
        if (slot < kMaxHits) hit[c * kMaxHits + slot] = s;
      }
    }
    __syncthreads();
    if (threadIdx.x < kStageColumns) {  // ascending s, whatever order the slots were claimed in
      int *h = hit + threadIdx.x * kMaxHits;
      const int n = min(count[threadIdx.x], kMaxHits);
      for (int i = 1; i < n; ++i) {
        const int v = h[i];
        int j = i - 1;
        for (; j >= 0 && h[j] > v; --j) h[j + 1] = h[j];
        h[j + 1] = v;
      }
    }
    __syncthreads();
  }
  __device__ __forceinline__ ColumnData Column(int b, int c, int local, const int *scratch) const {
    ColumnData col;
    col.is_blank = c == blank;
    col.hits = scratch[local];
#pragma unroll
    for (int k = 0; k < kMaxHits; ++k) col.s[k] = scratch[kStageColumns + local * kMaxHits + k];
    col.scale = gv.Scale(b);
    col.t_cut = gv.rnnt_type == K2AMD_REGULAR && gv.boundary != nullptr ? gv.boundary[4 * b + 3] : -1;
    return col;
  }
  __device__ __forceinline__ ElementData Prepare(int b, int t, int c, const ColumnData &) const {
    return ElementData{scale[((size_t)b * M + t) * N + c], T(0)};
  }
  // Rounds 0 .. kMaxHits-1: the column's k-th position s; the last round: the blank column's sums.
  __device__ __forceinline__ bool Wants(int k, const ColumnData &col, const ElementData &) const {
    return k < kMaxHits ? k < col.hits : col.is_blank;
  }
  __device__ __forceinline__ void Extra(int k, int b, int t, int c, const ColumnData &col,
                                        ElementData &e) const {
    if (k == kMaxHits) {
      T sum = 0;
      for (int g = 0; g < groups; ++g) sum += col_y[((size_t)b * groups + g) * M + t];
      if (col.is_blank) e.sym_sum += sum;
      return;
    }
    if (col.hits <= kMaxHits) {
      // Gx(b, s, t) of GradView, the load from position 0 where this column has no k-th position
      // (a round only runs where some column has one, so S > 0)
      const bool mine = k < col.hits;
      const int T1 = gv.rnnt_type == K2AMD_REGULAR ? gv.Tn + 1 : gv.Tn;
      const T raw = gv.px_grad[((size_t)b * gv.S + (mine ? col.s[k] : 0)) * T1 + t];
      const T g = MulRounded(raw, col.scale);
      if (mine && t != col.t_cut) e.sym_sum += g;
    } else if (k == 0) {  // a longer list: every position of the sequence, in order
      const int64_t *sym = symbols + (size_t)b * gv.S;
      for (int s = 0; s < gv.S; ++s)
        if (sym[s] == c) e.sym_sum += gv.Gx(b, s, t);
    }
  }
  __device__ __forceinline__ void Finish(int b, int t, int c, T acc, const ColumnData &,
                                         const ElementData &e) const {
    out[((size_t)b * M + t) * N + c] = -e.scale * acc + e.sym_sum;
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

// One pass over the lattice's gradients for the whole backward:
//   q[b,s,t] = (Gx + Gy) / denom                   the A operand of the two products
//   col_y[b,g,t] = sum of Gy(b,s,t) over group g's kSumsGroup rows s
//                                                  the termination terms of the am gradient
//   row_x / row_y[b,s,chunk] = sum of Gx / Gy over the chunk's kSumsChunk values of t
//                                                  the gathered terms of the lm gradient
// One workgroup per (chunk of t, group of s, b); each of its four wavefronts takes kSumsRows
// consecutive rows and requests all it reads at once, from addresses clamped into the tensors
// (one round trip to memory instead of one per row).  The consumers add the groups / chunks in
// order, and every sum here is added in a fixed order: no result depends on scheduling.
constexpr int kSumsChunk = 64, kSumsRows = 8, kSumsGroup = 4 * kSumsRows;

inline int SumsChunks(int Tn) { return (Tn + kSumsChunk - 1) / kSumsChunk; }
inline int SumsGroups(int S) { return (S + kSumsGroup) / kSumsGroup; }  // of the S + 1 rows

// Sums each of a lane's 2^kLog values over the wavefront.  Every step halves the values a lane
// still carries (it hands the other half to the lane it pairs with), so the 2^kLog sums cost
// 2^kLog - 1 + (6 - kLog) exchanges instead of 6 each.  Returns the complete sum of value
// number (lane >> (6 - kLog)), the same in every lane that shares the number.
template <typename T, int kLog>
__device__ __forceinline__ T WaveSumsTransposed(T (&v)[1 << kLog], int lane) {
  static_assert(kLog >= 1 && kLog <= 6, "");
#pragma unroll
  for (int step = 0; step < kLog; ++step) {
    const int n = (1 << kLog) >> (step + 1), off = kWave >> (step + 1);
    const bool upper = (lane & off) != 0;
#pragma unroll
    for (int i = 0; i < n; ++i) {
      const T keep = upper ? v[i + n] : v[i];
      const T send = upper ? v[i] : v[i + n];
      v[i] = keep + __shfl_xor(send, off, kWave);
    }
  }
  T r = v[0];
#pragma unroll
  for (int off = kWave >> (kLog + 1); off > 0; off >>= 1) r += __shfl_xor(r, off, kWave);
  return r;
}

template <typename T>
__global__ __launch_bounds__(256) void QSumsKernel(GradView<T> gv, const T *__restrict__ denom,
                                                   T *__restrict__ q, T *__restrict__ col_y,
                                                   T *__restrict__ row_x, T *__restrict__ row_y,
                                                   int chunks, int groups) {
  __shared__ T col[4][kSumsChunk];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int chunk = blockIdx.x, group = blockIdx.y, b = blockIdx.z;
  const int S = gv.S, Tn = gv.Tn;
  const int t = chunk * kSumsChunk + lane;
  const bool inside = t < Tn;
  const int tc = min(t, Tn - 1);
  const int s0 = group * kSumsGroup + wave * kSumsRows;
  const bool regular = gv.rnnt_type == K2AMD_REGULAR;
  const bool constrained = gv.rnnt_type == K2AMD_CONSTRAINED;
  const int T1 = regular ? Tn + 1 : Tn;
  const T scale = gv.Scale(b);
  const bool cut = regular && gv.boundary != nullptr && gv.boundary[4 * b + 3] == t;
  // rows s0 - 1 .. s0 + kSumsRows - 1 of px_grad (the first one only feeds a constrained lattice's
  // Gy), rows s0 .. of py_grad and denom
  T px_raw[kSumsRows + 1], py_raw[kSumsRows], den[kSumsRows];
#pragma unroll
  for (int j = 0; j <= kSumsRows; ++j) {
    const int s = min(max(s0 + j - 1, 0), S - 1);
    px_raw[j] = S > 0 && (j > 0 || constrained) ? gv.px_grad[((size_t)b * S + s) * T1 + tc] : T(0);
  }
#pragma unroll
  for (int j = 0; j < kSumsRows; ++j) {
    const size_t i = ((size_t)b * (S + 1) + min(s0 + j, S)) * Tn + tc;
    py_raw[j] = gv.py_grad[i];
    den[j] = denom[i];
  }
  T sums[2 * kSumsRows];  // of row j: Gx in 2 j, Gy in 2 j + 1
  T cy = 0;
  T gx_below = 0;  // Gx(b, s - 1, t)
  if (constrained && s0 >= 1 && s0 - 1 < S && inside && !cut) gx_below = MulRounded(px_raw[0], scale);
#pragma unroll
  for (int j = 0; j < kSumsRows; ++j) {
    const int s = s0 + j;
    const bool live = inside && s <= S;
    const T gx = live && s < S && !cut ? MulRounded(px_raw[j + 1], scale) : T(0);
    T gy = live ? MulRounded(py_raw[j], scale) : T(0);
    if (constrained && live && s >= 1) gy += gx_below;
    gx_below = gx;
    if (live) q[((size_t)b * (S + 1) + s) * Tn + t] = (gx + gy) / den[j];
    cy += gy;
    sums[2 * j] = gx;
    sums[2 * j + 1] = gy;
  }
  const T total = WaveSumsTransposed<T, 4>(sums, lane);
  if ((lane & 3) == 0) {
    const int which = lane >> 2, s = s0 + (which >> 1);
    if (s <= S) ((which & 1) ? row_y : row_x)[((size_t)b * (S + 1) + s) * chunks + chunk] = total;
  }
  col[wave][lane] = cy;
  __syncthreads();
  if (wave == 0 && inside)
    col_y[((size_t)b * groups + group) * Tn + t] =
        (col[0][lane] + col[1][lane]) + (col[2][lane] + col[3][lane]);
}

template <typename T>
int SimpleForward(const T *lm, const T *am, const int64_t *symbols, const int64_t *boundary, T *px,
                  T *py, T *lm_probs, T *am_probs, T *lm_max, T *am_max, T *denom, int B, int S,
                  int Tn, int C, int blank, int rnnt_type, hipStream_t st) {
  const long long lm_rows = (long long)B * (S + 1), am_rows = (long long)B * Tn;
  if (lm_rows + am_rows > 0)
    hipLaunchKernelGGL(RowMaxExpKernel<T>, dim3((unsigned)((lm_rows + am_rows + 3) / 4)), dim3(256), 0, st, lm, lm_probs, lm_max, lm_rows, am, am_probs, am_max, am_rows, C);
  const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
  if (rnnt_type == K2AMD_REGULAR && B * S > 0 && Tn == 0)  // else the product's epilogue writes it
    hipLaunchKernelGGL(LastColumnKernelS<T>, dim3((B * S + 255) / 256), dim3(256), 0, st, px, B * S, T1);
  if (B > 0 && Tn > 0) {
    ForwardEpilogue<T> epi{lm, am, lm_max, am_max, symbols, boundary, px, py, denom, S, Tn, C, blank, rnnt_type};
    MatView av{(size_t)(S + 1) * C, C, 1};  // A(m=s, k=c) = lm_probs[b][s][c]
    MatView bv{(size_t)Tn * C, 1, C};       // B(k=c, n=t) = am_probs[b][t][c]
    LaunchProduct<T, true, true>(lm_probs, av, am_probs, bv, S + 1, Tn, C, B, epi, st);
    if (rnnt_type == K2AMD_CONSTRAINED && S > 0)
      hipLaunchKernelGGL(ConstrainedKernelS<T>, dim3(512), dim3(256), 0, st, px, py, B, S, Tn);
  }
  return LaunchStatus();
}

template <typename T>
int SimpleBackward(const T *px_grad, const T *py_grad, const T *seq_scale, const int64_t *symbols,
                   const int64_t *boundary, const T *lm_probs, const T *am_probs, const T *denom,
                   T *lm_grad, T *am_grad, T *q, int B, int S, int Tn, int C, int blank,
                   int rnnt_type, hipStream_t st) {
  if (B == 0) return K2AMD_OK;
  GradView<T> gv{px_grad, py_grad, seq_scale, boundary, S, Tn, rnnt_type};
  if (Tn == 0) {  // no am rows; every term of the lm gradient is an empty sum
    hipLaunchKernelGGL(ZeroKernelS<T>, dim3(256), dim3(256), 0, st, lm_grad, (size_t)B * (S + 1) * C);
    return LaunchStatus();
  }
  const int chunks = SumsChunks(Tn), groups = SumsGroups(S);
  T *col_y = q + (size_t)B * (S + 1) * Tn;
  T *row_x = col_y + (size_t)B * groups * Tn;
  T *row_y = row_x + (size_t)B * (S + 1) * chunks;
  hipLaunchKernelGGL(QSumsKernel<T>, dim3(chunks, groups, B), dim3(256), 0, st, gv, denom, q, col_y, row_x, row_y, chunks, groups);
  {  // lm_grad[b][s][c] = -lm_probs * sum_t q[b][s][t] * am_probs[b][t][c]  (+ the gathered terms)
    LmGradEpilogue<T> epi{lm_probs, lm_grad, symbols, row_x, row_y, S, C, chunks, blank};
    MatView av{(size_t)(S + 1) * Tn, Tn, 1};  // A(m=s, k=t) = q[b][s][t]
    MatView bv{(size_t)Tn * C, C, 1};         // B(k=t, n=c) = am_probs[b][t][c]
    LaunchProduct<T, true, false>((const T *)q, av, am_probs, bv, S + 1, C, Tn, B, epi, st);
  }
  {  // am_grad[b][t][c] = -am_probs * sum_s q[b][s][t] * lm_probs[b][s][c]  (+ symbol and blank terms)
    AmGradEpilogue<T> epi{am_probs, am_grad, gv, symbols, col_y, Tn, C, blank, groups};
    MatView av{(size_t)(S + 1) * Tn, 1, Tn};   // A(m=t, k=s) = q[b][s][t]
    MatView bv{(size_t)(S + 1) * C, C, 1};     // B(k=s, n=c) = lm_probs[b][s][c]
    LaunchProduct<T, false, false>((const T *)q, av, lm_probs, bv, Tn, C, S + 1, B, epi, st);
  }
  return LaunchStatus();
}

bool ArgsOk(int B, int S, int T, int C, int blank, int rnnt_type, int dtype) {
  if (B < 0 || S < 0 || T < 0 || C <= 0 || blank < 0 || blank >= C) return false;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return false;
  return dtype == K2AMD_F32 || dtype == K2AMD_F64;
}

// What the launches take of valid arguments: the batch is gridDim.z, tile ids of the three
// products are ints.
bool ShapeServed(int B, int S, int T, int C) {
  if (B > 65535) return false;
  const long long ts = (S + 32) / 32, tt = (T + 31) / 32, tc = (C + 31) / 32, lim = 1ll << 30;
  return B * ts * tt <= lim && B * ts * tc <= lim && B * tt * tc <= lim;
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
  if (!ShapeServed(B, S, T, C)) return K2AMD_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SimpleForward<float>((const float *)lm, (const float *)am, symbols, boundary, (float *)px, (float *)py, (float *)lm_probs, (float *)am_probs, (float *)lm_max, (float *)am_max, (float *)denom, B, S, T, C, termination_symbol, rnnt_type, st);
  return SimpleForward<double>((const double *)lm, (const double *)am, symbols, boundary, (double *)px, (double *)py, (double *)lm_probs, (double *)am_probs, (double *)lm_max, (double *)am_max, (double *)denom, B, S, T, C, termination_symbol, rnnt_type, st);
}

size_t k2amd_rnnt_logprobs_simple_backward_scratch_elements(int B, int S, int T) {
  if (B <= 0 || S < 0 || T <= 0) return 0;
  const size_t rows = (size_t)B * (S + 1);
  return rows * T + (size_t)B * SumsGroups(S) * T + 2 * rows * SumsChunks(T);
}

int k2amd_rnnt_logprobs_simple_backward(const void *px_grad, const void *py_grad,
                                        const void *seq_scale, const int64_t *symbols, const int64_t *boundary,
                                        const void *lm_probs, const void *am_probs,
                                        const void *denom, void *lm_grad, void *am_grad,
                                        void *q_scratch, size_t q_scratch_elements, int B, int S,
                                        int T, int C, int termination_symbol, int rnnt_type,
                                        int dtype, void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (!ShapeServed(B, S, T, C)) return K2AMD_ERR_UNSUPPORTED;
  {  // no frames or no sequences: nothing is asked for, and a null pointer is as good as any
    const size_t need = k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T);
    if (need > 0 && (q_scratch == nullptr || q_scratch_elements < need)) return K2AMD_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SimpleBackward<float>((const float *)px_grad, (const float *)py_grad, (const float *)seq_scale, symbols, boundary, (const float *)lm_probs, (const float *)am_probs, (const float *)denom, (float *)lm_grad, (float *)am_grad, (float *)q_scratch, B, S, T, C, termination_symbol, rnnt_type, st);
  return SimpleBackward<double>((const double *)px_grad, (const double *)py_grad, (const double *)seq_scale, symbols, boundary, (const double *)lm_probs, (const double *)am_probs, (const double *)denom, (double *)lm_grad, (double *)am_grad, (double *)q_scratch, B, S, T, C, termination_symbol, rnnt_type, st);
}

}  // extern "C"
