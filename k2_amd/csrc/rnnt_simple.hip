// get_rnnt_logprobs for the "simple" joiner (am + lm), forward and backward
// (k2/python/k2/rnnt_loss.py:65-225).
//
// Forward:  row maxima + exponentials of am and lm (one wavefront per row), then a batched
// [S+1 x C] * [C x T] product (LDS-tiled 64x64, fp32 on the matrix cores) whose epilogue takes
// the log, adds the maxima back and emits
// px / py directly, so the normaliser never makes a round trip through HBM as a separate tensor
// apart from the `denom` buffer kept for the backward.
// Backward: Q = (dpx + dpy) / denom, two more batched products (Q * am_probs, Q^T * lm_probs)
// scaled by the saved exponentials; the symbol terms of the am gradient ride in that product's
// epilogue, the termination terms and the lm gradient's gathered terms have small kernels.
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
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + ty * 4 + i;
      if (m < M) pre[i] = epi.Prepare(b, m, n, column);
    }
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
  if (c_begin < c_end) {
    float ra[kAhead][8], rb[kAhead][8];
    const int c_last = c_end - 1;
#pragma unroll
    for (int d = 0; d < kAhead; ++d) {
      const int k = min(c_begin + d, c_last) * kChunk + half * 8;
      oa.Full(k, ra[d]);
      ob.Full(k, rb[d]);
    }
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
  if constexpr (Epilogue::kStaged) epi.Stage(b, n0, kMfmaTile, stage);
  if (n >= N) return;
  const auto column = epi.Column(b, n, col, stage);
  typename Epilogue::ElementData pre[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = m0 + wave * 8 + half * 4 + r;
    if (m < M) pre[r] = epi.Prepare(b, m, n, column);
  }
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
  if constexpr (Epilogue::kStaged) epi.Stage(b, n0, kTile, stage);
  const int n = n0 + qn + col;
  if (n >= N) return;
  const auto column = epi.Column(b, n, qn + col, stage);
  typename Epilogue::ElementData pre[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + qm + (r >> 2) * 8 + half * 4 + (r & 3);
    if (m < M) pre[r] = epi.Prepare(b, m, n, column);
  }
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
    if (big_tiles >= 512)  // two workgroups per compute unit without splitting K
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

// Epilogues work in two steps so that a thread can issue the loads of all its elements before
// the first store (the compiler cannot move a load across a store that might alias it, and one
// dependent round trip per element is what the tile's epilogue would otherwise cost):
//   epi.Stage(b, n0, width, scratch)          (only if Epilogue::kStaged; whole workgroup, has
//                                              barriers) what depends on the tile's columns
//   column = epi.Column(b, n, n - n0, scratch)   what depends on (b, n) only
//   pre    = epi.Prepare(b, m, n, column)        loads for element (m, n)
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

// Backward epilogue: out[b][m][n] = -scale[b][m][n] * acc  (scale = the saved exponentials).
template <typename T>
struct ScaleEpilogue {
  const T *scale;
  T *out;
  int M, N;
  struct ColumnData {};
  struct ElementData { T scale; };
  static constexpr bool kStaged = false;
  __device__ __forceinline__ ColumnData Column(int, int, int, const int *) const { return ColumnData(); }
  __device__ __forceinline__ ElementData Prepare(int b, int m, int n, const ColumnData &) const {
    return ElementData{scale[((size_t)b * M + m) * N + n]};
  }
  __device__ __forceinline__ void Finish(int b, int m, int n, T acc, const ColumnData &,
                                         const ElementData &e) const {
    out[((size_t)b * M + m) * N + n] = -e.scale * acc;
  }
};

// Epilogue of the am gradient, (m, n) = (t, c):
//   am_grad[b,t,c] = -am_probs[b,t,c] * acc + sum over s with symbols[b,s] == c of Gx(b,s,t).
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
  int M, N;  // Tn, C
  struct ColumnData {
    int hits;  // positions s with symbols[b,s] == c (all of them, also beyond kMaxHits)
    int s[kMaxHits];
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
  __device__ __forceinline__ ColumnData Column(int, int, int local, const int *scratch) const {
    ColumnData col;
    col.hits = scratch[local];
#pragma unroll
    for (int k = 0; k < kMaxHits; ++k) col.s[k] = scratch[kStageColumns + local * kMaxHits + k];
    return col;
  }
  __device__ __forceinline__ ElementData Prepare(int b, int t, int c, const ColumnData &col) const {
    ElementData e;
    e.scale = scale[((size_t)b * M + t) * N + c];
    e.sym_sum = 0;
    if (col.hits <= kMaxHits) {
#pragma unroll
      for (int k = 0; k < kMaxHits; ++k)
        if (k < col.hits) e.sym_sum += gv.Gx(b, col.s[k], t);
    } else {
      const int64_t *sym = symbols + (size_t)b * gv.S;
      for (int s = 0; s < gv.S; ++s)
        if (sym[s] == c) e.sym_sum += gv.Gx(b, s, t);
    }
    return e;
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

// am_grad[b,t,blank] += sum_s Gy(b,s,t).  One thread per (b,t); the reads of consecutive threads
// are consecutive.
template <typename T>
__global__ void AmBlankTermKernel(GradView<T> gv, T *__restrict__ am_grad, int B, int C,
                                  int blank) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= B * gv.Tn) return;
  const int b = i / gv.Tn, t = i - b * gv.Tn;
  T sy = 0;
  int s = 0;
  for (; s + 8 <= gv.S + 1; s += 8) {  // eight rows' loads in flight at a time
    T v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = gv.Gy(b, s + k, t);
#pragma unroll
    for (int k = 0; k < 8; ++k) sy += v[k];
  }
  for (; s <= gv.S; ++s) sy += gv.Gy(b, s, t);
  am_grad[(size_t)i * C + blank] += sy;
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
  if (Tn > 0) {
    hipLaunchKernelGGL(QKernel<T>, dim3(512), dim3(256), 0, st, gv, denom, q, B);
    {  // lm_grad[b][s][c] = -lm_probs * sum_t q[b][s][t] * am_probs[b][t][c]
      ScaleEpilogue<T> epi{lm_probs, lm_grad, S + 1, C};
      MatView av{(size_t)(S + 1) * Tn, Tn, 1};  // A(m=s, k=t) = q[b][s][t]
      MatView bv{(size_t)Tn * C, C, 1};         // B(k=t, n=c) = am_probs[b][t][c]
      LaunchProduct<T, true, false>((const T *)q, av, am_probs, bv, S + 1, C, Tn, B, epi, st);
    }
    {  // am_grad[b][t][c] = -am_probs * sum_s q[b][s][t] * lm_probs[b][s][c]
      AmGradEpilogue<T> epi{am_probs, am_grad, gv, symbols, Tn, C};
      MatView av{(size_t)(S + 1) * Tn, 1, Tn};   // A(m=t, k=s) = q[b][s][t]
      MatView bv{(size_t)(S + 1) * C, C, 1};     // B(k=s, n=c) = lm_probs[b][s][c]
      LaunchProduct<T, false, false>((const T *)q, av, lm_probs, bv, Tn, C, S + 1, B, epi, st);
    }
    hipLaunchKernelGGL(AmBlankTermKernel<T>, dim3((B * Tn + 255) / 256), dim3(256), 0, st, gv, am_grad, B, C, blank);
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
  {  // tile ids of the three products are ints
    const long long ts = (S + 32) / 32, tt = (T + 31) / 32, tc = (C + 31) / 32, lim = 1ll << 30;
    if (B * ts * tt > lim || B * ts * tc > lim || B * tt * tc > lim) return false;
  }
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
                                        const void *seq_scale, const int64_t *symbols, const int64_t *boundary,
                                        const void *lm_probs, const void *am_probs,
                                        const void *denom, void *lm_grad, void *am_grad,
                                        void *q_scratch, int B, int S, int T, int C,
                                        int termination_symbol, int rnnt_type, int dtype,
                                        void *stream) {
  if (!ArgsOk(B, S, T, C, termination_symbol, rnnt_type, dtype)) return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    return SimpleBackward<float>((const float *)px_grad, (const float *)py_grad, (const float *)seq_scale, symbols, boundary, (const float *)lm_probs, (const float *)am_probs, (const float *)denom, (float *)lm_grad, (float *)am_grad, (float *)q_scratch, B, S, T, C, termination_symbol, rnnt_type, st);
  return SimpleBackward<double>((const double *)px_grad, (const double *)py_grad, (const double *)seq_scale, symbols, boundary, (const double *)lm_probs, (const double *)am_probs, (const double *)denom, (double *)lm_grad, (double *)am_grad, (double *)q_scratch, B, S, T, C, termination_symbol, rnnt_type, st);
}

}  // extern "C"
