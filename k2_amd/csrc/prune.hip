// Pruning side of the RNN-T path: the integer prune ranges and the lm gather / scatter.
//   get_rnnt_prune_ranges             k2/python/k2/rnnt_loss.py:636-780
//   get_rnnt_prune_ranges_deprecated  k2/python/k2/rnnt_loss.py:786-910
//   do_rnnt_pruning        k2/python/k2/rnnt_loss.py:913-954
#include <cstdlib>
#include <cstring>

#include "common.h"

namespace k2amd {
namespace {

constexpr int kPruneThreads = 256;

// Reverse running minimum of n ints (Hillis-Steele on two rotating buffers whose elements lie
// `stride` ints apart: LDS, or global memory that only this workgroup touches).  Returns the
// buffer that holds the result.  Every thread of the workgroup must call it.
typedef int __attribute__((may_alias)) ScanInt;  // the global buffers are halves of 64-bit words
__device__ ScanInt *SuffixMin(ScanInt *a, ScanInt *b, int n, size_t stride) {
  for (int off = 1; off < n; off <<= 1) {
    for (int t = threadIdx.x; t < n; t += kPruneThreads) {
      int v = a[t * stride];
      if (t + off < n) v = min(v, a[(size_t)(t + off) * stride]);
      b[t * stride] = v;
    }
    __syncthreads();
    ScanInt *tmp = a; a = b; b = tmp;
  }
  return a;
}

// Step 1 of get_rnnt_prune_ranges: for every frame the window start with the largest
//   sum_{k<R} py_grad[b, w+k, t]  -  px_grad[b, w-1, t]        (k2/python/k2/rnnt_loss.py:730-747)
// A workgroup handles 64 frames of one sequence (reads are contiguous along t) and splits the
// candidate window starts over kArgSplit thread groups, whose results meet in LDS.
//
// The window sum adds the rows first to last in the input precision and subtracts px_grad
// afterwards, exactly as the reference's torch.sum / subtraction does, and the arg-max keeps the
// first maximum (torch.argmax), so that identical inputs give identical integers.  The raw
// arg-max goes to ranges[b, t, 0]; step 2 turns it into the final ranges in place.
constexpr int kArgFrames = 64;
constexpr int kArgSplit = 4;

// kR > 0: the window length as a compile-time constant (the usual s_range of 2..8), which lets the
// loads of four windows be issued together; kR == 0: any length, one window at a time.
template <typename T, int kR>
__global__ __launch_bounds__(kArgFrames * kArgSplit) void PruneArgmaxKernel(
    const T *__restrict__ px_grad, const T *__restrict__ py_grad, int64_t *__restrict__ ranges,
    int S, int Tn, int modified, int R_any, int frame_blocks) {
  __shared__ T best_v_s[kArgSplit][kArgFrames];
  __shared__ int best_w_s[kArgSplit][kArgFrames];
  const int R = kR > 0 ? kR : R_any;
  const int b = blockIdx.x / frame_blocks;
  const int tx = threadIdx.x % kArgFrames, grp = threadIdx.x / kArgFrames;
  const int t = (blockIdx.x - b * frame_blocks) * kArgFrames + tx;
  const int T1 = modified ? Tn : Tn + 1;
  const int S1 = S + 1;
  const int n_win = S1 - R + 1;
  const T *gx = px_grad + (size_t)b * S * T1;
  const T *gy = py_grad + (size_t)b * S1 * Tn;
  // group g takes the contiguous share [w_lo, w_hi) of the window starts, so that "first
  // maximum" inside a share and across shares (lower group wins ties) is the global first
  const int per = (n_win + kArgSplit - 1) / kArgSplit;
  const int w_lo = grp * per, w_hi = min(n_win, w_lo + per);
  T best_v = 0;
  int best = -1;
  auto window = [&](int w) -> T {
    T acc = gy[(size_t)w * Tn + t];
    if (kR > 0) {
#pragma unroll
      for (int k = 1; k < kR; ++k) acc = acc + gy[(size_t)(w + k) * Tn + t];
    } else {
      for (int k = 1; k < R; ++k) acc = acc + gy[(size_t)(w + k) * Tn + t];
    }
    return acc - (w == 0 ? T(0) : gx[(size_t)(w - 1) * T1 + t]);
  };
  if (t < Tn) {
    int w = w_lo;
    if (kR > 0) {
      for (; w + 4 <= w_hi; w += 4) {
        T v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = window(w + i);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (best < 0 || v[i] > best_v) { best_v = v[i]; best = w + i; }
      }
    }
    for (; w < w_hi; ++w) {
      const T v = window(w);
      if (best < 0 || v > best_v) { best_v = v; best = w; }
    }
  }
  best_v_s[grp][tx] = best_v;
  best_w_s[grp][tx] = best;
  __syncthreads();
  if (grp == 0 && t < Tn) {
    for (int g2 = 1; g2 < kArgSplit; ++g2) {
      const int w2 = best_w_s[g2][tx];
      const T v2 = best_v_s[g2][tx];
      if (w2 >= 0 && (best < 0 || v2 > best_v)) { best_v = v2; best = w2; }
    }
    ranges[((size_t)b * Tn + t) * R] = best < 0 ? 0 : best;
  }
}

template <typename T>
void LaunchArgmax(const T *px_grad, const T *py_grad, int64_t *ranges, int S, int Tn, int modified,
                  int R, int B, hipStream_t st) {
  // one workgroup per (sequence, 64 frames), the sequence slowest
  const int frame_blocks = (Tn + kArgFrames - 1) / kArgFrames;
  const dim3 grid((unsigned)((size_t)B * frame_blocks)), block(kArgFrames * kArgSplit);
#define K2AMD_ARGMAX(KR)                                                                         \
  hipLaunchKernelGGL((PruneArgmaxKernel<T, KR>), grid, block, 0, st, px_grad, py_grad, ranges, S, \
                     Tn, modified, R, frame_blocks)
  switch (R) {
    case 2: K2AMD_ARGMAX(2); break;
    case 3: K2AMD_ARGMAX(3); break;
    case 4: K2AMD_ARGMAX(4); break;
    case 5: K2AMD_ARGMAX(5); break;
    case 6: K2AMD_ARGMAX(6); break;
    case 7: K2AMD_ARGMAX(7); break;
    case 8: K2AMD_ARGMAX(8); break;
    default: K2AMD_ARGMAX(0); break;
  }
#undef K2AMD_ARGMAX
}

// Step 1 of get_rnnt_prune_ranges_deprecated (k2/python/k2/rnnt_loss.py:853-873): for every frame
// the window of R rows with the largest total occupation
//   prefix[w + R] - prefix[w],   prefix[k] = sum_{i<k} (px_grad[b,i,t] + py_grad[b,i,t])
// with px_grad's row S counting as zero, first maximum over w = 0 .. S + 1 - R.  The occupation of a
// cell is added in the input precision, as the reference's tensor addition does; a prefix is
// accumulated in double and rounded to the input precision once, which is how torch.cumsum forms
// it on the CPU; the difference of two prefixes is taken in the input precision again.  One
// thread per frame (loads contiguous along t) keeps the leading and the trailing prefix as two
// running sums, each the same function of the rows below it whoever computes it.
template <typename T>
__global__ __launch_bounds__(256) void PruneDeprecatedArgmaxKernel(
    const T *__restrict__ px_grad, const T *__restrict__ py_grad, int64_t *__restrict__ ranges,
    int S, int Tn, int modified, int R, int frame_blocks) {
  const int b = blockIdx.x / frame_blocks;
  const int t = (blockIdx.x - b * frame_blocks) * 256 + threadIdx.x;
  if (t >= Tn) return;
  const int T1 = modified ? Tn : Tn + 1;
  const T *gx = px_grad + (size_t)b * S * T1;
  const T *gy = py_grad + (size_t)b * (S + 1) * Tn;
  auto occupation = [&](int s) -> T {
    return (s < S ? gx[(size_t)s * T1 + t] : T(0)) + gy[(size_t)s * Tn + t];
  };
  double lead = 0, trail = 0;
  for (int s = 0; s < R; ++s) lead += (double)occupation(s);
  const int n_win = S + 2 - R;
  T best_v = 0;
  int best = -1;
  for (int w = 0; w < n_win; ++w) {
    const T v = (T)lead - (T)trail;
    if (best < 0 || v > best_v) { best_v = v; best = w; }
    if (w + 1 < n_win) {
      lead += (double)occupation(w + R);
      trail += (double)occupation(w);
    }
  }
  ranges[((size_t)b * Tn + t) * R] = best < 0 ? 0 : best;
}

// Step 2: one workgroup per sequence.  Frames from t_end - 1 on are pinned to
// max(s_end - R + 1, 0), then the two monotone passes of _adjust_pruning_lower_bound
// (k2/python/k2/rnnt_loss.py:580-630, 749-766) run as log-step scans and the ranges are written
// over the raw arg-max values.  The scans' two buffers of T ints lie in LDS (kInLds) or, for a T
// whose buffers LDS does not hold, in the sequence's own part of `ranges`: frame t's two ints
// are the halves of the 64-bit word ranges[b][t][0], which holds the raw arg-max until the first
// loop has read it and the frame's final range only after the last loop has read both halves.
template <bool kInLds>
__global__ __launch_bounds__(kPruneThreads) void PruneFinishKernel(
    const int64_t *__restrict__ boundary, int64_t *ranges, int Tn, int modified, int R) {
  HIP_DYNAMIC_SHARED(int, lds)
  const int b = blockIdx.x;
  const size_t stride = kInLds ? 1 : 2 * (size_t)R;
  ScanInt *buf0 = kInLds ? lds : reinterpret_cast<ScanInt *>(ranges + (size_t)b * Tn * R);
  ScanInt *buf1 = kInLds ? lds + Tn : buf0 + 1;
  const int64_t s_end = boundary[4 * b + 2], t_end = boundary[4 * b + 3];
  int64_t pad64 = s_end - R + 1;
  const int pad = pad64 < 0 ? 0 : (int)pad64;
  for (int t = threadIdx.x; t < Tn; t += kPruneThreads) {
    const int raw = (int)ranges[((size_t)b * Tn + t) * R];
    buf0[t * stride] = t < t_end - 1 ? raw : pad;
  }
  __syncthreads();
  const int ramp = (modified ? 2 : R) - 1;
  ScanInt *cur = SuffixMin(buf0, buf1, Tn, stride);
  ScanInt *other = cur == buf0 ? buf1 : buf0;
  for (int t = threadIdx.x; t < Tn; t += kPruneThreads) cur[t * stride] = -(cur[t * stride] - ramp * t);
  __syncthreads();
  cur = SuffixMin(cur, other, Tn, stride);
  for (int t = threadIdx.x; t < Tn; t += kPruneThreads) {
    int v = cur[t * stride];
    v = v < 0 ? 0 : v;
    const int64_t s_begin = -(int64_t)(v - ramp * t);
    int64_t *out = ranges + ((size_t)b * Tn + t) * R;
    for (int k = 0; k < R; ++k) out[k] = s_begin + k;
  }
}

template <typename T>
__global__ void GatherKernel(const T *__restrict__ lm, const int64_t *__restrict__ ranges,
                             T *__restrict__ out, int S1, int TR, int D, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / D;
    const int d = (int)(i - row * D);
    const size_t b = row / TR;
    const int64_t s = ranges[row];
    out[i] = (s >= 0 && s < S1) ? lm[(b * S1 + (size_t)s) * D + d] : T(0);
  }
}

template <typename T>
__global__ void ZeroKernel(T *__restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x)
    dst[i] = T(0);
}

// Hardware floating-point atomics: several (t,k) of one sequence point at the same lm row.
template <typename T>
__global__ void ScatterAddKernel(const T *__restrict__ grad, const int64_t *__restrict__ ranges,
                                 T *__restrict__ lm_grad, int S1, int TR, int D, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / D;
    const int d = (int)(i - row * D);
    const size_t b = row / TR;
    const int64_t s = ranges[row];
    if (s >= 0 && s < S1) unsafeAtomicAdd(lm_grad + (b * S1 + (size_t)s) * D + d, grad[i]);
  }
}

// The same sums without atomics and in a fixed order: one workgroup per lm row (b, s) lists the rows
// of grad that point at it, in the order of (t, k) (each thread looks at a contiguous share of
// ranges[b], an exclusive scan over the threads' counts places its finds).  The threads then split
// into kParts groups; group p adds up rows p, p + kParts, .. of the list for its columns, with four
// independent partial sums (rows j, j + kParts, j + 2 kParts, j + 3 kParts in flight together: a
// frame-synchronous lattice sends hundreds of rows to the same s, and one chain of dependent loads
// per column would take as long as the rest of the launch), and the groups' sums are added in order
// through LDS.  Which terms meet in which partial sum depends only on the list: the same bits in
// every run.
constexpr int kGatherThreads = 256;
template <typename T, int kVec>
__global__ __launch_bounds__(kGatherThreads) void GatherBackwardKernel(
    const T *__restrict__ grad, const int64_t *__restrict__ ranges, T *__restrict__ lm_grad, int S1,
    int TR, int D) {
  HIP_DYNAMIC_SHARED(unsigned char, gather_smem)
  int *found = reinterpret_cast<int *>(gather_smem);  // [TR] row numbers, in order
  __shared__ int counts[kGatherThreads + 1];
  const int b = blockIdx.x / S1, s = blockIdx.x - b * S1;
  const int64_t *r = ranges + (size_t)b * TR;
  const int per = (TR + kGatherThreads - 1) / kGatherThreads;
  const int lo = min((int)threadIdx.x * per, TR), hi = min(lo + per, TR);
  int mine = 0;
  for (int i = lo; i < hi; ++i) mine += r[i] == s;
  counts[threadIdx.x + 1] = mine;
  if (threadIdx.x == 0) counts[0] = 0;
  __syncthreads();
  for (int step = 1; step < kGatherThreads; step <<= 1) {  // inclusive scan of counts[1..]
    const int add = (int)threadIdx.x + 1 > step ? counts[threadIdx.x + 1 - step] : 0;
    __syncthreads();
    counts[threadIdx.x + 1] += add;
    __syncthreads();
  }
  int at = counts[threadIdx.x];
  for (int i = lo; i < hi; ++i)
    if (r[i] == s) found[at++] = i;
  __syncthreads();
  const int n = counts[kGatherThreads];
  const T *g = grad + (size_t)b * TR * D;
  T *out = lm_grad + ((size_t)b * S1 + s) * D;
  // groups of `width` threads, each thread kVec adjacent columns; the columns in passes of
  // width * kVec where D is wider than that
  const int groups_of = D / kVec;  // threads that cover a row once
  const int width = groups_of < kGatherThreads ? groups_of : kGatherThreads;
  const int parts = kGatherThreads / width, part = threadIdx.x / width, lane = threadIdx.x - part * width;
  T *partial = reinterpret_cast<T *>(gather_smem + (((size_t)TR * sizeof(int) + 15) / 16) * 16);  // [parts][width * kVec]
  for (int c0 = 0; c0 < D; c0 += width * kVec) {
    const int c = c0 + lane * kVec;
    T acc[4][kVec];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < kVec; ++e) acc[u][e] = 0;
    if (part < parts && c < D) {
      for (int j = part; j < n; j += 4 * parts) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int jj = j + u * parts;
          if (jj < n) {
            const T *src = g + (size_t)found[jj] * D + c;
#pragma unroll
            for (int e = 0; e < kVec; ++e) acc[u][e] += src[e];
          }
        }
      }
    }
    if (part < parts && c < D) {
#pragma unroll
      for (int e = 0; e < kVec; ++e)
        partial[(size_t)part * width * kVec + lane * kVec + e] = (acc[0][e] + acc[1][e]) + (acc[2][e] + acc[3][e]);
    }
    __syncthreads();
    if (part == 0 && c < D) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        T sum = partial[lane * kVec + e];
        for (int p = 1; p < parts; ++p) sum += partial[(size_t)p * width * kVec + lane * kVec + e];
        out[c + e] = sum;
      }
    }
    __syncthreads();
  }
}

constexpr size_t kFinishLdsLimit = 64 * 1024;

// K2AMD_PRUNE_SCAN_ROWS=global: the finishing kernel's scans run in `ranges` itself at any T
// (tests and comparisons; without it only where two rows of T ints exceed kFinishLdsLimit).
bool FinishRowsInRanges() {
  const char *e = std::getenv("K2AMD_PRUNE_SCAN_ROWS");
  return e != nullptr && std::strcmp(e, "global") == 0;
}

unsigned GridFor(size_t n) {
  size_t blocks = (n + 255) / 256;
  return (unsigned)(blocks > 8192 ? 8192 : (blocks == 0 ? 1 : blocks));
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

int k2amd_rnnt_prune_ranges(const void *px_grad, const void *py_grad, const int64_t *boundary,
                            int64_t *ranges, int B, int S, int T, int modified, int s_range,
                            int dtype, void *stream) {
  if (B < 0 || S < 0 || T < 0 || s_range < 1 || s_range > S + 1 || !boundary ||
      (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0 || T == 0) return K2AMD_OK;
  const size_t smem = 2 * (size_t)T * sizeof(int);
  // 32-bit element offsets inside a sequence, 32-bit workgroup counts
  if ((long long)(S + 1) * ((long long)T + 1) >= (1ll << 31) ||
      (long long)B * ((T + kArgFrames - 1) / kArgFrames) >= (1ll << 31))
    return K2AMD_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  modified = modified ? 1 : 0;
  if (dtype == K2AMD_F32)
    LaunchArgmax((const float *)px_grad, (const float *)py_grad, ranges, S, T, modified, s_range, B, st);
  else
    LaunchArgmax((const double *)px_grad, (const double *)py_grad, ranges, S, T, modified, s_range, B, st);
  if (smem <= kFinishLdsLimit && !FinishRowsInRanges())
    hipLaunchKernelGGL(PruneFinishKernel<true>, dim3(B), dim3(kPruneThreads), smem, st, boundary, ranges, T, modified, s_range);
  else
    hipLaunchKernelGGL(PruneFinishKernel<false>, dim3(B), dim3(kPruneThreads), 0, st, boundary, ranges, T, modified, s_range);
  return LaunchStatus();
}

int k2amd_rnnt_prune_ranges_deprecated(const void *px_grad, const void *py_grad,
                                       const int64_t *boundary, int64_t *ranges, int B, int S,
                                       int T, int modified, int s_range, int dtype, void *stream) {
  if (B < 0 || S < 0 || T < 0 || s_range < 1 || s_range > S + 1 || !boundary ||
      (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0 || T == 0) return K2AMD_OK;
  const size_t smem = 2 * (size_t)T * sizeof(int);
  const int frame_blocks = (T + 255) / 256;
  if ((long long)(S + 1) * ((long long)T + 1) >= (1ll << 31) || (long long)B * frame_blocks >= (1ll << 31))
    return K2AMD_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  modified = modified ? 1 : 0;
  const dim3 grid((unsigned)((size_t)B * frame_blocks));
  if (dtype == K2AMD_F32)
    hipLaunchKernelGGL(PruneDeprecatedArgmaxKernel<float>, grid, dim3(256), 0, st, (const float *)px_grad, (const float *)py_grad, ranges, S, T, modified, s_range, frame_blocks);
  else
    hipLaunchKernelGGL(PruneDeprecatedArgmaxKernel<double>, grid, dim3(256), 0, st, (const double *)px_grad, (const double *)py_grad, ranges, S, T, modified, s_range, frame_blocks);
  if (smem <= kFinishLdsLimit && !FinishRowsInRanges())
    hipLaunchKernelGGL(PruneFinishKernel<true>, dim3(B), dim3(kPruneThreads), smem, st, boundary, ranges, T, modified, s_range);
  else
    hipLaunchKernelGGL(PruneFinishKernel<false>, dim3(B), dim3(kPruneThreads), 0, st, boundary, ranges, T, modified, s_range);
  return LaunchStatus();
}

int k2amd_rnnt_prune_gather(const void *lm, const int64_t *ranges, void *lm_pruned, int B, int S1,
                            int T, int R, int D, int dtype, void *stream) {
  if (B < 0 || S1 < 0 || T < 0 || R < 0 || D < 0 || (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  const size_t n = (size_t)B * T * R * D;
  if (n == 0) return K2AMD_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == K2AMD_F32)
    hipLaunchKernelGGL(GatherKernel<float>, dim3(GridFor(n)), dim3(256), 0, st, (const float *)lm, ranges, (float *)lm_pruned, S1, T * R, D, n);
  else
    hipLaunchKernelGGL(GatherKernel<double>, dim3(GridFor(n)), dim3(256), 0, st, (const double *)lm, ranges, (double *)lm_pruned, S1, T * R, D, n);
  return LaunchStatus();
}

int k2amd_rnnt_prune_gather_backward(const void *grad, const int64_t *ranges, void *lm_grad, int B,
                                     int S1, int T, int R, int D, int dtype, void *stream) {
  if (B < 0 || S1 < 0 || T < 0 || R < 0 || D < 0 || (dtype != K2AMD_F32 && dtype != K2AMD_F64))
    return K2AMD_ERR_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t n_out = (size_t)B * S1 * D, n = (size_t)B * T * R * D;
  if (n_out == 0) return K2AMD_OK;
  const size_t list_bytes = (((size_t)T * R * sizeof(int) + 15) / 16) * 16;
  if (list_bytes <= 40 * 1024 && D >= 1 && (long long)B * S1 < (1ll << 31) && (long long)T * R * D < (1ll << 31)) {
    // the order-preserving kernel (a sequence's list of T * R row numbers fits its LDS)
    const dim3 grid((unsigned)(B * S1)), block(kGatherThreads);
    const bool vec = D % 4 == 0;  // 16-byte (fp32) / 32-byte (fp64) groups of columns per thread
    const size_t esz = dtype == K2AMD_F32 ? 4 : 8;
    const size_t smem = list_bytes + (size_t)kGatherThreads * (vec ? 4 : 1) * esz;
    if (dtype == K2AMD_F32) {
      if (vec) hipLaunchKernelGGL((GatherBackwardKernel<float, 4>), grid, block, smem, st, (const float *)grad, ranges, (float *)lm_grad, S1, T * R, D);
      else hipLaunchKernelGGL((GatherBackwardKernel<float, 1>), grid, block, smem, st, (const float *)grad, ranges, (float *)lm_grad, S1, T * R, D);
    } else {
      if (vec) hipLaunchKernelGGL((GatherBackwardKernel<double, 4>), grid, block, smem, st, (const double *)grad, ranges, (double *)lm_grad, S1, T * R, D);
      else hipLaunchKernelGGL((GatherBackwardKernel<double, 1>), grid, block, smem, st, (const double *)grad, ranges, (double *)lm_grad, S1, T * R, D);
    }
    return LaunchStatus();
  }
  if (dtype == K2AMD_F32) {
    hipLaunchKernelGGL(ZeroKernel<float>, dim3(GridFor(n_out)), dim3(256), 0, st, (float *)lm_grad, n_out);
    if (n) hipLaunchKernelGGL(ScatterAddKernel<float>, dim3(GridFor(n)), dim3(256), 0, st, (const float *)grad, ranges, (float *)lm_grad, S1, T * R, D, n);
  } else {
    hipLaunchKernelGGL(ZeroKernel<double>, dim3(GridFor(n_out)), dim3(256), 0, st, (double *)lm_grad, n_out);
    if (n) hipLaunchKernelGGL(ScatterAddKernel<double>, dim3(GridFor(n)), dim3(256), 0, st, (const double *)grad, ranges, (double *)lm_grad, S1, T * R, D, n);
  }
  return LaunchStatus();
}

}  // extern "C"
