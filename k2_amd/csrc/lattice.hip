// pruned_ranges_to_lattice (k2/python/csrc/torch/pruned_ranges_to_lattice.cu:60-263): the pruned
// RNN-T band as one acyclic lattice per sequence, for forced alignment.
//
// Sequence b with F = frames[b] frames has F * R + 1 states: state t * R + k is "frame t, k-th
// symbol position of the band" and the last one is the super-final state.  State (t, k):
//   k < R-1: a "vertical" arc to (t, k+1) with label symbols[b, ranges[b,t,k]] and score
//            logits[b,t,k,label];
//   a "horizontal" blank arc (label 0, score logits[b,t,k,0]) to (t+1, ranges[b,t,k] -
//            ranges[b,t+1,0]) when t < F-1 and that position is >= 0 (always counted for k = R-1);
//   the state before the super-final one only has the arc (label -1, score 0) into it.
// arc_map[arc] is the element index of the arc's score inside `logits`, or -1.
//
// Three launches instead of the reference's ragged-shape machinery: per-sequence arc counts with
// an exclusive scan inside the sequence (one workgroup per sequence), a scan over the B
// sequences (one workgroup), then one thread per state writes its arcs.  The caller reads the two
// totals between launch 2 and launch 3 to size the outputs, as the reference does.
#include <hip/hip_fp16.h>

#include "common.h"

namespace k2amd {
namespace {

constexpr int kScanThreads = 256;

struct LatticeGeom {
  int B, T, R;
};

// Arcs leaving local state s1 of sequence b (0, 1 or 2).
__device__ __forceinline__ int ArcsOfState(const int32_t *__restrict__ ranges, const LatticeGeom &g,
                                           int b, int F, int s1) {
  if (s1 == F * g.R) return 0;  // super-final state
  const int t = s1 / g.R, k = s1 - t * g.R;
  bool horizontal = false;
  if (t < F - 1) {
    const int32_t *r = ranges + ((size_t)b * g.T + t) * g.R;
    horizontal = r[k] >= r[g.R];  // ranges[b, t+1, 0]
  }
  return (k != g.R - 1 && horizontal) ? 2 : 1;
}

// Exclusive scan of `v` over the workgroup (kScanThreads threads); returns the total through
// *total.  `lds` holds kScanThreads ints.
__device__ __forceinline__ int BlockExclusiveScan(int v, int *lds, int *total) {
  const int tid = threadIdx.x;
  lds[tid] = v;
  __syncthreads();
  for (int off = 1; off < kScanThreads; off <<= 1) {
    const int add = tid >= off ? lds[tid - off] : 0;
    __syncthreads();
    lds[tid] += add;
    __syncthreads();
  }
  const int inclusive = lds[tid];
  *total = lds[kScanThreads - 1];
  __syncthreads();
  return inclusive - v;
}

// Launch 1: arc_local[b][s1] = arcs of sequence b that leave states before s1; seq_arcs[b] = all.
__global__ __launch_bounds__(kScanThreads) void LatticeCountKernel(
    const int32_t *__restrict__ ranges, const int32_t *__restrict__ frames,
    int32_t *__restrict__ arc_local, int32_t *__restrict__ seq_arcs, LatticeGeom g) {
  __shared__ int lds[kScanThreads];
  const int b = blockIdx.x;
  const int F = min(max(frames[b], 0), g.T);
  const int states = F * g.R + 1;
  int32_t *out = arc_local + (size_t)b * ((size_t)g.T * g.R + 1);
  int carry = 0;
  for (int base = 0; base < states; base += kScanThreads) {
    const int s1 = base + threadIdx.x;
    const int n = s1 < states ? ArcsOfState(ranges, g, b, F, s1) : 0;
    int total;
    const int before = BlockExclusiveScan(n, lds, &total);
    if (s1 < states) out[s1] = carry + before;
    carry += total;
  }
  if (threadIdx.x == 0) seq_arcs[b] = carry;
}

// Launch 2: state_splits[b] / arc_base[b] = states / arcs of the sequences before b, b = 0..B.
__global__ __launch_bounds__(kScanThreads) void LatticeOffsetsKernel(
    const int32_t *__restrict__ frames, const int32_t *__restrict__ seq_arcs,
    int32_t *__restrict__ state_splits, int32_t *__restrict__ arc_base, LatticeGeom g) {
  __shared__ int lds[kScanThreads];
  int carry_s = 0, carry_a = 0;
  for (int base = 0; base < g.B; base += kScanThreads) {
    const int b = base + threadIdx.x;
    const int ns = b < g.B ? min(max(frames[b], 0), g.T) * g.R + 1 : 0;
    const int na = b < g.B ? seq_arcs[b] : 0;
    int tot_s, tot_a;
    const int before_s = BlockExclusiveScan(ns, lds, &tot_s);
    const int before_a = BlockExclusiveScan(na, lds, &tot_a);
    if (b < g.B) {
      state_splits[b] = carry_s + before_s;
      arc_base[b] = carry_a + before_a;
    }
    carry_s += tot_s;
    carry_a += tot_a;
  }
  if (threadIdx.x == 0) {
    state_splits[g.B] = carry_s;
    arc_base[g.B] = carry_a;
  }
}

__device__ __forceinline__ float AsScore(float v) { return v; }
__device__ __forceinline__ float AsScore(double v) { return (float)v; }
__device__ __forceinline__ float AsScore(__half v) { return __half2float(v); }

struct ArcRecord {  // k2's Arc (k2/csrc/fsa.h): 16 bytes
  int32_t src, dest, label;
  float score;
};

// Launch 3: one thread per (b, local state).
template <typename T>
__global__ void LatticeFillKernel(const int32_t *__restrict__ ranges,
                                  const int32_t *__restrict__ frames,
                                  const int64_t *__restrict__ symbols, const T *__restrict__ logits,
                                  long long st0, long long st1, long long st2, long long st3,
                                  const int32_t *__restrict__ state_splits,
                                  const int32_t *__restrict__ arc_base,
                                  const int32_t *__restrict__ arc_local,
                                  int32_t *__restrict__ arc_splits, ArcRecord *__restrict__ arcs,
                                  int32_t *__restrict__ arc_map, LatticeGeom g, int S, int C) {
  const int per_seq = g.T * g.R + 1;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long long)g.B * per_seq) return;
  const int b = (int)(i / per_seq), s1 = (int)(i - (long long)b * per_seq);
  const int F = min(max(frames[b], 0), g.T);
  if (s1 > F * g.R) return;
  const int first = arc_base[b] + arc_local[(size_t)b * per_seq + s1];
  const int state01 = state_splits[b] + s1;
  arc_splits[state01] = first;
  if (b == g.B - 1 && s1 == F * g.R) arc_splits[state01 + 1] = arc_base[g.B];
  if (s1 == F * g.R) return;  // super-final state: no arcs
  ArcRecord arc;
  arc.src = s1;
  if (s1 == F * g.R - 1) {  // only the arc into the super-final state
    arc.dest = s1 + 1;
    arc.label = -1;
    arc.score = 0.f;
    arcs[first] = arc;
    arc_map[first] = -1;
    return;
  }
  const int t = s1 / g.R, k = s1 - t * g.R;
  const int32_t *r = ranges + ((size_t)b * g.T + t) * g.R;
  const long long row = b * st0 + t * st1 + k * st2;
  int n = 0;
  if (k < g.R - 1) {  // vertical arc with the symbol's label
    int32_t sym_idx = r[k];
    sym_idx = min(max(sym_idx, 0), S - 1);  // a corrupt range cannot drive the look-up outside
    int64_t label = symbols[(size_t)b * S + sym_idx];
    label = label < 0 ? 0 : (label >= C ? C - 1 : label);
    arc.dest = s1 + 1;
    arc.label = (int32_t)label;
    arc.score = AsScore(logits[row + label * st3]);
    arcs[first] = arc;
    arc_map[first] = (int32_t)(row + label * st3);
    n = 1;
  }
  const bool horizontal = t < F - 1 && r[k] >= r[g.R];
  if (k == g.R - 1 || horizontal) {  // blank arc to the next frame
    arc.dest = (t < F - 1 ? r[k] - r[g.R] : 0) + (t + 1) * g.R;
    arc.label = 0;
    arc.score = AsScore(logits[row]);
    arcs[first + n] = arc;
    arc_map[first + n] = (int32_t)row;
  }
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

int k2amd_lattice_count(const int32_t *ranges, const int32_t *frames, int32_t *arc_local,
                        int32_t *seq_arcs, int32_t *state_splits, int32_t *arc_base, int B, int T,
                        int R, void *stream) {
  if (B < 0 || T < 0 || R < 1) return K2AMD_ERR_INVALID_ARGUMENT;
  if ((long long)B * ((long long)T * R + 1) >= (1ll << 30)) return K2AMD_ERR_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  LatticeGeom g{B, T, R};
  if (B > 0)
    hipLaunchKernelGGL(LatticeCountKernel, dim3(B), dim3(kScanThreads), 0, st, ranges, frames, arc_local, seq_arcs, g);
  hipLaunchKernelGGL(LatticeOffsetsKernel, dim3(1), dim3(kScanThreads), 0, st, frames, seq_arcs, state_splits, arc_base, g);
  return LaunchStatus();
}

int k2amd_lattice_fill(const int32_t *ranges, const int32_t *frames, const int64_t *symbols,
                       const void *logits, const int64_t *logits_strides,
                       const int32_t *state_splits, const int32_t *arc_base,
                       const int32_t *arc_local, int32_t *arc_splits, void *arcs, int32_t *arc_map,
                       int B, int T, int R, int S, int C, int dtype, void *stream) {
  if (B < 0 || T < 0 || R < 1 || S < 1 || C < 1 || logits_strides == nullptr) return K2AMD_ERR_INVALID_ARGUMENT;
  if (dtype != K2AMD_F32 && dtype != K2AMD_F64 && dtype != K2AMD_F16) return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0) return K2AMD_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  LatticeGeom g{B, T, R};
  const long long n = (long long)B * ((long long)T * R + 1);
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  const long long s0 = logits_strides[0], s1 = logits_strides[1], s2 = logits_strides[2], s3 = logits_strides[3];
  ArcRecord *out = static_cast<ArcRecord *>(arcs);
  if (dtype == K2AMD_F32)
    hipLaunchKernelGGL(LatticeFillKernel<float>, grid, block, 0, st, ranges, frames, symbols, (const float *)logits, s0, s1, s2, s3, state_splits, arc_base, arc_local, arc_splits, out, arc_map, g, S, C);
  else if (dtype == K2AMD_F64)
    hipLaunchKernelGGL(LatticeFillKernel<double>, grid, block, 0, st, ranges, frames, symbols, (const double *)logits, s0, s1, s2, s3, state_splits, arc_base, arc_local, arc_splits, out, arc_map, g, S, C);
  else
    hipLaunchKernelGGL(LatticeFillKernel<__half>, grid, block, 0, st, ranges, frames, symbols, (const __half *)logits, s0, s1, s2, s3, state_splits, arc_base, arc_local, arc_splits, out, arc_map, g, S, C);
  return LaunchStatus();
}

}  // extern "C"
