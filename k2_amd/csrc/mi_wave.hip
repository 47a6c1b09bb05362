// fp64 throughput path of the mutual-information recursion: the lattice of a sequence in chunks
// of 64 rows, ONE WAVEFRONT per chunk (lane = row, one column per step), the chunks of a sequence
// running as a pipeline through device-coherent "edge" words like the fp32 kernels of mi_fast.hip.
//
// The exact kernels (mi_generic.hip) pay a workgroup barrier and libm's exp / log1p per
// anti-diagonal; here a step is wavefront-synchronous (the value of the row above moves with one
// lane shift, no LDS, no barrier) and uses exp / log(1 + exp(.)) written for the ranges the
// recursion needs (mi_wave_math.h, 1e-15 relative).  Everything else follows the exact kernels
// term for term (k2/python/csrc/torch/mutual_information_cpu.cu:89-121 forward, :179-251
// backward), in particular the cut-off of log_add (k2/csrc/utils.h:543-562) and the guards on the
// derivatives (mutual_information_cpu.cu:195-211).
//
// Forward, lane q of chunk c owns lattice row i = 64 c + q and is at column j = n - q * skew at
// step n (skew 1 on a regular lattice, where a cell needs the cell above it in the same column; 0
// on a modified one).  Backward: column j = nt - n + (63 - q) * skew, each lane forms its cell's
// px-edge derivative d1, hands d1 * G to the lane above and keeps (1 - d1) * G for its next cell.
// A lane reads its own rows of px / py / p sixteen columns ahead (two register sets); what lies
// outside the tensors is never addressed (clamped indices, values masked afterwards).
//
// Chunk borders: the last lane of a chunk publishes its value of every step as one word; the first
// lane of the next chunk takes them 32 at a time (the request for
// the block after is in flight while the current one is used) and writes the sentinel back, so the
// workspace ends every launch in its initial state.  Waits are bounded (sticky error flag, as in
// mi_fast.hip).  Workgroups take their (sequence, chunk) from the ticket counter, producers first.
#include "common.h"
#include "mi_internal.h"
#include "mi_wave_math.h"

namespace k2amd {
namespace {

constexpr int kRows = 64;        // rows per chunk = lanes
constexpr int kSet = 16;         // columns per register set
constexpr int kEdgeBlock = 32;   // words handed over at a time = steps per pass of the main loop
constexpr unsigned long long kSentinel64 = 0x7fc5a5a57fc5a5a5ull;  // two 32-bit sentinels of mi_fast.hip
constexpr int kSpinLimit64 = 1 << 20;

struct WaveHeader {  // the first words of the workspace (same layout as mi_fast.hip's header)
  unsigned ticket;
  unsigned done;
  unsigned error;
  unsigned pad[61];
};

__device__ __forceinline__ bool GaveUp(WaveHeader *hdr) {
  return __hip_atomic_load(&hdr->error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
}
__device__ __forceinline__ unsigned long long LoadWord(unsigned long long *w) {
  return __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void StoreWord(unsigned long long *w, unsigned long long v) {
  __hip_atomic_store(w, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// lane `from` (a constant or a scalar) of v, to every lane
__device__ __forceinline__ double ReadLane(double v, int from) {
  const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
  const unsigned lo = __builtin_amdgcn_readlane((unsigned)u, from);
  const unsigned hi = __builtin_amdgcn_readlane((unsigned)(u >> 32), from);
  return __builtin_bit_cast(double, ((unsigned long long)hi << 32) | lo);
}

// A chunk border carries one word per step of its consumer, numbered by that step: a block of 32
// words per pass of the consumer's main loop.  Words outside [first, last] are never written.
//
// Consumer: lanes 0 .. 31 take block `m` (waiting, bounded, for what is not there yet), put the
// sentinel back and ask for block m + 1, which is looked at when its turn comes.
struct EdgeReader {
  unsigned long long *words;
  int first, last;
  unsigned long long next;  // what the request for the next block returned
  __device__ __forceinline__ void Init(unsigned long long *w, int first_word, int last_word, int lane) {
    words = w; first = first_word; last = last_word;
    next = (lane < kEdgeBlock && lane >= first && lane <= last) ? LoadWord(words + lane) : kSentinel64;
  }
  // lane l < 32 returns word 32 m + l
  __device__ __forceinline__ double Take(int m, int lane, WaveHeader *hdr) {
    const int at = m * kEdgeBlock + lane;
    const bool mine = lane < kEdgeBlock && at >= first && at <= last;
    unsigned long long v = next;
    int spins = 0;
    while (mine && v == kSentinel64) {
      v = LoadWord(words + at);
      if (v != kSentinel64) break;
      ++spins;
      if (((spins & 255) == 0 && GaveUp(hdr)) || spins > kSpinLimit64) {
        __hip_atomic_store(&hdr->error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v = 0x7ff8000000000000ull;  // NaN: the results of this launch are void
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (mine) StoreWord(words + at, kSentinel64);
    const int ahead = at + kEdgeBlock;
    next = (lane < kEdgeBlock && ahead >= first && ahead <= last) ? LoadWord(words + ahead) : kSentinel64;
    return __builtin_bit_cast(double, v);
  }
};

// Producer: the lane that owns the border row stores its value as word `at`, one word per step.
__device__ __forceinline__ void PublishWord(unsigned long long *words, int at, double v) {
  unsigned long long u = __builtin_bit_cast(unsigned long long, v);
  if (u == kSentinel64) u = 0x7ff8000000000000ull;
  StoreWord(words + at, u);
}

// The value of the previous lane (wave_shr:1) or of the next one (wave_shl:1), by DPP on the two
// halves of the double: a few cycles on the vector ALU where a shuffle goes through the LDS
// crossbar.  Lane 0 (lane 63) keeps its own value.
template <int kCtrl>
__device__ __forceinline__ double WaveShift(double v) {
  const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
  const int lo = (int)(unsigned)u, hi = (int)(unsigned)(u >> 32);
  const unsigned slo = (unsigned)__builtin_amdgcn_update_dpp(lo, lo, kCtrl, 0xf, 0xf, false);
  const unsigned shi = (unsigned)__builtin_amdgcn_update_dpp(hi, hi, kCtrl, 0xf, 0xf, false);
  return __builtin_bit_cast(double, ((unsigned long long)shi << 32) | slo);
}
__device__ __forceinline__ double FromLaneBelow(double v) { return WaveShift<0x138>(v); }  // wave_shr:1
__device__ __forceinline__ double FromLaneAbove(double v) { return WaveShift<0x130>(v); }  // wave_shl:1

// k2's log_add (k2/csrc/utils.h:518-563) with the short log(1 + exp(.)) of mi_wave_math.h
__device__ __forceinline__ double LogAddWave(double x, double y) {
  double diff;
  if (x < y) { diff = x - y; x = y; } else { diff = y - x; }
  if (diff >= Real<double>::kMinLogDiff) return x + Log1pExpNeg(diff);
  return x;
}

struct WaveGeom {
  int B, S, Tn, nchunks, edge_stride;
};

// The workgroup that drew the last of a launch's tickets puts the counter back for the next
// launch (nobody draws after it).
__device__ __forceinline__ void PutTicketsBack(WaveHeader *hdr, unsigned ticket, unsigned total) {
  if (ticket + 1 == total) __hip_atomic_store(&hdr->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The special cells of the forward recursion are expressed in its operands, so that every cell
// is log_add(up + fx, P + fy): no px term (first row; first column of a modified lattice) is
// fx = -inf; no py term (first column) is fy = -inf, except at the origin, where fy = 0 on a
// running value that starts at 0 gives p = 0 (log_add with -inf returns its other operand
// unchanged, as the reference's branches do).
template <bool kModified>
__global__ __launch_bounds__(kRows) void MiWaveForwardKernel(
    const double *__restrict__ px, const double *__restrict__ py, const int64_t *__restrict__ boundary,
    double *__restrict__ p, double *__restrict__ ans, WaveHeader *hdr, unsigned long long *edge,
    const WaveGeom g) {
  constexpr int skew = kModified ? 0 : 1, off = kModified ? -1 : 0;
  const int lane = threadIdx.x;
  unsigned ticket = 0;
  if (lane == 0) ticket = atomicAdd(&hdr->ticket, 1u);
  ticket = __builtin_amdgcn_readfirstlane(ticket);
  const int b = ticket / g.nchunks, c = ticket - b * g.nchunks;
  const Box box = LoadBox(boundary, b, g.S, g.Tn);
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const int chunks = box.ok ? ns / kRows + 1 : 0;  // chunks of this sequence that hold rows
  if (!box.ok && c == 0 && lane == 0) ans[b] = __builtin_nan("");
  if (c < chunks) {
    const int T1 = kModified ? g.Tn : g.Tn + 1;
    const int i = c * kRows + lane;
    const bool row_ok = i <= ns;
    const int s = box.s0 + (row_ok ? i : ns);  // clamped: addresses stay inside the tensors
    const double *pxrow = px + ((size_t)b * g.S + (s > 0 ? s - 1 : 0)) * T1;  // used only where i >= 1
    const double *pyrow = py + ((size_t)b * (g.S + 1) + s) * g.Tn;
    double *prow = p + ((size_t)b * (g.S + 1) + s) * (g.Tn + 1) + box.t0;
    const bool have_px = g.S > 0 && T1 > 0, have_py = g.Tn > 0;
    const double ninf = Real<double>::NegInf();
    // words of a border are numbered by the consumer's step (its lane 0 is at column n at step n
    // and needs p[i-1][n + off]): words -off .. nt
    unsigned long long *edges = edge + (size_t)b * (g.nchunks + 1) * g.edge_stride;
    EdgeReader in;
    if (c > 0) in.Init(edges + (size_t)c * g.edge_stride, -off, nt, lane);
    const bool has_below = c + 1 < chunks;
    unsigned long long *out = edges + (size_t)(c + 1) * g.edge_stride;
    const int nsteps = nt + 1 + (kRows - 1) * skew;
    // operands of step n for this lane (column j = n - lane * skew)
    double fx[2][kSet], fy[2][kSet];
    auto fetch = [&](int n0, double (&x)[kSet], double (&y)[kSet]) {
      const int j0 = n0 - lane * skew;
#pragma unroll
      for (int u = 0; u < kSet; ++u) {
        const int j = j0 + u;
        // indices clamped into the tensors' rows; what a clamp changed is masked below
        const double vx = have_px ? pxrow[min(max(box.t0 + j + off, 0), T1 - 1)] : 0.0;
        const double vy = have_py ? pyrow[min(max(box.t0 + j - 1, 0), g.Tn - 1)] : 0.0;
        x[u] = (i >= 1 && j + off >= 0) ? vx : ninf;
        y[u] = j >= 1 ? vy : (i == 0 ? 0.0 : ninf);
      }
    };
    fetch(0, fx[0], fy[0]);
    double P = 0.0;
    for (int m = 0; m * kEdgeBlock < nsteps; ++m) {
      const int n0 = m * kEdgeBlock;
      double taken = 0.0;
      if (c > 0 && n0 <= nt) taken = in.Take(m, lane, hdr);  // words n0 .. n0 + 31
#pragma unroll
      for (int set = 0; set < 2; ++set) {
        const int base = n0 + set * kSet;
        fetch(base + kSet, fx[set ^ 1], fy[set ^ 1]);
        __builtin_amdgcn_sched_barrier(0);  // the requests stay ahead of the steps
#pragma unroll
        for (int u = 0; u < kSet; ++u) {
          const int n = base + u;
          const int j = n - lane * skew;
          double up = FromLaneBelow(P);  // p[i-1][j + off], one step old
          if (c > 0) {
            const double e = ReadLane(taken, set * kSet + u);
            if (lane == 0 && n >= -off && n <= nt) up = e;  // (words outside that range do not exist)
          }
          const double v = LogAddWave(up + fx[set][u], P + fy[set][u]);
          if (row_ok && j >= 0 && j <= nt) {
            P = v;
            prow[j] = v;
          }
          if (has_below) {
            // lane 63 is at column n - 63 skew; the consumer needs it at its step n - 63 skew - off
            const int w = n - (kRows - 1) * skew - off;
            if (lane == kRows - 1 && w >= -off && w <= nt) PublishWord(out, w, P);
          }
        }
      }
    }
    if (i == ns) ans[b] = GaveUp(hdr) ? __builtin_nan("") : P;
  }
  if (lane == 0) PutTicketsBack(hdr, ticket, gridDim.x);
}

// exp(term1 - total) with the reference's guards (see PxDeriv in mi_generic_impl.h)
__device__ __forceinline__ double PxDerivWave(double term1, double total, bool *ok) {
  if (total - total != 0) total = 0;
  const double d = FastExp(term1 - total);
  *ok = (d - d == 0);
  return d;
}

template <bool kModified>
__global__ __launch_bounds__(kRows) void MiWaveBackwardKernel(
    const double *__restrict__ px, const double *__restrict__ p, const int64_t *__restrict__ boundary,
    double *__restrict__ ans_grad, double *__restrict__ px_grad, double *__restrict__ py_grad,
    WaveHeader *hdr, unsigned long long *edge, const WaveGeom g, int overwrite_ans_grad) {
  constexpr int skew = kModified ? 0 : 1, off = kModified ? -1 : 0;
  const int lane = threadIdx.x;
  unsigned ticket = 0;
  if (lane == 0) ticket = atomicAdd(&hdr->ticket, 1u);
  ticket = __builtin_amdgcn_readfirstlane(ticket);
  const int b = ticket / g.nchunks;
  const int c = g.nchunks - 1 - (ticket - b * g.nchunks);  // lower chunks (the producers) first
  const Box box = LoadBox(boundary, b, g.S, g.Tn);
  const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
  const int chunks = box.ok ? ns / kRows + 1 : 0;
  if (c < chunks) {
    const int T1 = kModified ? g.Tn : g.Tn + 1;
    const int i = c * kRows + lane;
    const bool row_ok = i <= ns;
    const int s = box.s0 + (row_ok ? i : ns);
    const int sa = s > 0 ? s - 1 : 0;  // the row above, used only where i >= 1
    const double *pxrow = px + ((size_t)b * g.S + sa) * T1;
    const double *prow = p + ((size_t)b * (g.S + 1) + s) * (g.Tn + 1);
    const double *parow = p + ((size_t)b * (g.S + 1) + sa) * (g.Tn + 1);
    double *gxrow = px_grad + ((size_t)b * g.S + sa) * T1 + box.t0 + off;
    double *gyrow = py_grad + ((size_t)b * (g.S + 1) + s) * g.Tn + box.t0 - 1;
    const bool have_px = g.S > 0 && T1 > 0;
    // words of the border below are numbered by this chunk's step: its lane 63 is at column
    // nt - n at step n and takes what flows into (i, nt - n) from (i + 1, nt - n - off): steps
    // -off .. nt
    unsigned long long *edges = edge + (size_t)b * (g.nchunks + 1) * g.edge_stride;
    EdgeReader in;
    const bool has_below = c + 1 < chunks;
    if (has_below) in.Init(edges + (size_t)(c + 1) * g.edge_stride, -off, nt, lane);
    unsigned long long *out = edges + (size_t)c * g.edge_stride;
    const double seed = ans_grad[b];
    const int nsteps = nt + 1 + (kRows - 1) * skew;
    // column of this lane at step n: nt - n + (63 - lane) * skew
    double fp[2][kSet], fa[2][kSet], fx[2][kSet];  // p[i][j], p[i-1][j+off], px[i-1][j+off]
    auto fetch = [&](int n0, double (&pp)[kSet], double (&pa)[kSet], double (&x)[kSet]) {
      const int j0 = nt - n0 + (kRows - 1 - lane) * skew;
#pragma unroll
      for (int u = 0; u < kSet; ++u) {
        const int j = j0 - u;
        // indices clamped into the tensors' rows; what a clamp changed is never used
        const int tj = min(max(box.t0 + j, 0), g.Tn);
        const int ta = min(max(box.t0 + j + off, 0), g.Tn);
        pp[u] = prow[tj];
        pa[u] = parow[ta];
        x[u] = have_px ? pxrow[min(ta, T1 - 1)] : 0.0;
      }
    };
    fetch(0, fp[0], fa[0], fx[0]);
    double up_flow = 0.0, left_flow = 0.0;  // what this lane's last cell sends up / keeps
    double G = 0.0;
    for (int m = 0; m * kEdgeBlock < nsteps; ++m) {
      const int n0 = m * kEdgeBlock;
      double taken = 0.0;
      if (has_below && n0 <= nt) taken = in.Take(m, lane, hdr);
#pragma unroll
      for (int set = 0; set < 2; ++set) {
        const int base = n0 + set * kSet;
        fetch(base + kSet, fp[set ^ 1], fa[set ^ 1], fx[set ^ 1]);
        __builtin_amdgcn_sched_barrier(0);  // the requests stay ahead of the steps
#pragma unroll
        for (int u = 0; u < kSet; ++u) {
          const int n = base + u;
          const int j = nt - n + (kRows - 1 - lane) * skew;
          const bool active = row_ok && j >= 0 && j <= nt;
          double below = FromLaneAbove(up_flow);  // d1 G of cell (i+1, j - off), one step old
          if (has_below) {
            const double e = ReadLane(taken, set * kSet + u);
            if (lane == kRows - 1 && n >= -off && n <= nt) below = e;  // (other words do not exist)
          }
          // this cell's px-edge derivative: 0 where no cell above leads here, 1 in the first
          // column of a regular lattice (p[i][t0] = p[i-1][t0] + px[i-1][t0] exactly)
          bool ok;
          double d1 = PxDerivWave(fa[set][u] + fx[set][u], fp[set][u], &ok);
          const bool none = i == 0 || j + off < 0;
          if (none || j == 0) { d1 = none ? 0.0 : 1.0; ok = true; }
          const bool from_below = i < ns && j - off <= nt;
          double cell = (from_below ? below : 0.0) + (j < nt ? left_flow : 0.0);
          if (i == ns && j == nt) cell = seed;
          const double send_up = ok ? d1 * cell : 0.0;
          const double keep = ok ? (1.0 - d1) * cell : 0.0;
          if (active) {
            G = cell;
            up_flow = send_up;
            left_flow = keep;
            if (i >= 1 && j + off >= 0) gxrow[j] = send_up;
            if (j >= 1) gyrow[j] = keep;
          }
          if (c > 0) {
            // lane 0's cell (64 c, jj) sends into (64 c - 1, jj + off), which the chunk above takes
            // at its step nt - (jj + off)
            const int jj = nt - n + (kRows - 1) * skew;
            const int w = nt - jj - off;
            if (lane == 0 && jj >= 0 && jj <= nt && w >= -off && w <= nt) PublishWord(out, w, up_flow);
          }
        }
      }
    }
    // a lane's last cell is (i, 0): the origin's gradient is what reached the start
    if (i == 0 && overwrite_ans_grad) ans_grad[b] = GaveUp(hdr) ? __builtin_nan("") : G;
  }
  if (lane == 0) PutTicketsBack(hdr, ticket, gridDim.x);
}

// px_grad / py_grad outside the boundary boxes (the sweep assigns everything inside them).
__global__ void MiWaveClearKernel(const int64_t *__restrict__ boundary, double *__restrict__ px_grad,
                                  double *__restrict__ py_grad, int B, int S, int Tn, int modified) {
  const int T1 = modified ? Tn : Tn + 1, off = modified ? -1 : 0;
  const size_t nx = (size_t)B * S * T1, ny = (size_t)B * (S + 1) * Tn;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < nx + ny;
       e += (size_t)gridDim.x * blockDim.x) {
    if (e < nx) {
      const int b = (int)(e / ((size_t)S * T1));
      const size_t r = e - (size_t)b * S * T1;
      const int s = (int)(r / T1), t = (int)(r - (size_t)s * T1);
      const Box box = LoadBox(boundary, b, S, Tn);
      const bool inside = box.ok && s >= box.s0 && s < box.s1 && t >= box.t0 && t <= box.t1 + off;
      if (!inside) px_grad[e] = 0.0;
    } else {
      const size_t k = e - nx;
      const int b = (int)(k / ((size_t)(S + 1) * Tn));
      const size_t r = k - (size_t)b * (S + 1) * Tn;
      const int s = (int)(r / Tn), t = (int)(r - (size_t)s * Tn);
      const Box box = LoadBox(boundary, b, S, Tn);
      const bool inside = box.ok && s >= box.s0 && s <= box.s1 && t >= box.t0 && t < box.t1;
      if (!inside) py_grad[k] = 0.0;
    }
  }
}

int EdgeStride(int Tn) { return (Tn + 2 + kEdgeBlock + 3) / 4 * 4; }

}  // namespace

bool MiWaveSupports(int B, int S, int Tn) {
  return B >= 1 && (long long)B * (S + 1) * (Tn + 1) < (1ll << 31);
}

size_t MiWaveWorkspaceBytes(int B, int S, int Tn) {
  const int nchunks = S / kRows + 1;
  return sizeof(WaveHeader) + (size_t)B * (nchunks + 1) * EdgeStride(Tn) * sizeof(unsigned long long);
}

int MiForwardWave(const double *px, const double *py, const int64_t *boundary, double *p, double *ans,
                  int B, int S, int Tn, int modified, void *workspace, size_t workspace_bytes,
                  hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiWaveWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  WaveHeader *hdr = static_cast<WaveHeader *>(workspace);
  const WaveGeom g{B, S, Tn, S / kRows + 1, EdgeStride(Tn)};
  const dim3 grid((unsigned)(B * g.nchunks)), block(kRows);
  unsigned long long *edge = reinterpret_cast<unsigned long long *>(hdr + 1);
  if (modified)
    hipLaunchKernelGGL(MiWaveForwardKernel<true>, grid, block, 0, stream, px, py, boundary, p, ans, hdr, edge, g);
  else
    hipLaunchKernelGGL(MiWaveForwardKernel<false>, grid, block, 0, stream, px, py, boundary, p, ans, hdr, edge, g);
  return LaunchStatus();
}

int MiBackwardWave(const double *px, const double *p, const int64_t *boundary, double *ans_grad,
                   double *px_grad, double *py_grad, int B, int S, int Tn, int modified,
                   int overwrite_ans_grad, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiWaveWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  WaveHeader *hdr = static_cast<WaveHeader *>(workspace);
  const WaveGeom g{B, S, Tn, S / kRows + 1, EdgeStride(Tn)};
  if (boundary != nullptr)
    hipLaunchKernelGGL(MiWaveClearKernel, dim3(1024), dim3(256), 0, stream, boundary, px_grad, py_grad, B, S,
                       Tn, modified);
  const dim3 grid((unsigned)(B * g.nchunks)), block(kRows);
  unsigned long long *edge = reinterpret_cast<unsigned long long *>(hdr + 1);
  if (modified)
    hipLaunchKernelGGL(MiWaveBackwardKernel<true>, grid, block, 0, stream, px, p, boundary, ans_grad, px_grad,
                       py_grad, hdr, edge, g, overwrite_ans_grad);
  else
    hipLaunchKernelGGL(MiWaveBackwardKernel<false>, grid, block, 0, stream, px, p, boundary, ans_grad, px_grad,
                       py_grad, hdr, edge, g, overwrite_ans_grad);
  return LaunchStatus();
}

}  // namespace k2amd
