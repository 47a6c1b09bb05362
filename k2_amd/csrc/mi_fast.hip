// Throughput path of the fp32 mutual-information recursion on gfx950.
//
// Decomposition.  A sequence's lattice is cut into CHUNKS of 63 consecutive rows (s).  One
// workgroup owns one chunk; the chunks of a sequence form a pipeline, so one sequence draws its
// HBM bandwidth from several compute units (a single workgroup tops out near 100 GB/s on this
// part; 32 sequences alone could never fill 8 TB/s).
//
// Inside a workgroup:
//   * one CHAIN wavefront carries the recursion, lane = lattice row.  Lane l works on column
//     j = n - (l-1)*skew at step n (skew = 1 for the regular lattice, 0 for the modified one), so
//     every cell depends on the previous step only: its own lane's value and the neighbouring
//     lane's, fetched with a DPP wave shift (no LDS, no barrier inside a step).  Lane 0 is a
//     REPLAY lane: it re-emits the last row of the chunk above (or the origin for chunk 0).
//   * seven HELPER wavefronts move data: coalesced global loads of px / py row segments, placed
//     into an LDS ring PRE-SKEWED (element for lane l, step n at ring position n) so the chain
//     wavefront reads 4 steps per lane with one aligned ds_read_b128; results travel the same way
//     back and leave as contiguous row segments.  Loads run two blocks (64 steps) ahead of use.
//   * one barrier per block of 32 steps.
//
// Between workgroups: the last row of a chunk publishes p + px per step into a small edge buffer
// in global memory with device-scope atomic stores; the chunk below polls those words until they
// differ from a sentinel.  Each word is self-validating, so no fences and no cache flushes are
// needed.  Workgroups take their chunk from a ticket counter, which guarantees that the chunk a
// workgroup waits for has already started; every wait is bounded and raises an error flag.
//
// Arithmetic is the reference's log-domain recursion (k2/python/csrc/torch/
// mutual_information_cpu.cu:89-121, log-add of k2/csrc/utils.h:511-563) with hardware exp2/log2.
#include "common.h"
#include "mi_internal.h"

namespace k2amd {
namespace {

constexpr int kRows = 63;             // lattice rows per chunk (lanes 1..63 / 0..62)
constexpr int kW = 32;                // steps per block
constexpr int kRing = 3 * kW;         // ring positions per row
constexpr int kStride = kRing + 4;    // floats per LDS row; +4 spreads lanes over banks
constexpr int kHelperWaves = 7;
constexpr int kFastThreads = kWave * (1 + kHelperWaves);
constexpr int kHelperLanes = kWave * kHelperWaves;
constexpr unsigned kSentinel = 0x7fc5a5a5u;  // a quiet-NaN pattern arithmetic never produces
constexpr int kSpinLimit = 1 << 22;
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

struct FastHeader {
  unsigned ticket;
  unsigned error;
  unsigned pad[62];
};

struct __attribute__((packed, aligned(4))) Quad {
  float v[4];
};

__device__ __forceinline__ float NegInfF() { return -__builtin_huge_valf(); }

// value of lane l-1 (lane 0 keeps `keep`)
__device__ __forceinline__ float WaveShr1(float keep, float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(keep), __float_as_int(v), 0x138,
                                                    0xf, 0xf, false));
}
// value of lane l+1 (lane 63 keeps `keep`)
__device__ __forceinline__ float WaveShl1(float keep, float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(keep), __float_as_int(v), 0x130,
                                                    0xf, 0xf, false));
}

// log(exp(a) + exp(b)) on the fast transcendental units.  Matches k2's log-add to within one
// fp32 rounding of the larger operand: where k2 drops the smaller term (difference below
// log(eps)) the correction computed here is below 1.2e-7.  Two -inf operands give -inf.
__device__ __forceinline__ float LogAddFast(float a, float b) {
  const float mx = fmaxf(a, b), mn = fminf(a, b);
  float d = fmaxf(mn - mx, -126.0f);  // NaN (inf - inf) -> -126
  const float e = __builtin_amdgcn_exp2f(d * kLog2e);
  return __builtin_fmaf(__builtin_amdgcn_logf(1.0f + e), kLn2, mx);
}

struct ChunkGeom {
  int b, c;
  int s0, t0, ns, nt;  // box origin and extent
  int row0;            // local row (s - s0) of the chunk's first lattice row
  int nrows;           // lattice rows in this chunk (1..63)
  int skew;
  int nblocks;
};

__global__ void FastWsInitKernel(FastHeader *hdr, unsigned *edge, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i == 0) {
    hdr->ticket = 0;
    hdr->error = 0;
  }
  for (size_t k = i; k < n; k += (size_t)gridDim.x * blockDim.x) edge[k] = kSentinel;
}

__device__ __forceinline__ float PollEdge(const float *addr, FastHeader *hdr) {
  int spins = 0;
  for (;;) {
    const unsigned v = __hip_atomic_load(reinterpret_cast<const unsigned *>(addr), __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
    if (v != kSentinel) return __uint_as_float(v);
    if (++spins > kSpinLimit) {
      hdr->error = 1;
      return NegInfF();
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

__device__ __forceinline__ void PublishEdge(float *addr, float v) {
  unsigned u = __float_as_uint(v);
  if (u == kSentinel) u = 0x7fc00000u;
  __hip_atomic_store(reinterpret_cast<unsigned *>(addr), u, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------ forward

struct FwdLds {
  float fx[kWave][kStride];
  float fy[kWave][kStride];  // py on the way in, p on the way out (same slots)
  float uin[kRing];
  unsigned ticket;
};

__global__ __launch_bounds__(kFastThreads) void MiForwardFastKernel(
    const float *__restrict__ px, const float *__restrict__ py,
    const int64_t *__restrict__ boundary, float *__restrict__ p, float *__restrict__ ans,
    FastHeader *hdr, float *edge, int S, int Tn, int modified, int nchunks, int edge_stride) {
  __shared__ FwdLds lds;
  if (threadIdx.x == 0) lds.ticket = atomicAdd(&hdr->ticket, 1u);
  __syncthreads();
  ChunkGeom g;
  g.b = lds.ticket / nchunks;
  g.c = lds.ticket % nchunks;
  const Box box = LoadBox(boundary, g.b, S, Tn);
  if (!box.ok) {
    if (g.c == 0 && threadIdx.x == 0) ans[g.b] = __builtin_nanf("");
    return;
  }
  g.s0 = box.s0; g.t0 = box.t0; g.ns = box.s1 - box.s0; g.nt = box.t1 - box.t0;
  g.row0 = g.c * kRows;
  if (g.row0 > g.ns) return;
  g.nrows = min(kRows, g.ns - g.row0 + 1);
  g.skew = modified ? 0 : 1;
  const bool has_down = g.row0 + kRows <= g.ns;
  const int nsteps = g.nt + 2 + (kRows - 1) * g.skew;  // last needed step index + 1
  g.nblocks = (nsteps + kW - 1) / kW;

  const int T1 = modified ? Tn : Tn + 1;
  const float *pxb = px + (size_t)g.b * S * T1;
  const float *pyb = py + (size_t)g.b * (S + 1) * Tn;
  float *pb = p + (size_t)g.b * (S + 1) * (Tn + 1);
  float *edge_out = edge + ((size_t)g.b * nchunks + g.c + 1) * edge_stride;  // read by chunk c+1
  const float *edge_in = edge + ((size_t)g.b * nchunks + g.c) * edge_stride;

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const bool is_chain = wave == 0;
  const int hid = threadIdx.x - kWave;  // helper lane id 0..447 (negative for the chain wave)

  // replay lane's row: fx = 0 (it hands on exactly what it was given), fy = -inf
  for (int i = threadIdx.x; i < kRing; i += kFastThreads) {
    lds.fx[0][i] = 0.0f;
    lds.fy[0][i] = NegInfF();
  }

  // ---- helper-side pieces -------------------------------------------------------------
  // One work item = (row q in 0..62, quad m in 0..7) of a block: four consecutive steps.
  constexpr int kItems = kRows * (kW / 4);
  constexpr int kItemsPerLane = (kItems + kHelperLanes - 1) / kHelperLanes;  // 2
  float4 rx[kItemsPerLane], ry[kItemsPerLane];

  auto load_block = [&](int kb) {
#pragma unroll
    for (int it = 0; it < kItemsPerLane; ++it) {
      const int item = hid + it * kHelperLanes;
      float vx[4], vy[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) vx[e] = vy[e] = NegInfF();
      if (item < kItems && kb < g.nblocks) {
        const int q = item >> 3, m = item & 7;
        const int i = g.row0 + q;                       // local lattice row
        const int jp = kb * kW + 4 * m - 1 - q * g.skew;  // column (relative to t0) of element 0
        if (i <= g.ns) {
          const int s = g.s0 + i;
          const int hi_x = (i < g.ns) ? g.nt - modified : -1;  // last valid px column
          const int hi_y = g.nt - 1;
          const float *xr = pxb + (size_t)s * T1 + g.t0 + jp;
          const float *yr = pyb + (size_t)s * Tn + g.t0 + jp;
          if (i < g.ns) {
            if (jp >= 0 && jp + 3 <= hi_x) {
              const Quad v = *reinterpret_cast<const Quad *>(xr);
#pragma unroll
              for (int e = 0; e < 4; ++e) vx[e] = v.v[e];
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (jp + e >= 0 && jp + e <= hi_x) vx[e] = xr[e];
            }
          }
          if (jp >= 0 && jp + 3 <= hi_y) {
            const Quad v = *reinterpret_cast<const Quad *>(yr);
#pragma unroll
            for (int e = 0; e < 4; ++e) vy[e] = v.v[e];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (jp + e >= 0 && jp + e <= hi_y) vy[e] = yr[e];
          }
        }
      }
      rx[it] = make_float4(vx[0], vx[1], vx[2], vx[3]);
      ry[it] = make_float4(vy[0], vy[1], vy[2], vy[3]);
    }
  };

  auto commit_block = [&](int kb) {  // registers -> LDS ring
    if (kb >= g.nblocks) return;
#pragma unroll
    for (int it = 0; it < kItemsPerLane; ++it) {
      const int item = hid + it * kHelperLanes;
      if (item < kItems) {
        const int q = item >> 3, m = item & 7;
        const int pos = (kb % 3) * kW + 4 * m;
        *reinterpret_cast<float4 *>(&lds.fx[q + 1][pos]) = rx[it];
        *reinterpret_cast<float4 *>(&lds.fy[q + 1][pos]) = ry[it];
      }
    }
  };

  auto store_block = [&](int kb) {  // LDS ring -> p
#pragma unroll
    for (int it = 0; it < kItemsPerLane; ++it) {
      const int item = hid + it * kHelperLanes;
      if (item < kItems) {
        const int q = item >> 3, m = item & 7;
        const int i = g.row0 + q;
        if (i <= g.ns) {
          const int pos = (kb % 3) * kW + 4 * m;
          const float4 v = *reinterpret_cast<const float4 *>(&lds.fy[q + 1][pos]);
          const int j = kb * kW + 4 * m - q * g.skew;  // column of element 0
          float *dst = pb + (size_t)(g.s0 + i) * (Tn + 1) + g.t0 + j;
          const float vv[4] = {v.x, v.y, v.z, v.w};
          if (j >= 0 && j + 3 <= g.nt) {
            Quad o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o.v[e] = vv[e];
            *reinterpret_cast<Quad *>(dst) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (j + e >= 0 && j + e <= g.nt) dst[e] = vv[e];
          }
          if (i == g.ns) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (j + e == g.nt) ans[g.b] = vv[e];
          }
        }
      }
    }
  };

  auto load_uin = [&](int kb) {  // helper lanes 0..31: the replay lane's inputs for block kb
    if (hid >= 0 && hid < kW && kb < g.nblocks) {
      const int n = kb * kW + hid;
      float v;
      if (g.c == 0) {
        v = (n == 0) ? 0.0f : NegInfF();
      } else {
        const int idx = n + kRows * g.skew;
        // the chunk above publishes exactly nblocks * kW steps
        v = (idx < g.nblocks * kW) ? PollEdge(edge_in + idx, hdr) : NegInfF();
      }
      lds.uin[(kb % 3) * kW + hid] = v;
    }
  };

  // ---- prologue: blocks 0 and 1 in flight ------------------------------------------------
  if (!is_chain) {
    load_block(0);
    commit_block(0);
    load_uin(0);
    load_block(1);
  }
  float P = NegInfF();
  __syncthreads();

  for (int kb = 0; kb < g.nblocks; ++kb) {
    if (!is_chain) {
      // block kb+1 sits in registers (loaded one iteration ago); put it into the ring, start
      // the loads of block kb+2, and drain block kb-1.
      commit_block(kb + 1);
      load_uin(kb + 1);
      load_block(kb + 2);
      if (kb >= 1) store_block(kb - 1);
    } else {
      const int base = (kb % 3) * kW;
#pragma unroll 2
      for (int m = 0; m < kW / 4; ++m) {
        const int pos = base + 4 * m;
        const float4 fx4 = *reinterpret_cast<const float4 *>(&lds.fx[lane][pos]);
        const float4 fy4 = *reinterpret_cast<const float4 *>(&lds.fy[lane][pos]);
        const float4 u4 = *reinterpret_cast<const float4 *>(&lds.uin[pos]);
        const float fxs[4] = {fx4.x, fx4.y, fx4.z, fx4.w};
        const float fys[4] = {fy4.x, fy4.y, fy4.z, fy4.w};
        const float uis[4] = {u4.x, u4.y, u4.z, u4.w};
        float out[4], us[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (lane == 0) P = uis[e];
          const float u = P + fxs[e];
          const float x = P + fys[e];
          const float inc = WaveShr1(NegInfF(), u);
          P = LogAddFast(inc, x);
          out[e] = P;
          us[e] = u;
        }
        *reinterpret_cast<float4 *>(&lds.fy[lane][pos]) = make_float4(out[0], out[1], out[2], out[3]);
        if (has_down && lane == kWave - 1) {
          const int n = kb * kW + 4 * m;
#pragma unroll
          for (int e = 0; e < 4; ++e) PublishEdge(edge_out + n + e, us[e]);
        }
      }
    }
    __syncthreads();
  }
  if (!is_chain) store_block(g.nblocks - 1);
}


// ------------------------------------------------------------------------------ backward
//
// Mass-flow form of the reference's backward sweep (k2/python/csrc/torch/
// mutual_information_cpu.cu:179-251).  For a destination cell D = (s, t) that holds gradient g:
//     d1 = exp(p[s-1][t+o] + px[s-1][t+o] - p[s][t])        (o = -1 modified, 0 regular)
//     h  = d1 * g        -> px_grad[s-1][t+o], and flows to cell (s-1, t+o)
//     c  = (1 - d1) * g  -> py_grad[s][t-1],   and flows to cell (s, t-1)
// so every cell needs ONE exponential, computed by the helper wavefronts (E = d1, OME = 1 - d1,
// with the reference's guards folded in: first row E = 0, first column of a regular lattice
// E = 1, non-finite d1 -> both 0).  The chain wavefront then does, per position m (descending),
//     h = E * G;  c = OME * G;  G = h(lane + 1) + c
// i.e. two multiplies and one DPP add.  Lane l handles lattice row row0 + l; lane 63 replays the
// h values of the first row of the chunk below, so here the LOWER chunk runs ahead.
struct BwdLds {
  float e[kWave][kStride];    // d1 on the way in, h (px_grad) on the way out
  float ome[kWave][kStride];  // 1 - d1 on the way in, c (py_grad) on the way out
  float rin[kRing];
  unsigned ticket;
};

__global__ __launch_bounds__(kFastThreads) void MiBackwardFastKernel(
    const float *__restrict__ px, const float *__restrict__ p,
    const int64_t *__restrict__ boundary, float *__restrict__ ans_grad,
    float *__restrict__ px_grad, float *__restrict__ py_grad, FastHeader *hdr, float *edge, int S,
    int Tn, int modified, int nchunks, int edge_stride, int overwrite_ans_grad) {
  __shared__ BwdLds lds;
  if (threadIdx.x == 0) lds.ticket = atomicAdd(&hdr->ticket, 1u);
  __syncthreads();
  ChunkGeom g;
  g.b = lds.ticket / nchunks;
  g.c = nchunks - 1 - (int)(lds.ticket % nchunks);  // lower chunks take earlier tickets
  const Box box = LoadBox(boundary, g.b, S, Tn);
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  const float *pxb = px + (size_t)g.b * S * T1;
  const float *pb = p + (size_t)g.b * (S + 1) * (Tn + 1);
  float *gxb = px_grad + (size_t)g.b * S * T1;
  float *gyb = py_grad + (size_t)g.b * (S + 1) * Tn;

  // Zero everything the sweep does not assign, for the rows this workgroup is responsible for
  // BY ARRAY ROW (independent of the box), so every element of both outputs is written once.
  {
    const int r_lo = g.c * kRows, r_hi = min(r_lo + kRows, S + 1);
    const int xs0 = box.ok ? box.s0 : 0, xs1 = box.ok ? box.s1 : 0;
    const int xt0 = box.ok ? box.t0 : 0, xt1 = box.ok ? box.t1 + off + 1 : 0;
    const int ys1 = box.ok ? box.s1 + 1 : 0, yt1 = box.ok ? box.t1 : 0;
    for (int r = r_lo; r < r_hi; ++r) {
      if (r < S) {
        const bool row_in = r >= xs0 && r < xs1;
        for (int t = threadIdx.x; t < T1; t += kFastThreads)
          if (!(row_in && t >= xt0 && t < xt1)) gxb[(size_t)r * T1 + t] = 0.0f;
      }
      const bool row_in = r >= xs0 && r < ys1;
      for (int t = threadIdx.x; t < Tn; t += kFastThreads)
        if (!(row_in && t >= xt0 && t < yt1)) gyb[(size_t)r * Tn + t] = 0.0f;
    }
  }
  if (!box.ok) return;
  g.s0 = box.s0; g.t0 = box.t0; g.ns = box.s1 - box.s0; g.nt = box.t1 - box.t0;
  g.row0 = g.c * kRows;
  if (g.row0 > g.ns) return;
  g.nrows = min(kRows, g.ns - g.row0 + 1);
  g.skew = modified ? 0 : 1;
  const bool has_down = g.row0 + kRows <= g.ns;
  const bool has_up = g.c > 0;
  const int npos = g.nt + 2 + (kRows - 1) * g.skew;
  g.nblocks = (npos + kW - 1) / kW;
  float *edge_out = edge + ((size_t)g.b * nchunks + g.c) * edge_stride;            // read by c-1
  const float *edge_in = edge + ((size_t)g.b * nchunks + g.c + 1) * edge_stride;   // from c+1

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const bool is_chain = wave == 0;
  const int hid = threadIdx.x - kWave;

  // lane 63 is the replay lane: its E / OME rows are never used (h is overwritten, c is unused)
  for (int i = threadIdx.x; i < kRing; i += kFastThreads) {
    lds.e[kWave - 1][i] = 0.0f;
    lds.ome[kWave - 1][i] = 0.0f;
  }

  constexpr int kItems = kRows * (kW / 4);
  constexpr int kItemsPerLane = (kItems + kHelperLanes - 1) / kHelperLanes;
  float4 re[kItemsPerLane], ro[kItemsPerLane];

  // E / OME of the four destination cells (row q, positions kb*32 + 4m .. +3)
  auto load_block = [&](int kb) {
#pragma unroll
    for (int it = 0; it < kItemsPerLane; ++it) {
      const int item = hid + it * kHelperLanes;
      float ve[4] = {0.f, 0.f, 0.f, 0.f}, vo[4] = {0.f, 0.f, 0.f, 0.f};
      if (item < kItems && kb >= 0) {
        const int q = item >> 3, m = item & 7;
        const int i = g.row0 + q;
        const int jd = kb * kW + 4 * m - q * g.skew;  // destination column of element 0
        if (i <= g.ns) {
          const int s = g.s0 + i;
          if (i == 0) {
            // first row: everything flows along py; beyond the end cell nothing flows, except
            // that the last row carries the seed towards the end cell (see below)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (jd + e >= 1 && jd + e <= g.nt) vo[e] = 1.0f;
          } else {
            const int js = jd - 1 + g.skew;  // source column of the px edge of element 0
            const float *pd = pb + (size_t)s * (Tn + 1) + g.t0 + jd;
            const float *ps = pb + (size_t)(s - 1) * (Tn + 1) + g.t0 + js;
            const float *xs = pxb + (size_t)(s - 1) * T1 + g.t0 + js;
            float vd[4], vs[4], vx[4];
            if (jd >= 1 && jd + 3 <= g.nt) {
              const Quad a = *reinterpret_cast<const Quad *>(pd);
              const Quad bq = *reinterpret_cast<const Quad *>(ps);
              const Quad cq = *reinterpret_cast<const Quad *>(xs);
#pragma unroll
              for (int e = 0; e < 4; ++e) { vd[e] = a.v[e]; vs[e] = bq.v[e]; vx[e] = cq.v[e]; }
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const bool in = jd + e >= 1 && jd + e <= g.nt;
                vd[e] = in ? pd[e] : 0.0f;
                vs[e] = in ? ps[e] : 0.0f;
                vx[e] = in ? xs[e] : 0.0f;
              }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int j = jd + e;
              if (j >= 1 && j <= g.nt) {
                float total = vd[e];
                if (total - total != 0.0f) total = 0.0f;
                const float d1 = __expf((vs[e] + vx[e]) - total);
                if (d1 - d1 == 0.0f) { ve[e] = d1; vo[e] = 1.0f - d1; }
              } else if (j == 0 && !modified) {
                ve[e] = 1.0f;  // first column of a regular lattice: all of it flows up
              }
            }
          }
          if (i == g.ns) {
            // virtual cells right of the end cell hand the seed leftwards unchanged
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (jd + e > g.nt) { ve[e] = 0.0f; vo[e] = 1.0f; }
          }
        }
      }
      re[it] = make_float4(ve[0], ve[1], ve[2], ve[3]);
      ro[it] = make_float4(vo[0], vo[1], vo[2], vo[3]);
    }
  };

  auto commit_block = [&](int kb) {
    if (kb < 0) return;
#pragma unroll
    for (int it = 0; it < kItemsPerLane; ++it) {
      const int item = hid + it * kHelperLanes;
      if (item < kItems) {
        const int q = item >> 3, m = item & 7;
        const int pos = (kb % 3) * kW + 4 * m;
        *reinterpret_cast<float4 *>(&lds.e[q][pos]) = re[it];
        *reinterpret_cast<float4 *>(&lds.ome[q][pos]) = ro[it];
      }
    }
  };

  auto store_block = [&](int kb) {
#pragma unroll
    for (int it = 0; it < kItemsPerLane; ++it) {
      const int item = hid + it * kHelperLanes;
      if (item < kItems) {
        const int q = item >> 3, m = item & 7;
        const int i = g.row0 + q;
        if (i <= g.ns) {
          const int pos = (kb % 3) * kW + 4 * m;
          const float4 h4 = *reinterpret_cast<const float4 *>(&lds.e[q][pos]);
          const float4 c4 = *reinterpret_cast<const float4 *>(&lds.ome[q][pos]);
          const float hv[4] = {h4.x, h4.y, h4.z, h4.w}, cv[4] = {c4.x, c4.y, c4.z, c4.w};
          const int jd = kb * kW + 4 * m - q * g.skew;
          const int s = g.s0 + i;
          // py_grad[s][t0 + jd - 1 + e]   for destination columns 1..nt
          float *dy = gyb + (size_t)s * Tn + g.t0 + jd - 1;
          if (jd >= 1 && jd + 3 <= g.nt) {
            Quad o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o.v[e] = cv[e];
            *reinterpret_cast<Quad *>(dy) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (jd + e >= 1 && jd + e <= g.nt) dy[e] = cv[e];
          }
          // px_grad[s-1][t0 + jd - 1 + skew + e]   for destination columns (1 - skew)..nt
          if (i >= 1) {
            float *dx = gxb + (size_t)(s - 1) * T1 + g.t0 + jd - 1 + g.skew;
            const int lo = 1 - g.skew;
            if (jd >= lo && jd + 3 <= g.nt) {
              Quad o;
#pragma unroll
              for (int e = 0; e < 4; ++e) o.v[e] = hv[e];
              *reinterpret_cast<Quad *>(dx) = o;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (jd + e >= lo && jd + e <= g.nt) dx[e] = hv[e];
            }
          }
        }
      }
    }
  };

  auto load_rin = [&](int kb) {
    if (hid >= 0 && hid < kW && kb >= 0) {
      const int mpos = kb * kW + hid;
      float v = 0.0f;
      if (has_down) {
        const int idx = mpos - kRows * g.skew;
        if (idx >= 0 && idx < g.nblocks * kW) v = PollEdge(edge_in + idx, hdr);
      }
      lds.rin[(kb % 3) * kW + hid] = v;
    }
  };

  const int top = g.nblocks - 1;
  if (!is_chain) {
    load_block(top);
    commit_block(top);
    load_rin(top);
    load_block(top - 1);
  }
  // gradient at the (virtual) right end of each row: the seed on the sequence's last row
  float G = 0.0f;
  if (is_chain && g.row0 + lane == g.ns && lane < kRows) G = ans_grad[g.b];
  float g_origin = 0.0f;
  __syncthreads();

  for (int kb = top; kb >= 0; --kb) {
    if (!is_chain) {
      commit_block(kb - 1);
      load_rin(kb - 1);
      load_block(kb - 2);
      if (kb < top) store_block(kb + 1);
    } else {
      const int base = (kb % 3) * kW;
#pragma unroll 2
      for (int m = kW / 4 - 1; m >= 0; --m) {
        const int pos = base + 4 * m;
        const float4 e4 = *reinterpret_cast<const float4 *>(&lds.e[lane][pos]);
        const float4 o4 = *reinterpret_cast<const float4 *>(&lds.ome[lane][pos]);
        const float4 r4 = *reinterpret_cast<const float4 *>(&lds.rin[pos]);
        const float es[4] = {e4.x, e4.y, e4.z, e4.w};
        const float os[4] = {o4.x, o4.y, o4.z, o4.w};
        const float rs[4] = {r4.x, r4.y, r4.z, r4.w};
        float hs[4], cs[4];
#pragma unroll
        for (int e = 3; e >= 0; --e) {
          if (kb == 0 && m == 0 && e == 0) g_origin = G;
          float h = es[e] * G;
          const float c = os[e] * G;
          if (lane == kWave - 1) h = rs[e];
          G = WaveShl1(0.0f, h) + c;
          hs[e] = h;
          cs[e] = c;
        }
        *reinterpret_cast<float4 *>(&lds.e[lane][pos]) = make_float4(hs[0], hs[1], hs[2], hs[3]);
        *reinterpret_cast<float4 *>(&lds.ome[lane][pos]) = make_float4(cs[0], cs[1], cs[2], cs[3]);
        if (has_up && lane == 0) {
          const int mpos = kb * kW + 4 * m;
#pragma unroll
          for (int e = 0; e < 4; ++e) PublishEdge(edge_out + mpos + e, hs[e]);
        }
      }
    }
    __syncthreads();
  }
  if (!is_chain) store_block(0);
  if (overwrite_ans_grad && is_chain && g.c == 0 && lane == 0) ans_grad[g.b] = g_origin;
}

}  // namespace

size_t MiFastWorkspaceBytes(int B, int S, int Tn) {
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const size_t edge_stride = ((size_t)Tn + 2 + kRows + kW + 3) / 4 * 4 + kW;
  return sizeof(FastHeader) + (size_t)B * (nchunks + 1) * edge_stride * sizeof(float);
}

int MiForwardFast(const float *px, const float *py, const int64_t *boundary, float *p, float *ans,
                  int B, int S, int Tn, int modified, void *workspace, size_t workspace_bytes,
                  hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiFastWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const int edge_stride = (int)(((size_t)Tn + 2 + kRows + kW + 3) / 4 * 4 + kW);
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  float *edge = reinterpret_cast<float *>(hdr + 1);
  const size_t n_edge = (size_t)B * (nchunks + 1) * edge_stride;
  hipLaunchKernelGGL(FastWsInitKernel, dim3((unsigned)min((size_t)256, (n_edge + 255) / 256)), dim3(256), 0,
                     stream, hdr, reinterpret_cast<unsigned *>(edge), n_edge);
  hipLaunchKernelGGL(MiForwardFastKernel, dim3((unsigned)(B * nchunks)), dim3(kFastThreads), 0, stream,
                     px, py, boundary, p, ans, hdr, edge, S, Tn, modified, nchunks, edge_stride);
  return LaunchStatus();
}


int MiBackwardFast(const float *px, const float *p, const int64_t *boundary, float *ans_grad,
                   float *px_grad, float *py_grad, int B, int S, int Tn, int modified,
                   int overwrite_ans_grad, void *workspace, size_t workspace_bytes,
                   hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiFastWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const int edge_stride = (int)(((size_t)Tn + 2 + kRows + kW + 3) / 4 * 4 + kW);
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  float *edge = reinterpret_cast<float *>(hdr + 1);
  const size_t n_edge = (size_t)B * (nchunks + 1) * edge_stride;
  hipLaunchKernelGGL(FastWsInitKernel, dim3((unsigned)min((size_t)256, (n_edge + 255) / 256)), dim3(256), 0,
                     stream, hdr, reinterpret_cast<unsigned *>(edge), n_edge);
  hipLaunchKernelGGL(MiBackwardFastKernel, dim3((unsigned)(B * nchunks)), dim3(kFastThreads), 0, stream,
                     px, p, boundary, ans_grad, px_grad, py_grad, hdr, edge, S, Tn, modified, nchunks,
                     edge_stride, overwrite_ans_grad);
  return LaunchStatus();
}

}  // namespace k2amd
