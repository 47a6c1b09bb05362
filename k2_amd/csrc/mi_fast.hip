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
// differ from a sentinel, and writes the sentinel back once it has the value, so the buffer is
// clean again when the kernel ends.  Each word is self-validating, so no fences and no cache
// flushes are needed.  Workgroups take their chunk from a ticket counter, which guarantees that
// the chunk a workgroup waits for has already started; the last workgroup to finish resets the
// counter.  The workspace therefore needs ONE initialisation (MiFastWorkspaceInit) and no
// per-call setup kernel.  Every wait is bounded; a timeout raises the header's error flag, after
// which every later wait returns at once.
//
// Arithmetic is the reference's log-domain recursion (k2/python/csrc/torch/
// mutual_information_cpu.cu:89-121, log-add of k2/csrc/utils.h:511-563) with hardware exp2/log2.
#include "common.h"
#include "mi_internal.h"

namespace k2amd {
namespace {

constexpr int kRows = 64;             // lattice rows per chunk, one per lane of the chain wavefront
constexpr int kW = 32;                // steps per block
constexpr int kRing = 3 * kW;         // ring positions per row
constexpr int kStride = kRing + 4;    // floats per LDS row; +4 spreads lanes over banks
constexpr int kHelperWaves = 8;
constexpr int kFastThreads = kWave * (1 + kHelperWaves);
constexpr int kHelperLanes = kWave * kHelperWaves;
constexpr unsigned kSentinel = 0x7fc5a5a5u;  // a quiet-NaN pattern arithmetic never produces
constexpr int kSpinLimit = 1 << 20;
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

struct FastHeader {
  unsigned ticket;  // next chunk to hand out; reset by the last workgroup of a launch
  unsigned done;    // workgroups finished in this launch
  unsigned error;   // set when a bounded wait timed out (sticky until re-initialised)
  unsigned pad[61];
};

struct __attribute__((packed, aligned(4))) Quad {
  float v[4];
};

__device__ __forceinline__ float NegInfF() { return -__builtin_huge_valf(); }

// Inside the forward chain "minus infinity" is this finite stand-in: differences of two such
// values are finite, so the log-add needs no NaN guard on its critical path.  Helpers translate
// at the LDS boundary in both directions.
constexpr float kLogZero = -1.0e30f;
constexpr float kLogZeroTest = -1.0e29f;  // anything below counts as -inf when p leaves the chain

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

// log(exp(a) + exp(b)) for FINITE a, b on the fast transcendental units: max + log1p(exp(-|a-b|)).
// Matches k2's log-add to within one fp32 rounding of the larger operand: where k2 drops the
// smaller term (difference below log(eps)) the correction computed here is below 1.2e-7.
// Dependent chain: sub, mul (|.| and negation are free source modifiers), exp2, add, log2, fma.
__device__ __forceinline__ float LogAddFinite(float a, float b) {
  const float mx = __builtin_fmaxf(a, b);  // off the critical path
  const float e = __builtin_amdgcn_exp2f(-__builtin_fabsf(a - b) * kLog2e);
  return __builtin_fmaf(__builtin_amdgcn_logf(1.0f + e), kLn2, mx);
}

// lane l gets  P(lane l-1) + add ; lane 0, which has no lane below it, keeps `lane0`.
__device__ __forceinline__ float ShiftAdd(float lane0, float P, float add) {
  float r = lane0;
  // a DPP source written by the preceding VALU instruction needs two wait states; inline
  // assembly is opaque to the compiler's hazard recogniser, so they are spelled out here
  asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %1, %2 wave_shr:1 row_mask:0xf bank_mask:0xf"
               : "+v"(r)
               : "v"(P), "v"(add));
  return r;
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
    hdr->done = 0;
    hdr->error = 0;
  }
  for (size_t k = i; k < n; k += (size_t)gridDim.x * blockDim.x) edge[k] = kSentinel;
}

// Waits for one published word, takes it and leaves the sentinel behind.
__device__ __forceinline__ float TakeEdge(float *addr, FastHeader *hdr, float on_timeout) {
  unsigned *word = reinterpret_cast<unsigned *>(addr);
  int spins = 0;
  for (;;) {
    const unsigned v = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (v != kSentinel) {
      __hip_atomic_store(word, kSentinel, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return __uint_as_float(v);
    }
    ++spins;
    if ((spins & 255) == 0 &&
        __hip_atomic_load(&hdr->error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)
      return on_timeout;
    if (spins > kSpinLimit) {
      __hip_atomic_store(&hdr->error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return on_timeout;
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

// Called by one thread after the workgroup's last barrier.
__device__ __forceinline__ void FinishWorkgroup(FastHeader *hdr, unsigned total) {
  const unsigned n = atomicAdd(&hdr->done, 1u);
  if (n + 1 == total) {
    __hip_atomic_store(&hdr->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&hdr->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

__device__ __forceinline__ void PublishEdge(float *addr, float v) {
  unsigned u = __float_as_uint(v);
  if (u == kSentinel) u = 0x7fc00000u;
  __hip_atomic_store(reinterpret_cast<unsigned *>(addr), u, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// ------------------------------------------------------------------------------ helpers' tiles
//
// One helper work item = (row q in 0..62, quad m in 0..7) of a block: four consecutive steps of
// one lattice row; 504 items per block, one per helper lane.  Loads are issued RAW and
// branch-free (addresses clamped into the valid region; validity is applied when the registers
// are committed to LDS two iterations later), so no wavefront ever waits on a load inside the
// iteration that issued it.
constexpr int kItems = kRows * (kW / 4);
static_assert(kItems <= kHelperLanes, "one work item per helper lane");
constexpr int kQuadsPerRow = kStride / 4;
constexpr int kQuadsPerBlock = kW / 4;

__device__ __forceinline__ float4 LoadQuad(const float *ptr) {
  const Quad v = *reinterpret_cast<const Quad *>(ptr);
  return make_float4(v.v[0], v.v[1], v.v[2], v.v[3]);
}
__device__ __forceinline__ void StoreQuad(float *ptr, float4 v) {
  Quad o;
  o.v[0] = v.x; o.v[1] = v.y; o.v[2] = v.z; o.v[3] = v.w;
  *reinterpret_cast<Quad *>(ptr) = o;
}
// four columns j0..j0+3 of one row, each clamped into [lo, hi] (hi >= lo)
__device__ __forceinline__ float4 LoadClamped(const float *row, int j0, int lo, int hi) {
  float4 r;
  r.x = row[min(max(j0 + 0, lo), hi)];
  r.y = row[min(max(j0 + 1, lo), hi)];
  r.z = row[min(max(j0 + 2, lo), hi)];
  r.w = row[min(max(j0 + 3, lo), hi)];
  return r;
}

// ------------------------------------------------------------------------------ forward
//
// Lane q of the chain wavefront owns lattice row row0 + q and is at column j = n - q*skew at step
// n.  Ring position n of a lane's LDS row holds what the step into column j needs:
//     fx[q][n] = px[row-1][jp + skew]   (the px edge arriving from the row above)
//     fy[q][n] = py[row][jp]            (the py edge arriving from the left),  jp = j - 1
// and receives p[row][j] in place of fy once the step is done.  Lane 0's "row above" is the
// last row of the chunk above; its p arrives through uin[n].
struct FwdLds {
  float4 fx[kWave][kQuadsPerRow];
  float4 fy[kWave][kQuadsPerRow];
  float4 uin[kRing / 4];
  unsigned ticket;
};

struct FwdRegs {
  float4 x, y;
};

__global__ __launch_bounds__(kFastThreads) void MiForwardFastKernel(
    const float *__restrict__ px, const float *__restrict__ py,
    const int64_t *__restrict__ boundary, float *__restrict__ p, float *__restrict__ ans,
    FastHeader *hdr, float *edge, int S, int Tn, int modified, int nchunks, int edge_stride) {
  __shared__ FwdLds lds;
  const unsigned total_wgs = gridDim.x;
  if (threadIdx.x == 0) lds.ticket = atomicAdd(&hdr->ticket, 1u);
  __syncthreads();
  ChunkGeom g;
  g.b = lds.ticket / nchunks;
  g.c = lds.ticket % nchunks;
  const Box box = LoadBox(boundary, g.b, S, Tn);
  g.s0 = box.s0; g.t0 = box.t0; g.ns = box.s1 - box.s0; g.nt = box.t1 - box.t0;
  g.row0 = g.c * kRows;
  if (!box.ok || g.row0 > g.ns) {
    if (!box.ok && g.c == 0 && threadIdx.x == 0) ans[g.b] = __builtin_nanf("");
    if (threadIdx.x == 0) FinishWorkgroup(hdr, total_wgs);
    return;
  }
  g.nrows = min(kRows, g.ns - g.row0 + 1);
  g.skew = modified ? 0 : 1;
  const bool has_down = g.row0 + kRows <= g.ns;
  const int nsteps = g.nt + 1 + (kRows - 1) * g.skew;  // last needed step index + 1
  g.nblocks = (nsteps + kW - 1) / kW;
  const int edge_shift = kRows * g.skew - 1;  // step n here <-> step n + edge_shift one chunk up

  const int T1 = modified ? Tn : Tn + 1;
  const float *pxb = px + (size_t)g.b * S * T1;
  const float *pyb = py + (size_t)g.b * (S + 1) * Tn;
  float *pb = p + (size_t)g.b * (S + 1) * (Tn + 1);
  float *edge_out = edge + ((size_t)g.b * nchunks + g.c + 1) * edge_stride;  // read by chunk c+1
  float *edge_in = edge + ((size_t)g.b * nchunks + g.c) * edge_stride;

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const bool is_chain = wave == 0;
  const int hid = threadIdx.x - kWave;  // helper lane id (negative for the chain wave)
  const bool has_item = hid >= 0 && hid < kItems;
  const int item = min(max(hid, 0), kItems - 1);
  const int q = item >> 3, m = item & 7;  // this helper lane's row and quad
  const int row_i = g.row0 + q;           // local lattice row

  const int hi_x = g.nt - modified, hi_y = g.nt - 1;  // last valid px / py column
  const bool row_x = row_i >= 1 && row_i <= g.ns, row_y = row_i <= g.ns;
  const bool any_x = g.ns >= 1 && hi_x >= 0, any_y = hi_y >= 0;
  const float *xrow = pxb + (size_t)(g.s0 + min(max(row_i, 1), max(g.ns, 1)) - 1) * T1 + g.t0;
  const float *yrow = pyb + (size_t)(g.s0 + min(row_i, g.ns)) * Tn + g.t0;

  auto load_block = [&](int kb, FwdRegs &r) {
    if (kb >= g.nblocks || !has_item) return;
    // every quad of every row of this block inside the valid columns?  (uniform)
    const bool interior = kb * kW - 1 - (kRows - 1) * g.skew >= 0 && kb * kW + 30 <= g.nt - 1;
    const int jp = kb * kW + 4 * m - 1 - q * g.skew;  // column left of element 0's cell
    if (interior) {
      if (any_x) r.x = LoadQuad(xrow + jp + g.skew);
      r.y = LoadQuad(yrow + jp);
    } else {
      if (any_x) r.x = LoadClamped(xrow, jp + g.skew, 0, hi_x);
      if (any_y) r.y = LoadClamped(yrow, jp, 0, hi_y);
    }
  };

  auto commit_block = [&](int kb, const FwdRegs &r) {  // registers -> LDS ring
    if (kb >= g.nblocks || !has_item) return;
    const int jp = kb * kW + 4 * m - 1 - q * g.skew;
    const int jx = jp + g.skew;
    float4 vx, vy;
    vx.x = (row_x && jx + 0 >= 0 && jx + 0 <= hi_x) ? fmaxf(r.x.x, kLogZero) : kLogZero;
    vx.y = (row_x && jx + 1 >= 0 && jx + 1 <= hi_x) ? fmaxf(r.x.y, kLogZero) : kLogZero;
    vx.z = (row_x && jx + 2 >= 0 && jx + 2 <= hi_x) ? fmaxf(r.x.z, kLogZero) : kLogZero;
    vx.w = (row_x && jx + 3 >= 0 && jx + 3 <= hi_x) ? fmaxf(r.x.w, kLogZero) : kLogZero;
    vy.x = (row_y && jp + 0 >= 0 && jp + 0 <= hi_y) ? fmaxf(r.y.x, kLogZero) : kLogZero;
    vy.y = (row_y && jp + 1 >= 0 && jp + 1 <= hi_y) ? fmaxf(r.y.y, kLogZero) : kLogZero;
    vy.z = (row_y && jp + 2 >= 0 && jp + 2 <= hi_y) ? fmaxf(r.y.z, kLogZero) : kLogZero;
    vy.w = (row_y && jp + 3 >= 0 && jp + 3 <= hi_y) ? fmaxf(r.y.w, kLogZero) : kLogZero;
    // the origin: p[s_begin][t_begin] = 0 enters as "0 arriving from above" at step 0
    if (row_i == 0 && kb == 0 && m == 0) vx.x = 0.0f;
    const int pq = (kb % 3) * kQuadsPerBlock + m;
    lds.fx[q][pq] = vx;
    lds.fy[q][pq] = vy;
  };

  auto store_block = [&](int kb) {  // LDS ring -> p
    if (kb < 0 || !has_item || row_i > g.ns) return;
    float4 v = lds.fy[q][(kb % 3) * kQuadsPerBlock + m];
    const float ninf = NegInfF();
    v.x = v.x < kLogZeroTest ? ninf : v.x;
    v.y = v.y < kLogZeroTest ? ninf : v.y;
    v.z = v.z < kLogZeroTest ? ninf : v.z;
    v.w = v.w < kLogZeroTest ? ninf : v.w;
    const int j = kb * kW + 4 * m - q * g.skew;  // column of element 0
    float *dst = pb + (size_t)(g.s0 + row_i) * (Tn + 1) + g.t0 + j;
    const float vv[4] = {v.x, v.y, v.z, v.w};
    if (j >= 0 && j + 3 <= g.nt) {
      StoreQuad(dst, v);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (j + e >= 0 && j + e <= g.nt) dst[e] = vv[e];
    }
    if (row_i == g.ns) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (j + e == g.nt) ans[g.b] = vv[e];
    }
  };

  // helper wavefront 1, lanes 0..31: p of the row above lane 0 for block kb
  auto load_uin = [&](int kb) {
    if (hid >= 0 && hid < kW && kb < g.nblocks) {
      const int n = kb * kW + hid;
      float v = kLogZero;
      if (g.c == 0) {
        if (n == 0) v = 0.0f;  // pairs with the 0 placed in fx[0][0]
      } else {
        const int idx = n + edge_shift;
        if (idx >= 0 && idx < g.nblocks * kW) v = TakeEdge(edge_in + idx, hdr, kLogZero);
      }
      reinterpret_cast<float *>(lds.uin)[(kb % 3) * kW + hid] = v;
    }
  };

  // helper wavefront 2, lanes 0..31: hand block kb of the last row to the chunk below.  Only
  // words the chunk below will take are published, so the buffer ends the launch clean.
  auto publish = [&](int kb) {
    if (has_down && kb >= 0 && hid >= kWave && hid < kWave + kW) {
      const int n = kb * kW + (hid - kWave);
      // the chunk below takes word n at its step n - edge_shift, which must exist
      if (n >= edge_shift && n - edge_shift < g.nblocks * kW)
        PublishEdge(edge_out + n, reinterpret_cast<const float *>(&lds.fy[kWave - 1][0])[(kb % 3) * kW + (hid - kWave)]);
    }
  };

  float P = kLogZero;
  auto chain_block = [&](int kb) {
    const int base = (kb % 3) * kQuadsPerBlock;
    P = fmaxf(P, -1.0e36f);  // lanes idling on the stand-in for -inf must never reach -inf itself
    float4 nfx = lds.fx[lane][base], nfy = lds.fy[lane][base], nu = lds.uin[base];
#pragma unroll
    for (int mm = 0; mm < kQuadsPerBlock; ++mm) {
      const float4 fx4 = nfx, fy4 = nfy, u4 = nu;
      if (mm + 1 < kQuadsPerBlock) {
        nfx = lds.fx[lane][base + mm + 1];
        nfy = lds.fy[lane][base + mm + 1];
        nu = lds.uin[base + mm + 1];
      }
      const float fxs[4] = {fx4.x, fx4.y, fx4.z, fx4.w};
      const float fys[4] = {fy4.x, fy4.y, fy4.z, fy4.w};
      const float uis[4] = {u4.x, u4.y, u4.z, u4.w};
      float out[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x = P + fys[e];                              // arriving along py
        const float inc = ShiftAdd(uis[e] + fxs[e], P, fxs[e]);  // arriving along px
        P = LogAddFinite(inc, x);
        out[e] = P;
      }
      lds.fy[lane][base + mm] = make_float4(out[0], out[1], out[2], out[3]);
    }
  };

  // ---- prologue: block 0 committed, blocks 1 and 2 in flight ---------------------------------
  FwdRegs ra, rb;
  if (!is_chain) {
    load_block(0, ra);
    commit_block(0, ra);
    load_uin(0);
    load_block(1, ra);
    load_block(2, rb);
  }
  __syncthreads();

  // One iteration: the chain wavefront computes block kb while the helpers commit block kb+1
  // (loaded two iterations ago), start the loads of block kb+3, and drain block kb-1.
  auto iteration = [&](int kb, FwdRegs &r) {
    if (!is_chain) {
      publish(kb - 1);
      commit_block(kb + 1, r);
      load_uin(kb + 1);
      load_block(kb + 3, r);
      store_block(kb - 1);
    } else {
      chain_block(kb);
    }
    __syncthreads();
  };
  for (int kb = 0; kb < g.nblocks; kb += 2) {
    iteration(kb, ra);
    if (kb + 1 < g.nblocks) iteration(kb + 1, rb);
  }
  if (!is_chain) {
    publish(g.nblocks - 1);
    store_block(g.nblocks - 1);
  }
  if (threadIdx.x == 0) FinishWorkgroup(hdr, total_wgs);
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
// i.e. two multiplies, one DPP move and one add.  Lane l handles lattice row row0 + l; lane 63
// has no lane above it in the wavefront and receives, through the DPP's "old" operand, the h of
// the first row of the chunk below, so here the LOWER chunk runs ahead.
struct BwdLds {
  float4 e[kWave][kQuadsPerRow];    // d1 on the way in, h (px_grad) on the way out
  float4 ome[kWave][kQuadsPerRow];  // 1 - d1 on the way in, c (py_grad) on the way out
  float4 rin[kRing / 4];            // replay lane's inputs (from the chunk below)
  float4 hout[kRing / 4];           // first row's h, on its way to the chunk above
  unsigned ticket;
};

struct BwdRegs {
  float4 d, s, x;  // p[dest], p[src], px[src]
};

__global__ __launch_bounds__(kFastThreads) void MiBackwardFastKernel(
    const float *__restrict__ px, const float *__restrict__ p,
    const int64_t *__restrict__ boundary, float *__restrict__ ans_grad,
    float *__restrict__ px_grad, float *__restrict__ py_grad, FastHeader *hdr, float *edge, int S,
    int Tn, int modified, int nchunks, int edge_stride, int overwrite_ans_grad) {
  __shared__ BwdLds lds;
  const unsigned total_wgs = gridDim.x;
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

  // Everything the sweep does not assign is zero.  Each workgroup owns 63 ARRAY rows
  // (independent of the box) and clears them a column slice at a time, one slice per pipeline
  // iteration, so the clearing hides behind the sweep.
  const int zr_lo = g.c * kRows, zr_hi = min(zr_lo + kRows, S + 1);
  const int xs0 = box.ok ? box.s0 : 0, xs1 = box.ok ? box.s1 : 0;
  const int xt0 = box.ok ? box.t0 : 0, xt1 = box.ok ? box.t1 + off + 1 : 0;
  const int ys1 = box.ok ? box.s1 + 1 : 0, yt1 = box.ok ? box.t1 : 0;
  auto zero_slice = [&](int c_lo, int c_hi, int first, int stride) {
    const int width = c_hi - c_lo;
    if (width <= 0) return;
    const int total = (zr_hi - zr_lo) * width;
    for (int idx = first; idx < total; idx += stride) {
      const int r = zr_lo + idx / width, t = c_lo + idx % width;
      if (r < S && t < T1 && !(r >= xs0 && r < xs1 && t >= xt0 && t < xt1)) gxb[(size_t)r * T1 + t] = 0.0f;
      if (t < Tn && !(r >= xs0 && r < ys1 && t >= xt0 && t < yt1)) gyb[(size_t)r * Tn + t] = 0.0f;
    }
  };

  g.s0 = box.s0; g.t0 = box.t0; g.ns = box.s1 - box.s0; g.nt = box.t1 - box.t0;
  g.row0 = g.c * kRows;
  if (!box.ok || g.row0 > g.ns) {
    zero_slice(0, T1, threadIdx.x, kFastThreads);  // nothing to sweep: clear the rows and leave
    if (threadIdx.x == 0) FinishWorkgroup(hdr, total_wgs);
    return;
  }
  g.nrows = min(kRows, g.ns - g.row0 + 1);
  g.skew = modified ? 0 : 1;
  const bool has_down = g.row0 + kRows <= g.ns;
  const bool has_up = g.c > 0;
  const int npos = g.nt + 2 + (kRows - 1) * g.skew;  // one virtual column right of the end cell
  g.nblocks = (npos + kW - 1) / kW;
  const int edge_shift = kRows * g.skew;  // position m here <-> position m - edge_shift one chunk down
  float *edge_out = edge + ((size_t)g.b * nchunks + g.c) * edge_stride;      // read by chunk c-1
  float *edge_in = edge + ((size_t)g.b * nchunks + g.c + 1) * edge_stride;   // from chunk c+1
  const int zero_cols = (T1 + g.nblocks - 1) / g.nblocks;  // columns cleared per iteration

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const bool is_chain = wave == 0;
  const int hid = threadIdx.x - kWave;
  const bool has_item = hid >= 0 && hid < kItems;
  const int item = min(max(hid, 0), kItems - 1);
  const int q = item >> 3, m = item & 7;
  const int row_i = g.row0 + q;
  const bool any_cell = g.ns >= 1 && g.nt >= 1;  // is there any cell with both edges?
  const int row_c = min(max(row_i, 1), max(g.ns, 1));  // a row that has a row above it
  const float *pd_row = pb + (size_t)(g.s0 + row_c) * (Tn + 1) + g.t0;
  const float *ps_row = pb + (size_t)(g.s0 + row_c - 1) * (Tn + 1) + g.t0 - 1 + g.skew;
  const float *xs_row = pxb + (size_t)(g.s0 + row_c - 1) * T1 + g.t0 - 1 + g.skew;

  // raw loads for the four destination cells (row q, positions kb*32 + 4m .. +3)
  auto load_block = [&](int kb, BwdRegs &r) {
    if (kb < 0 || !any_cell || !has_item) return;
    const bool interior = kb * kW - (kRows - 1) * g.skew >= 1 && kb * kW + 31 <= g.nt;
    const int jd = kb * kW + 4 * m - q * g.skew;  // destination column of element 0
    if (interior) {
      r.d = LoadQuad(pd_row + jd);
      r.s = LoadQuad(ps_row + jd);
      r.x = LoadQuad(xs_row + jd);
    } else {
      r.d = LoadClamped(pd_row, jd, 1, g.nt);
      r.s = LoadClamped(ps_row, jd, 1, g.nt);
      r.x = LoadClamped(xs_row, jd, 1, g.nt);
    }
  };

  auto coeffs = [&](int j, float pd, float psrc, float xsrc, float *e_out, float *o_out) {
    float ve = 0.0f, vo = 0.0f;
    if (row_i <= g.ns) {
      if (row_i == 0) {
        if (j >= 1 && j <= g.nt) vo = 1.0f;  // first row: everything flows along py
      } else if (j >= 1 && j <= g.nt) {
        float total = pd;
        if (total - total != 0.0f) total = 0.0f;
        const float d1 = __expf((psrc + xsrc) - total);
        if (d1 - d1 == 0.0f) { ve = d1; vo = 1.0f - d1; }
      } else if (j == 0 && !modified) {
        ve = 1.0f;  // first column of a regular lattice: all of it flows up
      }
      // virtual cells right of the end cell hand the seed leftwards unchanged
      if (row_i == g.ns && j > g.nt) { ve = 0.0f; vo = 1.0f; }
    }
    *e_out = ve;
    *o_out = vo;
  };

  auto commit_block = [&](int kb, const BwdRegs &r) {
    if (kb < 0 || !has_item) return;
    const int jd = kb * kW + 4 * m - q * g.skew;
    float4 ve, vo;
    coeffs(jd + 0, r.d.x, r.s.x, r.x.x, &ve.x, &vo.x);
    coeffs(jd + 1, r.d.y, r.s.y, r.x.y, &ve.y, &vo.y);
    coeffs(jd + 2, r.d.z, r.s.z, r.x.z, &ve.z, &vo.z);
    coeffs(jd + 3, r.d.w, r.s.w, r.x.w, &ve.w, &vo.w);
    const int pq = (kb % 3) * kQuadsPerBlock + m;
    lds.e[q][pq] = ve;
    lds.ome[q][pq] = vo;
  };

  auto store_block = [&](int kb) {
    if (kb >= g.nblocks || !has_item || row_i > g.ns) return;
    const int pq = (kb % 3) * kQuadsPerBlock + m;
    const float4 h4 = lds.e[q][pq];
    const float4 c4 = lds.ome[q][pq];
    const float hv[4] = {h4.x, h4.y, h4.z, h4.w}, cv[4] = {c4.x, c4.y, c4.z, c4.w};
    const int jd = kb * kW + 4 * m - q * g.skew;
    const int s = g.s0 + row_i;
    // py_grad[s][t0 + jd - 1 + e]   for destination columns 1..nt
    float *dy = gyb + (size_t)s * Tn + g.t0 + jd - 1;
    if (jd >= 1 && jd + 3 <= g.nt) {
      StoreQuad(dy, c4);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (jd + e >= 1 && jd + e <= g.nt) dy[e] = cv[e];
    }
    // px_grad[s-1][t0 + jd - 1 + skew + e]   for destination columns (1 - skew)..nt
    if (row_i >= 1) {
      float *dx = gxb + (size_t)(s - 1) * T1 + g.t0 + jd - 1 + g.skew;
      const int lo = 1 - g.skew;
      if (jd >= lo && jd + 3 <= g.nt) {
        StoreQuad(dx, h4);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (jd + e >= lo && jd + e <= g.nt) dx[e] = hv[e];
      }
    }
  };

  auto load_rin = [&](int kb) {
    if (hid >= 0 && hid < kW && kb >= 0) {
      const int mpos = kb * kW + hid;
      float v = 0.0f;
      if (has_down) {
        const int idx = mpos - edge_shift;  // position of the same column in the chunk below
        if (idx >= 0) v = TakeEdge(edge_in + idx, hdr, 0.0f);
      }
      reinterpret_cast<float *>(lds.rin)[(kb % 3) * kW + hid] = v;
    }
  };

  // only words the chunk above will take are published (positions it maps inside its range)
  auto publish = [&](int kb) {
    if (has_up && kb < g.nblocks && hid >= kWave && hid < kWave + kW) {
      const int mpos = kb * kW + (hid - kWave);
      if (mpos + edge_shift < g.nblocks * kW)
        PublishEdge(edge_out + mpos, reinterpret_cast<const float *>(lds.hout)[(kb % 3) * kW + (hid - kWave)]);
    }
  };

  // gradient at the (virtual) right end of each row: the seed on the sequence's last row
  float G = 0.0f;
  if (is_chain && g.row0 + lane == g.ns) G = ans_grad[g.b];
  float g_origin = 0.0f;
  auto chain_block = [&](int kb) {
    const int base = (kb % 3) * kQuadsPerBlock;
    float4 ne = lds.e[lane][base + kQuadsPerBlock - 1], no = lds.ome[lane][base + kQuadsPerBlock - 1],
           nr = lds.rin[base + kQuadsPerBlock - 1];
#pragma unroll
    for (int mm = kQuadsPerBlock - 1; mm >= 0; --mm) {
      const float4 e4 = ne, o4 = no, r4 = nr;
      if (mm > 0) {
        ne = lds.e[lane][base + mm - 1];
        no = lds.ome[lane][base + mm - 1];
        nr = lds.rin[base + mm - 1];
      }
      const float es[4] = {e4.x, e4.y, e4.z, e4.w};
      const float os[4] = {o4.x, o4.y, o4.z, o4.w};
      const float rs4[4] = {r4.x, r4.y, r4.z, r4.w};
      float hs[4], cs[4];
#pragma unroll
      for (int e = 3; e >= 0; --e) {
        if (kb == 0 && mm == 0 && e == 0) g_origin = G;
        const float h = es[e] * G;
        const float c = os[e] * G;
        G = WaveShl1(rs4[e], h) + c;  // lane 63 takes the h arriving from the chunk below
        hs[e] = h;
        cs[e] = c;
      }
      const float4 h4 = make_float4(hs[0], hs[1], hs[2], hs[3]);
      lds.e[lane][base + mm] = h4;
      lds.ome[lane][base + mm] = make_float4(cs[0], cs[1], cs[2], cs[3]);
      if (lane == 0) lds.hout[base + mm] = h4;
    }
  };

  const int top = g.nblocks - 1;
  BwdRegs ra, rb;
  if (!is_chain) {
    load_block(top, ra);
    commit_block(top, ra);
    load_rin(top);
    load_block(top - 1, ra);
    load_block(top - 2, rb);
  }
  __syncthreads();

  auto iteration = [&](int kb, BwdRegs &r) {
    if (!is_chain) {
      commit_block(kb - 1, r);
      load_rin(kb - 1);
      load_block(kb - 3, r);
      store_block(kb + 1);
      publish(kb + 1);
      const int it = top - kb;
      zero_slice(it * zero_cols, min((it + 1) * zero_cols, T1), hid, kHelperLanes);
    } else {
      chain_block(kb);
    }
    __syncthreads();
  };
  for (int kb = top; kb >= 0; kb -= 2) {
    iteration(kb, ra);
    if (kb - 1 >= 0) iteration(kb - 1, rb);
  }
  if (!is_chain) {
    store_block(0);
    publish(0);
  }
  if (overwrite_ans_grad && is_chain && g.c == 0 && lane == 0) ans_grad[g.b] = g_origin;
  if (threadIdx.x == 0) FinishWorkgroup(hdr, total_wgs);
}

}  // namespace

size_t MiFastWorkspaceBytes(int B, int S, int Tn) {
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const size_t edge_stride = ((size_t)Tn + 2 + kRows + kW + 3) / 4 * 4 + kW;
  return sizeof(FastHeader) + (size_t)B * (nchunks + 1) * edge_stride * sizeof(float);
}

int MiFastWorkspaceInit(void *workspace, size_t workspace_bytes, hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < sizeof(FastHeader)) return K2AMD_ERR_WORKSPACE;
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  const size_t n_edge = (workspace_bytes - sizeof(FastHeader)) / sizeof(float);
  hipLaunchKernelGGL(FastWsInitKernel, dim3((unsigned)min((size_t)256, (n_edge + 255) / 256 + 1)),
                     dim3(256), 0, stream, hdr, reinterpret_cast<unsigned *>(hdr + 1), n_edge);
  return LaunchStatus();
}

int MiForwardFast(const float *px, const float *py, const int64_t *boundary, float *p, float *ans,
                  int B, int S, int Tn, int modified, void *workspace, size_t workspace_bytes,
                  hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiFastWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const int edge_stride = (int)(((size_t)Tn + 2 + kRows + kW + 3) / 4 * 4 + kW);
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  float *edge = reinterpret_cast<float *>(hdr + 1);
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
  hipLaunchKernelGGL(MiBackwardFastKernel, dim3((unsigned)(B * nchunks)), dim3(kFastThreads), 0, stream,
                     px, p, boundary, ans_grad, px_grad, py_grad, hdr, edge, S, Tn, modified, nchunks,
                     edge_stride, overwrite_ans_grad);
  return LaunchStatus();
}

}  // namespace k2amd
