// Throughput path of the fp32 mutual-information recursion on gfx950.
//
// Decomposition.  A sequence's lattice is cut into CHUNKS of 64 consecutive rows (s).  One
// workgroup owns one chunk; the chunks of a sequence form a pipeline, so one sequence draws its
// HBM bandwidth from several compute units (a single workgroup tops out near 100 GB/s on this
// part; 32 sequences alone could never fill 8 TB/s).
//
// Inside a workgroup (ten wavefronts, each with one job, so that no wavefront that loads ever
// has to wait for a store to be acknowledged):
//   * one CHAIN wavefront carries the recursion, lane = lattice row.  Lane q works on column
//     j = n - q*skew at step n (skew = 1 for the regular lattice, 0 for the modified one), so
//     every cell depends on the previous step only: its own lane's value and the neighbouring
//     lane's, fetched with a DPP wave shift (no LDS, no barrier inside a step).  The lane at the
//     end of the wavefront has no neighbour: the DPP operation leaves its register as it is, and
//     what that register holds is the value arriving from the adjacent chunk (an extra LDS row
//     filled by the edge wavefront).
//   * four LOADER wavefronts issue coalesced, branch-free quad loads of row segments three blocks
//     ahead of use and, two iterations later, place them into an LDS ring PRE-SKEWED (element for
//     lane q, step n at ring position n) so the chain wavefront reads 4 steps per lane with one
//     aligned ds_read_b128.
//   * four STORER wavefronts drain the ring: results leave as contiguous row segments.
//   * one EDGE wavefront takes the words published by the adjacent chunk and publishes this
//     chunk's boundary row.
//   * one barrier per block of 32 steps; it orders LDS traffic only, so global loads and stores
//     stay in flight across it.
//
// Between workgroups: the boundary row of a chunk is published per step into a small edge buffer
// in global memory with device-scope atomic stores; the adjacent chunk polls those words until
// they differ from a sentinel, and writes the sentinel back once it has the value, so the buffer
// is clean again when the kernel ends.  Each word is self-validating, so no fences and no cache
// flushes are needed.  Workgroups take their chunk from a ticket counter, which guarantees that
// the chunk a workgroup waits for has already started; the workgroup that draws a launch's last
// ticket puts the counter back.  The workspace therefore needs ONE initialisation (k2amd_mi_workspace_init) and no
// per-call setup kernel.  Every wait is bounded; a timeout raises the header's error flag, after
// which every later wait returns at once.
//
// Three kernels share the two sweeps (MiForwardChunk, MiBackwardChunk): the forward alone, the
// backward alone, and both in one launch for callers that want the gradients with the scores.
// In that launch, and in the two-call pair that goes with it, the forward hands the backward the
// logarithm of every cell's px-edge derivative in a tensor that takes p's place, so the backward
// reads one value per cell.  The single launch hands its work out as tasks through the same ticket
// counter to persistent workgroups; a task only ever waits for tasks with EARLIER tickets, which
// running workgroups hold, so the launch makes progress with any number of resident workgroups
// (deadlock freedom depends on exactly that: no task may wait for a later ticket).
//
// Arithmetic is the reference's log-domain recursion (k2/python/csrc/torch/
// mutual_information_cpu.cu:89-121, log-add of k2/csrc/utils.h:511-563) with hardware exp2/log2.
// The forward sweeps of the single launch carry p in base-2 logarithms and relative to a FRAME
// (a multiple of 64 that follows the values block by block, see ChainStep2 and Frames): p never
// leaves that launch, and values of a few hundred carry an ulp of 1e-5 where the thousands that
// p itself reaches carry 2.4e-4 and more.
#include <algorithm>
#include <atomic>
#include <cstdlib>

#include <cstddef>

#include "common.h"
#include "mi_generic_impl.h"
#include "mi_internal.h"

namespace k2amd {
namespace {

constexpr int kRows = 64;           // lattice rows per chunk, one per lane of the chain wavefront
constexpr int kW = 32;              // steps per block
constexpr int kRing = 3 * kW;       // ring positions per row
constexpr int kStride = kRing + 4;  // floats per LDS row; +4 spreads lanes over banks
constexpr int kStorerWaves = 4;
constexpr unsigned kSentinel = 0x7fc5a5a5u;  // a quiet-NaN pattern arithmetic never produces
constexpr int kSpinLimit = 1 << 20;
constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;
constexpr int kQuadsPerRow = kStride / 4;
constexpr int kQuadsPerBlock = kW / 4;
// One work item = (row q in 0..63, quad m in 0..7) of a block: four consecutive steps of one
// lattice row; 512 items per block.  The four storer wavefronts take two items per lane (rows q
// and q + 32, same quad); the loader wavefronts (four in either kernel: with more of them the
// compute unit's total instruction issue, which is what the backward's iteration is bound by,
// does not grow) take 512 / lanes items per lane.  A
// wave-wide 16-byte load or store occupies its wavefront for about a hundred cycles once the
// memory pipeline is busy, so the movers' work is spread over all their wavefronts in every
// iteration, and the loaders keep two register sets so that a block's loads stay in flight for
// two iterations.
constexpr int kBlockItems = kRows * kQuadsPerBlock;
template <int kLoaderWavesT>
struct Layout {
  static constexpr int kLoaderWaves = kLoaderWavesT;
  static constexpr int kLoaderLanes = kWave * kLoaderWaves;
  static constexpr int kLoadItems = kBlockItems / kLoaderLanes;        // items per loader lane
  static constexpr int kRowStep = kLoaderLanes / kQuadsPerBlock;       // rows between a lane's items
  static constexpr int kThreads = kWave * (2 + kLoaderWaves + kStorerWaves);
  static_assert(kLoadItems * kLoaderLanes == kBlockItems, "loader lanes must divide the block");
};
typedef Layout<4> FwdLayout;
typedef Layout<4> BwdLayout;
static_assert(kBlockItems == 2 * kWave * kStorerWaves, "two work items per storer lane");

struct FastHeader {
  unsigned ticket;    // next chunk to hand out; put back by the drawer of a launch's last ticket
  unsigned reserved;  // stays 0
  unsigned error;     // set when a bounded wait timed out (sticky until re-initialised)
  unsigned pad[61];
};

__device__ __forceinline__ float NegInfF() { return -__builtin_huge_valf(); }

// Inside the forward chain "minus infinity" is this finite stand-in: differences of two such
// values are finite, so the log-add needs no NaN guard on its critical path.  The loaders and
// storers translate at the LDS boundary in both directions.
constexpr float kLogZero = -1.0e30f;
constexpr float kLogZeroTest = -1.0e29f;  // anything below counts as -inf when p leaves the chain

// One step of the forward chain for every row (lane) of the chunk:
//     x   = P + fy                       the path arriving along py (same row, previous column)
//     inc = P(lane - 1) + fx             the path arriving along px (row above); lane 0 has no
//                                        lane above it: the DPP add leaves its register alone,
//                                        so its `fx` must already be that whole sum
//     P'  = log(exp(inc) + exp(x)) = max + log2(1 + exp2(-|inc - x| log2e)) ln2   on the fast
//           transcendental units.  All values are finite (see kLogZero).  This matches k2's
//           log-add to within one fp32 rounding of the larger operand: where k2 drops the
//           smaller term (difference below log(eps)) the correction computed here is < 1.2e-7.
// The first half is spelled out in assembly: the DPP add needs two wait states after the VALU
// write of P (the add of x and one s_nop provide them; the compiler's hazard recogniser does
// not look inside), and v_max_f32 on known-finite numbers needs no canonicalising pre-pass.
__device__ __forceinline__ float ChainStep(float P, float fx, float fy) {
  float x, mx, d, inc = fx;
  asm volatile(
      "v_add_f32 %[x], %[P], %[fy]\n\t"
      "s_nop 0\n\t"
      "v_add_f32_dpp %[inc], %[P], %[inc] wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32 %[mx], %[inc], %[x]\n\t"
      "v_sub_f32 %[d], %[inc], %[x]"
      : [x] "=&v"(x), [inc] "+&v"(inc), [mx] "=&v"(mx), [d] "=&v"(d)
      : [P] "v"(P), [fy] "v"(fy));
  const float e = __builtin_amdgcn_exp2f(-__builtin_fabsf(d) * kLog2e);
  return __builtin_fmaf(__builtin_amdgcn_logf(1.0f + e), kLn2, mx);
}

// The same step in base-2 logarithms (P, fx, fy all scaled by log2 e): the dependent multiply in
// front of the exponential and the one behind the logarithm are gone,
//     P' = max + log2(1 + exp2(-|inc - x|)).
// Used where p never leaves the launch (the single launch): a p that went through a scaling is
// one rounding away from the reference's, which matters where p itself is handed on, and does
// not where only differences of p (the log-derivatives) and the score are.
__device__ __forceinline__ float ChainStep2(float P, float fx, float fy) {
  float x, mx, d, inc = fx;
  asm volatile(
      "v_add_f32 %[x], %[P], %[fy]\n\t"
      "s_nop 0\n\t"
      "v_add_f32_dpp %[inc], %[P], %[inc] wave_shr:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32 %[mx], %[inc], %[x]\n\t"
      "v_sub_f32 %[d], %[inc], %[x]"
      : [x] "=&v"(x), [inc] "+&v"(inc), [mx] "=&v"(mx), [d] "=&v"(d)
      : [P] "v"(P), [fy] "v"(fy));
  const float e = __builtin_amdgcn_exp2f(-__builtin_fabsf(d));
  return mx + __builtin_amdgcn_logf(1.0f + e);
}

// Frames.  A forward sweep of the single launch keeps, per chunk and per 32-step block, a FRAME: a
// multiple of 64 (so that adding and subtracting frames is exact) that is subtracted from every
// value the chain carries in that block.  ANY sequence of frames gives the same mathematics; a
// frame near the values keeps them small, and with them their rounding errors.  The chain
// wavefront moves its values from one block's frame to the next at the block boundary and picks
// the frame two blocks ahead (so that a barrier lies between the choice and every other
// wavefront's use of it) by extrapolating the largest live value; a chunk's first two blocks take
// the frame of the first words that arrive from the chunk above.  Between chunks every published
// block of edge words comes with its frame (one more self-validating word); on the cut every
// chunk publishes the frame of its last block next to its 64 values.
constexpr int kFrameRing = 8;
constexpr float kFrameUnit = 64.0f;
__device__ __forceinline__ float RoundToFrame(float v) {
  v = fminf(fmaxf(v, -1.0e9f), 1.0e9f);
  return kFrameUnit * __builtin_rintf(v * (1.0f / kFrameUnit));
}

// The gauge.  Adding a constant to every px and another to every py of a sequence changes the score
// by a known amount (every path from the origin to the end cell takes the same number of edges of
// either kind) and the gradients not at all.  The single launch subtracts from px and py (in
// base-2 logarithms) the means of a small sample of each, rounded to sixteenths, before the chain
// sees them: what the chain then carries grows like the logarithm of the number of paths instead
// of like the sum of the log-probabilities along one, and the frames have little left to follow.
// ANY pair of constants gives the same mathematics, but every task of a sequence must use the
// SAME pair: all of them take it from the same sixteen floats of the sequence's first px and py
// row with the same arithmetic (GaugeOf), and the join adds back what the pair took off the score.
struct Gauge {
  float x, y;  // subtracted from px * log2(e), py * log2(e)
};
// The sample: lanes 0..15 of a wavefront hold the first 16 floats of the sequence's first px row,
// lanes 16..31 those of its first py row (lattice coordinates; `valid`: the float exists).  Each
// constant is the mean of the sample's values that lie within kGaugeBand of its largest one (an
// edge that is blocked or all but blocked says nothing about the edges that the paths that matter
// take), in base-2 logarithms, rounded to sixteenths.  Reductions over rows of 16 lanes in a fixed
// order: every wavefront of every task gets the same bits.
constexpr int kGaugeSample = 16;
constexpr float kGaugeBand = 20.0f;
#define K2AMD_ROW_BUTTERFLY_F(v, op)                                                          \
  v = op(v, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0xB1, 0xf, 0xf, true)));  \
  v = op(v, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x4E, 0xf, 0xf, true)));  \
  v = op(v, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x141, 0xf, 0xf, true))); \
  v = op(v, __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), 0x140, 0xf, 0xf, true)))
__device__ __forceinline__ float GaugeMaxF(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ float GaugeAddF(float a, float b) { return a + b; }
__device__ __forceinline__ Gauge GaugeOf(float v, bool valid, int ns) {
  const bool ok = valid && __builtin_fabsf(v) < 1.0e29f;  // (NaN: not ok)
  float top = ok ? v : -3.0e38f;
  K2AMD_ROW_BUTTERFLY_F(top, GaugeMaxF);
  const bool in = ok && v >= top - kGaugeBand;
  float sum = in ? v : 0.0f, cnt = in ? 1.0f : 0.0f;
  K2AMD_ROW_BUTTERFLY_F(sum, GaugeAddF);
  K2AMD_ROW_BUTTERFLY_F(cnt, GaugeAddF);
  const float mean = cnt > 0.0f ? sum / cnt * kLog2e : 0.0f;
  const float r = __builtin_rintf(fminf(fmaxf(mean, -1.0e6f), 1.0e6f) * 16.0f) * (1.0f / 16.0f);
  Gauge g;
  g.x = ns > 0 ? __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(r), 0)) : 0.0f;
  g.y = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(r), kGaugeSample));
  return g;
}
#undef K2AMD_ROW_BUTTERFLY_F

// Everything these kernels reach through a pointer is device memory, and they say so: the tasks
// of the single launch get their pointers from a structure in LDS, where the compiler cannot see
// that, and an access through a pointer of unknown kind is a FLAT one, which also goes through
// the LDS queue and counts against the waits for LDS data (the storers' gradient stores then
// held up their own LDS reads: 6 us of a 56 us launch).
typedef __attribute__((address_space(1))) float GFloat;
typedef __attribute__((address_space(1))) unsigned GWord;
__device__ __forceinline__ GFloat *Global(float *p) { return (GFloat *)p; }
__device__ __forceinline__ const GFloat *Global(const float *p) { return (const GFloat *)p; }
__device__ __forceinline__ GWord *Global(unsigned *p) { return (GWord *)p; }
__device__ __forceinline__ const GWord *Global(const unsigned *p) { return (const GWord *)p; }

typedef float QuadU __attribute__((ext_vector_type(4), aligned(4)));  // four floats at any float
__device__ __forceinline__ void StoreQuad(GFloat *ptr, float4 v) {
  QuadU o;
  o.x = v.x; o.y = v.y; o.z = v.z; o.w = v.w;
  *(__attribute__((address_space(1))) QuadU *)ptr = o;
}
__device__ __forceinline__ void StoreQuad(float *ptr, float4 v) { StoreQuad(Global(ptr), v); }

// Loads go through raw buffer resources (one per tensor): the hardware range-checks every dword
// against the tensor's size and returns 0 beyond it, so no load can leave the tensor whatever
// the boundary tensor holds, and no address clamping code sits in the loaders.
//
// The loaders' loads are issued from inline assembly and waited for with explicit s_waitcnt:
// a block's loads have to stay in flight across two loop iterations, and the compiler's own
// wait-count insertion falls back to "wait for everything" for loads carried around a loop,
// which would stall every iteration for a full memory round trip.  The loader loop issues no
// other vector memory operation, so the counts below are exact.  Two rules keep this sound:
// every register set is drained with WaitLoads<0> before it goes out of scope (a load that
// lands later would overwrite whatever the compiler has put into its registers by then), and
// nothing reads or copies a set between AsyncQuad and the WaitLoads that covers it.
typedef int int4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int4v MakeResource(const float *base, size_t elems) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(base);
  int4v r;
  r.x = __builtin_amdgcn_readfirstlane((int)(a & 0xffffffffull));
  r.y = __builtin_amdgcn_readfirstlane((int)(a >> 32));  // stride 0: a raw buffer
  r.z = __builtin_amdgcn_readfirstlane((int)(elems * sizeof(float)));
  r.w = 0x00020000;
  return r;
}
// starts the load of four consecutive floats from float index max(idx, 0); the result may be
// read only after a WaitLoads that covers it
__device__ __forceinline__ float4v AsyncQuad(int4v rs, int idx) {
  float4v v;
  const int off = max(idx, 0) * 4;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(v) : "v"(off), "s"(rs) : "memory");
  return v;
}
__device__ __forceinline__ float4 AsFloat4(float4v v) { return make_float4(v.x, v.y, v.z, v.w); }

// The same load, and a 16-byte store, at device coherence (sc1): they are performed where every
// compute unit of the device sees them, past the L2 of the issuing unit's XCD, as the
// device-scope atomic accesses of the edge words are.  The single launch moves the
// log-derivatives between workgroups this way: a forward sweep's stores are read, later in the
// same launch, by whichever compute unit sweeps that chunk back, and handing them over with a
// device-scope release / acquire pair instead would write back and invalidate a whole L2 at
// every hand-over (measured: 7 us each, and every other workgroup of the XCD slowed down).
__device__ __forceinline__ float4v AsyncQuadCoherent(int4v rs, int idx) {
  float4v v;
  const int off = max(idx, 0) * 4;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen sc1" : "=v"(v) : "v"(off), "s"(rs) : "memory");
  return v;
}
__device__ __forceinline__ void StoreQuadCoherent(float *ptr, float4 v) {
  float4v w;
  w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w;
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(ptr), "v"(w) : "memory");
}
__device__ __forceinline__ void StoreCoherent(float *ptr, float v) {
  __hip_atomic_store(Global(ptr), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A quad whose first float would lie in front of the tensor (idx < 0: only possible for the
// tensor's very first row) is loaded from index 0 instead; this moves the floats back to the
// positions they were asked for.  The floats in front of the tensor belong to columns outside
// the box and are masked by the caller.
__device__ __forceinline__ float4 ShiftQuad(float4 v, int idx) {
  const int sh = idx < 0 ? -idx : 0;
  float4 r;
  r.x = v.x;
  r.y = sh == 0 ? v.y : v.x;
  r.z = sh == 0 ? v.z : (sh == 1 ? v.y : v.x);
  r.w = sh == 0 ? v.w : (sh == 1 ? v.z : (sh == 2 ? v.y : v.x));
  return r;
}

// Workgroup barrier that orders LDS traffic only.  Everything the wavefronts of a workgroup hand
// to each other goes through LDS, so global loads (the loaders' prefetch) and global stores (the
// storers' output) stay in flight across it; a full __syncthreads() would drain them
// (s_waitcnt vmcnt(0)) every iteration and serialise the pipeline on HBM latency.
__device__ __forceinline__ void LdsBarrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct ChunkGeom {
  int b, c;
  int s0, t0, ns, nt;  // box origin and extent
  int row0;            // local row (s - s0) of the chunk's first lattice row
  int skew;
  int nblocks;
};

// The part of a sequence's lattice that one sweep covers.  The single launch splits every lattice
// at a "cut" diagonal (cells with s + t = const on a regular lattice, a column on a modified
// one) into two halves that are swept at the same time: the first half in the lattice's own
// coordinates from the origin up to the cut, the second half MIRRORED, i.e. from the end cell
// back to the cut in coordinates s' = ns - s, t' = nt - t, in which the recursion for
//     beta[s][t] = log_add(px[s][t] + beta[s+1][t-o], py[s][t] + beta[s][t+1])
// is the forward recursion again, on px and py read backwards along both axes.  A sweep over a
// half works in ITS coordinates throughout; only the addresses of what it loads and stores know
// about the mirror.  dmax = last diagonal of the half (own coordinates).  The two-kernel pair
// sweeps whole lattices: kBidir = false compiles all of this away.
struct Half {
  int mirror;  // 0: own coordinates = the lattice's; 1: reversed along both axes
  int dmax;    // cells with row * skew + column <= dmax belong to the half
#ifdef K2AMD_MI_TRACE
  unsigned long long *trace;
#endif
};
#ifdef K2AMD_MI_TRACE
#define K2AMD_TRACE_MARK(half, i) do { if ((half).trace != nullptr && threadIdx.x == 0) (half).trace[i] = wall_clock64(); } while (0)
#define K2AMD_TRACE_MARK_IF(half, i, cond) do { if ((half).trace != nullptr && (cond)) (half).trace[i] = wall_clock64(); } while (0)
#else
#define K2AMD_TRACE_MARK(half, i) do { } while (0)
#define K2AMD_TRACE_MARK_IF(half, i, cond) do { } while (0)
#endif

// The single launch keeps the log-derivatives of every half-sweep in a slab of its own, laid out
// the way they are produced and consumed: per (sequence, half, chunk) a run of 32-position blocks,
// each 64 rows x 32 positions of the half's own coordinates.  A wavefront's 16-byte accesses then
// cover 1 KB of consecutive bytes and every 128-byte line is written whole, by one instruction
// (rows of a [S + 1][T + 2] array would put 128-byte runs 4 KB apart, straddling two lines each,
// which device-coherent stores send to memory as the partial lines they are).
// Blocks a chunk of a half can have: its positions end one past the cut diagonal, and the cut
// lies half way along the lattice's longest path.
// Floats per (sequence, chunk + 1) row of the edge buffer: the edge words of every step a chunk can
// have, then one frame word per block (single launch).
__host__ __device__ inline int EdgeWords(int Tn) { return (int)(((size_t)Tn + 2 + kRows + kW + 3) / 4 * 4 + kW); }
__host__ __device__ inline int EdgeStride(int Tn) { return EdgeWords(Tn) + (EdgeWords(Tn) / kW + 4 + 3) / 4 * 4; }

constexpr int kSlabBlockFloats = kRows * kW;
__host__ __device__ inline int SlabBlocks(int S, int Tn, int modified) {
  const int diagonals = Tn + (modified ? 0 : S);
  return (diagonals - diagonals / 2 + 2 + kW - 1) / kW;
}
__host__ __device__ inline size_t SlabFloatsPerSequence(int S, int Tn, int modified) {
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  return 2 * (size_t)nchunks * SlabBlocks(S, Tn, modified) * kSlabBlockFloats;
}

__device__ __forceinline__ float4 Rev4(float4 v) { return make_float4(v.w, v.z, v.y, v.x); }

enum Role { kChain = 0, kEdge = 1, kLoader = 2, kStorer = 3 };

// wave:   0      1     2 ..           .. last
// role:   chain  edge  loaders        storers (kStorerWaves)
template <typename L>
__device__ __forceinline__ int RoleOf(int wave) {
  return wave == 0 ? kChain : (wave == 1 ? kEdge : (wave < 2 + L::kLoaderWaves ? kLoader : kStorer));
}
// lane id of a loader (or storer) lane among the lanes of its kind
template <typename L>
__device__ __forceinline__ int MoverLane(int wave, int lane) {
  const int first = wave < 2 + L::kLoaderWaves ? 2 : 2 + L::kLoaderWaves;
  return (wave - first) * kWave + lane;
}

__global__ void FastWsInitKernel(FastHeader *hdr, unsigned *edge, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i == 0) {
    hdr->ticket = 0;
    hdr->reserved = 0;
    hdr->error = 0;
  }
  for (size_t k = i; k < n; k += (size_t)gridDim.x * blockDim.x) edge[k] = kSentinel;
}

// Waits for one published word, takes it and leaves the sentinel behind.  One poll in flight at
// a time: several polls of the same word a quarter of a trip apart (so that it is looked at more
// often than once per trip) made every hand-over slower, not faster (a launch of 56 us took 70).
__device__ __forceinline__ float TakeEdge(float *addr, FastHeader *hdr, float on_timeout) {
  unsigned *word = reinterpret_cast<unsigned *>(addr);
  int spins = 0;
  for (;;) {
    const unsigned v = __hip_atomic_load(Global(word), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (v != kSentinel) {
      __hip_atomic_store(Global(word), kSentinel, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return __uint_as_float(v);
    }
    ++spins;
    if ((spins & 255) == 0 &&
        __hip_atomic_load(Global(&hdr->error), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)
      return on_timeout;
    if (spins > kSpinLimit) {
      __hip_atomic_store(Global(&hdr->error), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return on_timeout;
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

// True once a wait of this or an earlier launch on the workspace has timed out.  Results are then
// invalid, and the kernels say so where a caller looks first: ans (and the ans_grad they hand
// back) become NaN, in that launch where the store comes after the timeout and in every later
// launch until the workspace is initialised again.
__device__ __forceinline__ bool GaveUp(FastHeader *hdr) {
  return __hip_atomic_load(Global(&hdr->error), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
}

// Called by the thread that drew ticket `ticket` of the `total` that a launch draws in all: the
// one that drew the last of them puts the counter back for the next launch (nobody draws after
// it; no counter of finished workgroups, whose answer every workgroup would have to wait for
// before it ends).
__device__ __forceinline__ void PutTicketsBack(FastHeader *hdr, unsigned ticket, unsigned total) {
  if (ticket + 1 == total)
    __hip_atomic_store(Global(&hdr->ticket), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void PublishEdge(float *addr, float v) {
  unsigned u = __float_as_uint(v);
  if (u == kSentinel) u = 0x7fc00000u;
  __hip_atomic_store(Global(reinterpret_cast<unsigned *>(addr)), u, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// Values on the cut diagonal go through device-coherent stores and loads like the edge words (the
// readers are other workgroups, on any compute unit) and validate themselves the same way; they
// have several readers, so a reader leaves them as they are (the last one to finish puts the
// sentinels back, see MiBidirKernel).
__device__ __forceinline__ void PublishCut(float *addr, float v) { PublishEdge(addr, v); }


// ---- the cut of the single launch (see MiBidirKernel) ----
constexpr int kCutRows = 2056;  // lattice rows (S + 2 at most) the single launch serves
constexpr int kCutWordsPerSeqHeader = 16;
constexpr int kCutChunks = (kCutRows + kRows - 1) / kRows;  // chunks a half can have

struct CutShared {
  // alpha / beta of the sequence's cut cells by lattice row, then exp(alpha + beta - best); also
  // the two rotating rows of the exact recursion
  float a[kCutRows];
  float b[kCutRows];
  // the frames of the chunks' values on the cut (see Frames), by chunk of each half
  float fa[kCutChunks], fb[kCutChunks];
  float total;   // the sequence's score, from the join of this task
  float scale;   // the gradient of the sequence's score
  int split_ok;  // the score is finite: the halves sweep back from the cut
  int departed_set;   // the task has already said that it is through with the cut words,
  unsigned departed;  // and this is what the counter held before
  int last;
  unsigned ticket;
};

// Per sequence, in the workspace: depart (readers of the cut finished), the gradient of the
// sequence's score, stored (forward sweeps whose log-derivatives have all reached memory), then
// alpha by own row of the first half and beta by own row of the second (base-2 logarithms, each
// chunk's 64 relative to the chunk's frame), then those frames by chunk.  Counters count up from
// the sentinel, which is what the workspace is initialised to.
struct CutWords {
  unsigned *depart, *stored;
  float *scale, *alpha, *beta, *frame_alpha, *frame_beta;
  float *gauge;  // two words: what the sweeps subtracted from px and py (see Gauge)
  int words;
};
__host__ __device__ inline int CutFrameWords(int nchunks) { return (nchunks + 3) / 4 * 4; }
__host__ __device__ inline int CutWordsPerSequence(int nchunks) {
  return kCutWordsPerSeqHeader + 2 * nchunks * kRows + 2 * CutFrameWords(nchunks);
}
__device__ __forceinline__ CutWords CutOf(float *cut, int b, int nchunks) {
  CutWords w;
  w.words = CutWordsPerSequence(nchunks);
  float *base = cut + (size_t)b * w.words;
  w.depart = reinterpret_cast<unsigned *>(base) + 1;
  w.scale = base + 2;
  w.stored = reinterpret_cast<unsigned *>(base) + 3;
  w.gauge = base + 4;
  w.alpha = base + kCutWordsPerSeqHeader;
  w.beta = w.alpha + nchunks * kRows;
  w.frame_alpha = w.beta + nchunks * kRows;
  w.frame_beta = w.frame_alpha + CutFrameWords(nchunks);
  return w;
}

// One thread waits until a counter has reached a value (bounded, like TakeEdge).
__device__ __forceinline__ void WaitCount(unsigned *word, unsigned want, FastHeader *hdr) {
  int spins = 0;
  for (;;) {
    if (__hip_atomic_load(Global(word), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == want) return;
    ++spins;
    if ((spins & 255) == 0 &&
        __hip_atomic_load(Global(&hdr->error), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)
      return;
    if (spins > kSpinLimit) {
      __hip_atomic_store(Global(&hdr->error), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    __builtin_amdgcn_s_sleep(2);
  }
}

// Reductions over a wavefront through the data-parallel lane permutations (a few cycles per step;
// the LDS crossbar that __shfl goes through costs a hundred).  Four steps leave the result of
// each row of 16 lanes in all of its lanes, the four rows are combined in a fixed order: every
// lane gets the same bits.
template <int kCtrl>
__device__ __forceinline__ float DppF(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), kCtrl, 0xf, 0xf, true));
}
template <int kCtrl>
__device__ __forceinline__ int DppI(int v) {
  return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xf, 0xf, true);
}
// quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror
#define K2AMD_ROW_BUTTERFLY(v, Dpp, op)  \
  v = op(v, Dpp<0xB1>(v));               \
  v = op(v, Dpp<0x4E>(v));               \
  v = op(v, Dpp<0x141>(v));              \
  v = op(v, Dpp<0x140>(v))
__device__ __forceinline__ float LaneF(float v, int lane) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}
__device__ __forceinline__ float AddF(float a, float b) { return a + b; }
__device__ __forceinline__ int MinI(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ float WaveMaxF(float v) {
  K2AMD_ROW_BUTTERFLY(v, DppF, fmaxf);
  return fmaxf(fmaxf(LaneF(v, 0), LaneF(v, 16)), fmaxf(LaneF(v, 32), LaneF(v, 48)));
}
__device__ __forceinline__ float WaveSumF(float v) {
  K2AMD_ROW_BUTTERFLY(v, DppF, AddF);
  return (LaneF(v, 0) + LaneF(v, 16)) + (LaneF(v, 32) + LaneF(v, 48));
}
__device__ __forceinline__ int WaveMinI(int v) {
  K2AMD_ROW_BUTTERFLY(v, DppI, MinI);
  return MinI(MinI(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
              MinI(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}
#undef K2AMD_ROW_BUTTERFLY

// What a backward task needs for the join on its sequence's cut.
struct BidirJoin {
  CutShared *sh;
  CutWords cw;
  float *ans;  // where the sequence's score goes (the task of chunk 0 of the first half), or null
};

// The join on the cut of a sequence with ns + 1 rows, by ONE wavefront (the others of the
// workgroup are fetching the sweep's first blocks meanwhile): waits for the sequence's alpha and
// beta, returns the score (to every lane; -inf when no path reaches the end cell) and, to lane q,
// the gradient seed of own row row0 + q of a half (lattice row = own row, or ns - own row when
// mirrored).  Every task of a sequence adds the same numbers in the same order, so all of them
// get the same bits.
// alpha and beta are of the size of the score (thousands, where one ulp is 2.4e-4) while their
// sum only matters relative to the largest one: both are taken relative to the best cell's
// values BEFORE they are added, which keeps the shares exact to a few ulps of themselves.
// (Inlined: as a function of its own it would take the words' addresses and hand back its results
// through scratch memory, a trip there for each.)
__device__ __forceinline__ float WaveCutJoin(CutShared &sh, const CutWords cw, int ns, int py_edges, int row0,
                                             int mirror, FastHeader *hdr, float *seed_out,
                                             float *scale_out) {
  const int lane = threadIdx.x & (kWave - 1);
  // Every pass asks for all of the sequence's words before it looks at any (one trip to memory
  // per pass, whatever the number of rows), until none of them is the sentinel.
  constexpr int kBatch = 4;
  const unsigned *wa = reinterpret_cast<const unsigned *>(cw.alpha);
  const unsigned *wb = reinterpret_cast<const unsigned *>(cw.beta);
  const unsigned *wfa = reinterpret_cast<const unsigned *>(cw.frame_alpha);
  const unsigned *wfb = reinterpret_cast<const unsigned *>(cw.frame_beta);
  const int nchunks = ns / kRows + 1;  // chunks that hold rows of this sequence
  float scale = 0.0f, gauge_x = 0.0f, gauge_y = 0.0f;
  for (int spins = 0;; ++spins) {
    const unsigned us = __hip_atomic_load(Global(reinterpret_cast<const unsigned *>(cw.scale)), __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
    const unsigned ugx = __hip_atomic_load(Global(reinterpret_cast<const unsigned *>(cw.gauge)), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
    const unsigned ugy = __hip_atomic_load(Global(reinterpret_cast<const unsigned *>(cw.gauge) + 1), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
    const int fc = min(lane, nchunks - 1);
    const unsigned ufa = __hip_atomic_load(Global(wfa + fc), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned ufb = __hip_atomic_load(Global(wfb + fc), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool missing = false;
    for (int s0 = lane; s0 <= ns; s0 += kWave * kBatch) {
      unsigned ua[kBatch], ub[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int s = min(s0 + i * kWave, ns);
        ua[i] = __hip_atomic_load(Global(wa + s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ub[i] = __hip_atomic_load(Global(wb + (ns - s)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int s = s0 + i * kWave;
        if (s <= ns) {
          missing |= ua[i] == kSentinel || ub[i] == kSentinel;
          sh.a[s] = __uint_as_float(ua[i]);
          sh.b[s] = __uint_as_float(ub[i]);
        }
      }
    }
    static_assert(kCutChunks <= kWave, "one lane per chunk's frame");
    if (lane < nchunks) {
      missing |= ufa == kSentinel || ufb == kSentinel;
      sh.fa[lane] = __uint_as_float(ufa);
      sh.fb[lane] = __uint_as_float(ufb);
    }
    missing |= us == kSentinel || ugx == kSentinel || ugy == kSentinel;
    scale = __uint_as_float(us);
    gauge_x = __uint_as_float(ugx);
    gauge_y = __uint_as_float(ugy);
    if (!__any(missing)) break;
    // bounded like every wait: what is missing stays a NaN, the score comes out as not finite
    // and the error flag turns the results into NaN
    if ((spins & 255) == 255 &&
        __hip_atomic_load(Global(&hdr->error), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)
      break;
    if (spins > kSpinLimit) {
      __hip_atomic_store(Global(&hdr->error), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  // Lattice row s is own row s of the first half (chunk s / 64) and own row ns - s of the second.
  float best = -3.0e38f;
  int best_s = 0x7fffffff;
  for (int s = lane; s <= ns; s += kWave) {
    const float u = (sh.a[s] + sh.b[s]) + (sh.fa[s / kRows] + sh.fb[(ns - s) / kRows]);
    if (u > best) { best = u; best_s = s; }
  }
  // the largest sum (to the rounding of the frames' sum: any cell near the best one serves as the
  // reference), the smallest row among equals
  const float wave_best = WaveMaxF(best);
  best_s = WaveMinI(best == wave_best ? best_s : 0x7fffffff);
  const int at = best_s <= ns ? best_s : 0;  // (no candidate at all: every sum was NaN)
  // One wavefront's LDS accesses are served in the order it issues them: the fences only keep
  // the compiler from moving them.
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  const float a_ref = sh.a[at], b_ref = sh.b[at];
  const float fa_ref = sh.fa[at / kRows], fb_ref = sh.fb[(ns - at) / kRows];
  const bool reachable = a_ref + b_ref > kLogZeroTest;
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  float sum = 0.0f;
  for (int s = lane; s <= ns; s += kWave) {
    // differences of values of like size first, the (exact) differences of the frames added to them
    const float da = (sh.a[s] - a_ref) + (sh.fa[s / kRows] - fa_ref);
    const float db = (sh.b[s] - b_ref) + (sh.fb[(ns - s) / kRows] - fb_ref);
    const float w = reachable ? __builtin_amdgcn_exp2f(da + db) : 0.0f;
    sh.a[s] = w;
    sum += w;
  }
  sum = WaveSumF(sum);  // >= 1 when reachable
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  const int own = row0 + lane;
  const int s_own = min(max(mirror ? ns - own : own, 0), ns);
  const float share = sh.a[s_own];
  *seed_out = reachable && own <= ns ? share / sum * scale : 0.0f;
  *scale_out = scale;
  // The score in natural logarithms: the best cell's values and the sum (small), the two frames
  // (thousands, exact) and what the gauge took off every path (ns px edges, py_edges py edges),
  // added in double so that the one rounding that matters is the last.
  const double log2_score = ((double)a_ref + (double)b_ref) + (double)__builtin_amdgcn_logf(sum) +
                            ((double)fa_ref + (double)fb_ref) + (double)ns * (double)gauge_x +
                            (double)py_edges * (double)gauge_y;
  return reachable ? (float)(log2_score * 0.69314718055994530942) : NegInfF();
}

// ------------------------------------------------------------------------------ forward
//
// Lane q of the chain wavefront owns lattice row row0 + q and is at column j = n - q*skew at step
// n.  Ring position n of a lane's LDS row holds what the step into column j needs:
//     fx[q][n] = px[row-1][jp + skew]   (the px edge arriving from the row above)
//     fy[q][n] = py[row][jp]            (the py edge arriving from the left),  jp = j - 1
// and receives p[row][j] in place of fy once the step is done.  Lane 0's "row above" is the
// last row of the chunk above: the edge wavefront adds that row's p and px and stores the sum
// in row 64 of fx.
struct FwdLds {
  float4 fx[kWave + 1][kQuadsPerRow];  // row 64: see below
  float4 fy[kWave][kQuadsPerRow];
  // p of each row at the last position of the three most recent blocks (written by the storers,
  // only when the launch keeps the px-edge log-derivatives)
  float last[3][kWave];
  // px of the row above the chunk (the last row of the chunk above), block by block: written by
  // the loaders one block ahead of the rest, read by the edge wavefront
  float px_above[4][kW];
  // the chunk's frame of each recent block (single launch, see Frames), and what it lies above
  // the block before's; slot kb % kFrameRing
  float frame[kFrameRing], shift[kFrameRing];
  unsigned ticket;
};

struct FwdRegs {
  float4v x[FwdLayout::kLoadItems], y[FwdLayout::kLoadItems];
  float4v above;  // a quad of the row above the chunk, for the block AFTER the set's block
};
// waits until at most kYounger of this wavefront's loads are outstanding and ties the registers
// to the wait, so that no read of them moves in front of it
template <int kYounger>
__device__ __forceinline__ void WaitLoads(FwdRegs &r) {
  static_assert(FwdLayout::kLoadItems == 2, "operand list below");
  asm volatile("s_waitcnt vmcnt(%5)"
               : "+v"(r.x[0]), "+v"(r.y[0]), "+v"(r.x[1]), "+v"(r.y[1]), "+v"(r.above)
               : "n"(kYounger));
}
constexpr int kFwdLoadsPerBlock = 2 * FwdLayout::kLoadItems + 1;

// kKeep: also write log_deriv[b][s][t] = (p[s-1][t+o] + px[s-1][t+o]) - p[s][t], the logarithm of
// the px edge's share of cell (s, t) exactly as the backward sweep forms it
// (k2/python/csrc/torch/mutual_information_cpu.cu:195-211), laid out like p.  The chain step has
// both terms in registers; the storers rebuild them from the ring, so the backward kernel reads
// one tensor instead of p twice and px once.  Cells of a sequence's first row and first column
// hold values the backward never uses.  kWriteP = false (only with kKeep): p itself is not stored,
// for callers that want nothing but ans and the gradients.
// The whole workgroup sweeps chunk `chunk` (64 lattice rows) of sequence `seq`.
// kBidir: the sweep covers the half `half` of the lattice (see Half) and ends on its cut
// diagonal; what the chain holds there (p of the half's last cell of every row) goes to
// cut_out[0..63] (the chunk's 64 own rows; the finite stand-in for -inf where a row has no cell
// on the cut; nothing for rows of a chunk that lies past the sequence's last row altogether), ans
// is not written, and log_deriv is the launch's slab of blocks (SlabBlocks).
template <bool kKeep, bool kWriteP, bool kBidir>
__device__ __forceinline__ void MiForwardChunk(
    FwdLds &lds, const float *__restrict__ px, const float *__restrict__ py, const Box &box,
    float *__restrict__ p, float *__restrict__ ans,
    float *__restrict__ log_deriv, FastHeader *hdr, float *edge, int B, int S, int Tn,
    int modified, int nchunks, int edge_stride, int seq, int chunk, Half half, float *cut_out,
    float *cut_frame_out, float *gauge_out) {
  static_assert(!kBidir || (kKeep && !kWriteP), "the halves keep the log-derivatives only");
  ChunkGeom g;
  g.b = seq;
  g.c = chunk;
  g.s0 = box.s0; g.t0 = box.t0; g.ns = box.s1 - box.s0; g.nt = box.t1 - box.t0;
  g.row0 = g.c * kRows;
  if (!box.ok || g.row0 > g.ns) {
    if (!kBidir && !box.ok && g.c == 0 && threadIdx.x == 0) ans[g.b] = __builtin_nanf("");
    return;
  }
  g.skew = modified ? 0 : 1;
  const int mirror = kBidir ? half.mirror : 0;
  const int nsteps_full = g.nt + 1 + (kRows - 1) * g.skew;  // last needed step index + 1
  // steps (and 32-step blocks) that the chunk at local row r0 runs: up to the cut diagonal
  auto steps_of = [&](int r0) { return kBidir ? min(nsteps_full, half.dmax - r0 * g.skew + 1) : nsteps_full; };
  auto blocks_of = [&](int r0) { return max(steps_of(r0) + kW - 1, 0) / kW; };
  const int nsteps = steps_of(g.row0);
  const int n_last = nsteps - 1;  // the chunk's step on the cut diagonal (kBidir)
  g.nblocks = blocks_of(g.row0);
  if (kBidir && g.nblocks == 0) {  // no cell of these rows lies in the half
    if (threadIdx.x < kRows) PublishCut(cut_out + threadIdx.x, kLogZero);
    if (threadIdx.x == 0) PublishCut(cut_frame_out, 0.0f);
    return;
  }
  const bool has_down = g.row0 + kRows <= g.ns && blocks_of(g.row0 + kRows) > 0;
  const int nblocks_down = has_down ? blocks_of(g.row0 + kRows) : 0;
  const int nblocks_up = g.c > 0 ? blocks_of(g.row0 - kRows) : 0;
  const int edge_shift = kRows * g.skew - 1;  // step n here <-> step n + edge_shift one chunk up

  const int T1 = modified ? Tn : Tn + 1;
  const int LS = Tn + 1;  // floats per row of log_deriv (the two-kernel pair's tensor)
  const GFloat *pxb = Global(px) + (size_t)g.b * S * T1;
  GFloat *pb = kWriteP ? Global(p) + (size_t)g.b * (S + 1) * (Tn + 1) : nullptr;
  // (kBidir: the run of blocks of this chunk of this half in the launch's slab)
  float *ldb = !kKeep ? nullptr
               : kBidir ? log_deriv + (size_t)g.b * SlabFloatsPerSequence(S, Tn, modified) +
                              (size_t)(mirror * nchunks + g.c) * SlabBlocks(S, Tn, modified) * kSlabBlockFloats
                        : log_deriv + (size_t)g.b * (S + 1) * LS;
  float *edge_out = edge + ((size_t)g.b * nchunks + g.c + 1) * edge_stride;  // read by chunk c+1
  float *edge_in = edge + ((size_t)g.b * nchunks + g.c) * edge_stride;
  // (single launch) the frames of the published blocks: one word per block behind a row's edge words
  float *frame_out = edge_out + EdgeWords(Tn), *frame_in = edge_in + EdgeWords(Tn);
  // The blocks of the chunk above whose words this chunk takes (it takes their frames with them),
  // and the same for the chunk below and this chunk's blocks: both sides work it out alike.
  auto frames_lo = [&]() { return max(edge_shift, 0) / kW; };
  auto frames_hi = [&](int blocks_above, int blocks_below) {
    return (min(blocks_above * kW - 1, blocks_below * kW - 1 + edge_shift)) / kW;
  };
  // natural logarithms in the two-launch kernels, base-2 ones less the gauge in the single launch
  const float in_scale = kBidir ? kLog2e : 1.0f;
  // what block kb's frame lies above block kb-1's (a multiple of 64; kb >= 1)
  auto frame_step = [&](int kb) { return lds.shift[kb & (kFrameRing - 1)]; };

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  Gauge gauge{0.0f, 0.0f};  // (set in the prologue by the wavefronts that scale inputs)
  // where the gauge's sample lies: the first floats of the box's first px and py row
  const int gauge_idx_x = (g.b * S + g.s0) * T1 + g.t0, gauge_idx_y = (g.b * (S + 1) + g.s0) * Tn + g.t0;
  // lanes 0..15: px, 16..31: py (the row's valid columns; px has no row at all where ns = 0)
  const bool gauge_valid = lane < 2 * kGaugeSample &&
                           ((lane & kGaugeSample) ? (lane & (kGaugeSample - 1)) < g.nt
                                                  : g.ns > 0 && (lane & (kGaugeSample - 1)) < g.nt + 1 - modified);
  typedef FwdLayout L;
  constexpr int kLoadItems = L::kLoadItems, kRowStep = L::kRowStep;
  const int role = RoleOf<L>(wave);
  const int mid = MoverLane<L>(wave, lane);  // lane id among the loader (or storer) lanes
  const int mq = mid >> 3, mm = mid & 7;     // storers: rows mq and mq + 32, quad mm
  const int lq = mq;                         // loaders: rows lq + kRowStep*it, quad mm

  const int hi_x = g.nt - modified, hi_y = g.nt - 1;  // last valid px / py column

  // ---- loaders ---------------------------------------------------------------------------
  const int4v rsx = MakeResource(px, (size_t)B * S * T1);
  const int4v rsy = MakeResource(py, (size_t)B * (S + 1) * Tn);
  int idx_x[kLoadItems], idx_y[kLoadItems];  // float index of local column 0 of the item's row
  bool rowx_ok[kLoadItems], rowy_ok[kLoadItems];
#pragma unroll
  for (int it = 0; it < kLoadItems; ++it) {
    const int row_i = g.row0 + lq + kRowStep * it;
    rowx_ok[it] = row_i >= 1 && row_i <= g.ns;
    rowy_ok[it] = row_i <= g.ns;
    const int rx = min(max(row_i, 1), max(g.ns, 1)) - 1;  // a px row inside the box if any
    const int ry = min(row_i, g.ns);
    // mirrored: own row r of px is the lattice's row ns-1-r, own column c its column hi_x-c (py:
    // row ns-r, column nt-1-c), so own column c lies at index idx - c
    idx_x[it] = mirror ? (g.b * S + g.s0 + max(g.ns - 1 - rx, 0)) * T1 + g.t0 + hi_x
                       : (g.b * S + g.s0 + rx) * T1 + g.t0;
    idx_y[it] = mirror ? (g.b * (S + 1) + g.s0 + g.ns - ry) * Tn + g.t0 + hi_y
                       : (g.b * (S + 1) + g.s0 + ry) * Tn + g.t0;
  }
  // float index of local column 0 of the row above the chunk (any px row where there is none)
  const int row_above = max(g.row0 - 1, 0);
  const int idx_above = mirror ? (g.b * S + g.s0 + max(g.ns - 1 - row_above, 0)) * T1 + g.t0 + hi_x
                               : (g.b * S + g.s0 + row_above) * T1 + g.t0;
  // index of the quad that holds own columns c .. c+3 of a row whose column 0 is at idx (mirrored:
  // the quad comes back in descending column order, see Unmirror)
  auto quad_at = [&](int idx, int c) { return mirror ? idx - c - 3 : idx + c; };
  // every quad of every row of block kb inside the valid columns?  (uniform over the workgroup)
  auto interior = [&](int kb) {
    return kb * kW - 1 - (kRows - 1) * g.skew >= 0 && kb * kW + 30 <= g.nt - 1;
  };
  // One code path for every block: quads that reach outside the valid columns pick up
  // neighbouring floats (or zeros past the tensor's end) that the commit masks.
  // Always issues kFwdLoadsPerBlock loads, so that the counts given to WaitLoads hold in every
  // iteration; for blocks past the last one it reads the last block again (cache hits).
  auto load_block = [&](int kb, FwdRegs &r) {
    kb = min(kb, g.nblocks - 1);
#pragma unroll
    for (int it = 0; it < kLoadItems; ++it) {
      const int jp = kb * kW + 4 * mm - 1 - (lq + kRowStep * it) * g.skew;  // column left of element 0
      r.x[it] = AsyncQuad(rsx, quad_at(idx_x[it], jp + g.skew));
      r.y[it] = AsyncQuad(rsy, quad_at(idx_y[it], jp));
    }
    // every lane asks (the count of loads in flight is the same for all wavefronts); the eight
    // lanes of loader row 0 keep what arrives
    r.above = AsyncQuad(rsx, quad_at(idx_above, (kb + 1) * kW + 4 * mm - 1 + g.skew));
  };
  // a loaded quad in ascending order of own columns (`at` = the index it was loaded from)
  auto unmirror = [&](float4 v, int at, bool rim) {
    // (a quad can start in front of the tensor for the first sequences: always for the first
    // row of sequence 0, and for later ones where a sequence is shorter than a quad)
    if (rim) v = ShiftQuad(v, at);
    return mirror ? Rev4(v) : v;
  };
  // `inner` is uniform over the workgroup: the masking code for blocks on the rim of the box is
  // a real branch (the empty asm statement keeps the compiler from flattening it into selects
  // that every block would pay for).
  auto commit_block = [&](int kb, FwdRegs &r) {  // registers -> LDS ring
    if (kb >= g.nblocks) return;
    const bool inner = interior(kb);
#pragma unroll
    for (int it = 0; it < kLoadItems; ++it) {
      const int q = lq + kRowStep * it;
      float4 qx = AsFloat4(r.x[it]), qy = AsFloat4(r.y[it]);
      float vx[4], vy[4];
      if (inner) {
        if (kBidir) {
          qx = unmirror(qx, 0, false);
          qy = unmirror(qy, 0, false);
        }
        const float in_x[4] = {qx.x, qx.y, qx.z, qx.w}, in_y[4] = {qy.x, qy.y, qy.z, qy.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vx[e] = rowx_ok[it] ? fmaxf(__builtin_fmaf(in_x[e], in_scale, -gauge.x), kLogZero) : kLogZero;
          vy[e] = rowy_ok[it] ? fmaxf(__builtin_fmaf(in_y[e], in_scale, -gauge.y), kLogZero) : kLogZero;
        }
      } else {
        asm volatile("");
        const int jp = kb * kW + 4 * mm - 1 - q * g.skew;
        const int jx = jp + g.skew;
        qx = unmirror(qx, quad_at(idx_x[it], jx), true);
        qy = unmirror(qy, quad_at(idx_y[it], jp), true);
        const float in_x[4] = {qx.x, qx.y, qx.z, qx.w}, in_y[4] = {qy.x, qy.y, qy.z, qy.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool okx = rowx_ok[it] && jx + e >= 0 && jx + e <= hi_x;
          const bool oky = rowy_ok[it] && jp + e >= 0 && jp + e <= hi_y;
          vx[e] = okx ? fmaxf(__builtin_fmaf(in_x[e], in_scale, -gauge.x), kLogZero) : kLogZero;
          vy[e] = oky ? fmaxf(__builtin_fmaf(in_y[e], in_scale, -gauge.y), kLogZero) : kLogZero;
        }
      }
      const int pq = (kb % 3) * kQuadsPerBlock + mm;
      lds.fx[q][pq] = make_float4(vx[0], vx[1], vx[2], vx[3]);
      lds.fy[q][pq] = make_float4(vy[0], vy[1], vy[2], vy[3]);
    }
  };

  // the set of block kb carries the row above the chunk for block kb + 1
  auto commit_above = [&](int kb, FwdRegs &r) {
    if (lq != 0 || kb + 1 >= g.nblocks) return;
    const float4 qa = unmirror(AsFloat4(r.above), quad_at(idx_above, (kb + 1) * kW + 4 * mm - 1 + g.skew), true);
    const float in[4] = {qa.x, qa.y, qa.z, qa.w};
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int jx = (kb + 1) * kW + 4 * mm + e - 1 + g.skew;
      v[e] = g.c > 0 && jx >= 0 && jx <= hi_x ? fmaxf(__builtin_fmaf(in[e], in_scale, -gauge.x), kLogZero) : kLogZero;
    }
    *reinterpret_cast<float4 *>(&lds.px_above[(kb + 1) & 3][4 * mm]) = make_float4(v[0], v[1], v[2], v[3]);
  };

  // ---- storers ---------------------------------------------------------------------------
  auto store_block = [&](int kb) {  // LDS ring -> p
    if (kb < 0) return;
    // columns kb*32 - 63*skew .. kb*32 + 31 all inside 0..nt-1 (the end cell is never "inner"),
    // and every step of the block inside the half
    const bool inner = kb * kW - (kRows - 1) * g.skew >= 0 && kb * kW + kW - 1 <= g.nt - 1 &&
                       (!kBidir || kb * kW + kW - 1 <= n_last);
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int q = mq + 32 * it;
      const int row_i = g.row0 + q;
      if (row_i > g.ns) continue;
      const int pq = (kb % 3) * kQuadsPerBlock + mm;
      const float4 raw = lds.fy[q][pq];
      float4 v = raw;
      if (kWriteP || !inner) {  // p (or ans, on the rim) leaves the chain: stand-ins become -inf
        const float ninf = NegInfF();
        v.x = v.x < kLogZeroTest ? ninf : v.x;
        v.y = v.y < kLogZeroTest ? ninf : v.y;
        v.z = v.z < kLogZeroTest ? ninf : v.z;
        v.w = v.w < kLogZeroTest ? ninf : v.w;
      }
      const int j = kb * kW + 4 * mm - q * g.skew;  // column of element 0
      // where own columns j .. j+3 of the row lie: the mirrored half stores the lattice's cell
      // (ns - row, nt - column) one column to the right of its place, columns descending
      const ptrdiff_t at = (ptrdiff_t)(g.s0 + row_i) * LS + g.t0 + j;
      GFloat *dst = pb + at;
      float ld[4] = {0.f, 0.f, 0.f, 0.f};
      if (kKeep) {
        // What arrived along px at each step: for row 0 of the chunk the edge wavefront's sum
        // (row 64 of fx, same position); otherwise p of the row above one position earlier plus
        // this row's fx.  Stand-ins for -inf need no conversion here: anything that small gives
        // exp() = 0 in the backward, as -inf does.
        float t1[4];
        if (q == 0) {
          const float4 a = lds.fx[kWave][pq];
          t1[0] = a.x; t1[1] = a.y; t1[2] = a.z; t1[3] = a.w;
        } else {
          const float4 x4 = lds.fx[q][pq];
          float4 a = lds.fy[q - 1][pq];
          asm volatile("" : "+v"(a.x), "+v"(a.y), "+v"(a.z), "+v"(a.w));  // one 16-byte read
          float before;
          if (mm > 0) {
            float4 b4 = lds.fy[q - 1][pq - 1];
            asm volatile("" : "+v"(b4.x), "+v"(b4.y), "+v"(b4.z), "+v"(b4.w));
            before = b4.w;
          } else {
            // (single launch: the chain moved that value into this block's frame with the same
            // subtraction before lane q saw it)
            before = kb > 0 ? lds.last[(kb + 2) % 3][q - 1] : kLogZero;
            if (kBidir && kb > 0) before = fmaxf(before, -1.0e36f) - frame_step(kb);
          }
          t1[0] = before + x4.x; t1[1] = a.x + x4.y; t1[2] = a.y + x4.z; t1[3] = a.z + x4.w;
        }
        // the backward's "total": p of the cell, or 0 where p is not finite (the stand-in for
        // -inf counts as not finite)
        const float own[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          ld[e] = t1[e] - (__builtin_fabsf(own[e]) < -kLogZeroTest ? own[e] : 0.0f);
        if (mm == kQuadsPerBlock - 1) lds.last[kb % 3][q] = raw.w;
      }
      if (kBidir) {
        // Whole quads in the half's own order, also where the block reaches outside the box or
        // past the cut: the backward sweep decides by position what it uses.
        StoreQuadCoherent(ldb + (size_t)kb * kSlabBlockFloats + q * kW + 4 * mm,
                          make_float4(ld[0], ld[1], ld[2], ld[3]));
      } else if (inner) {  // uniform: every column of the block lies in 0..nt-1 for every row
        if (kWriteP) StoreQuad(dst, v);
        if (kKeep) StoreQuad(ldb + at, make_float4(ld[0], ld[1], ld[2], ld[3]));
      } else {
        asm volatile("");  // keeps this path a branch of its own
        const float vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (j + e >= 0 && j + e <= g.nt) {
            if (kWriteP) dst[e] = vv[e];
            if (kKeep) ldb[at + e] = ld[e];
          }
        if (!kBidir && row_i == g.ns) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (j + e == g.nt) ans[g.b] = GaveUp(hdr) ? __builtin_nanf("") : vv[e];
        }
      }
    }
  };

  // (single launch) The frame of block kb + 2, chosen in iteration kb by the first storer wavefront
  // (off the chain's path; a barrier lies between the choice and every use: the edge wavefront's
  // in iteration kb + 1, the chain's in kb + 2, the storers' in kb + 3): half way between the
  // largest and the smallest live value at the end of block kb - 2, the last one whose results all
  // storers have passed on, but never far below the largest (rows behind an all but blocked edge
  // carry no weight).  The gauge has taken the trend out of the values, so what they were four
  // blocks earlier is a fair guess of what they will be.
  auto choose_frame = [&](int kb) {
    const int to = (kb + 2) & (kFrameRing - 1), from = (kb + 1) & (kFrameRing - 1);
    float next = lds.frame[from];
    if (kb >= 2) {
      const float v = lds.last[(kb - 2) % 3][lane];
      const bool live = g.row0 + lane <= g.ns && v > kLogZeroTest;
      const float top = WaveMaxF(live ? v : -3.0e38f), bottom = -WaveMaxF(live ? -v : -3.0e38f);
      if (top > kLogZeroTest)
        next = RoundToFrame(lds.frame[(kb - 2) & (kFrameRing - 1)] + (top - fminf(0.5f * (top - bottom), 256.0f)));
    }
    if (lane == 0) {
      lds.shift[to] = next - lds.frame[from];
      lds.frame[to] = next;
    }
  };

  // ---- edge wavefront ----------------------------------------------------------------------
  // Lanes 0..31 prepare, for each step n of block kb, what arrives at lane 0 along px:
  //     p[row0-1][..] (taken from the chunk above) + px[row0-1][..]
  // and put it into row 64 of the fx array, which lane 0 of the chain reads in place of a row of
  // its own (the DPP add of the chain step leaves lane 0's register as it is).  The px values
  // of blocks 0 and 1 are loaded by this wavefront itself; from block 2 on they come from the
  // loaders' LDS ring, so that no load of this wavefront stands between it and the edge words
  // (its loads return in order, and a px value that came from HBM kept every hand-over waiting).
  auto edge_px = [&](int kb) -> float {
    const int jx = kb * kW + lane - 1 + g.skew;
    float v = kLogZero;
    if (g.c > 0 && lane < kW && jx >= 0 && jx <= hi_x)
      v = fmaxf(__builtin_fmaf(mirror ? pxb[(size_t)(g.s0 + g.ns - g.row0) * T1 + g.t0 + hi_x - jx]
                                      : pxb[(size_t)(g.s0 + g.row0 - 1) * T1 + g.t0 + jx],
                               in_scale, -gauge.x), kLogZero);
    return v;
  };
  // (single launch) frames of the chunk above that this wavefront has taken so far: the newest
  // one and the one before it, by block of the chunk above; wave-uniform
  int up_taken = frames_lo() - 1;
  float up_frame_new = 0.0f, up_frame_old = 0.0f;
  const int up_hi = kBidir && g.c > 0 && nblocks_up > 0 ? frames_hi(nblocks_up, g.nblocks) : -1;
  auto take_block = [&](int kb, float px_above) {
    if (kb >= g.nblocks) return;  // (uniform)
    const int n = kb * kW + lane;
    const int idx = n + edge_shift;
    const bool word = lane < kW && g.c > 0 && idx >= 0 && idx < nblocks_up * kW;
    // Lanes 32 and 33 take the frames of the blocks above that this block's words lie in, where
    // they have not been taken yet (blocks come in order, so at most two are new, and two only
    // for this chunk's first block), in the same trip to memory as the words.
    const int j_last = min((kb * kW + kW - 1 + edge_shift) / kW, up_hi);
    const int j_want = lane - kW + up_taken + 1;  // lane 32: the next one, lane 33: the one after
    const bool frame = kBidir && (lane == kW || lane == kW + 1) && j_want <= j_last;
    float v = kLogZero;
    if (word || frame) v = TakeEdge(word ? edge_in + idx : frame_in + j_want, hdr, word ? kLogZero : 0.0f);
    float own = 0.0f;  // (single launch) this block's frame
    if (kBidir) {
      const int got = min(j_last - up_taken, 2);  // (uniform) frames taken just now: <= 0, 1 or 2
      if (got == 2) {
        up_frame_old = LaneF(v, kW);
        up_frame_new = LaneF(v, kW + 1);
      } else if (got == 1) {
        up_frame_old = up_frame_new;
        up_frame_new = LaneF(v, kW);
      }
      if (got > 0) up_taken += got;
      if (kb == 0) {
        // a chunk's first two blocks take the frame of the first words that arrive (chunk 0: 0)
        own = got == 2 ? up_frame_old : (got == 1 ? up_frame_new : 0.0f);
        if (lane == 0) {
          lds.frame[0] = own;
          lds.frame[1] = own;
          lds.shift[0] = 0.0f;
          lds.shift[1] = 0.0f;
        }
      } else {
        own = lds.frame[kb & (kFrameRing - 1)];  // chosen by the chain two iterations ago
      }
    }
    if (lane < kW) {
      if (g.c == 0) {
        v = n == 0 ? 0.0f : kLogZero;  // the origin: p[s_begin][t_begin] = 0 "arrives" at step 0
      } else if (word) {
        // (single launch) from the frame of the block above that the word lies in to this block's
        if (kBidir) v = fmaxf(v, -1.0e36f) + ((idx / kW == up_taken ? up_frame_new : up_frame_old) - own);
        v += px_above;
      }
      reinterpret_cast<float *>(lds.fx[kWave])[(kb % 3) * kW + lane] = v;
    }
  };
  // lanes 32..63: hand block kb of the last row to the chunk below.  Only words the chunk below
  // will take are published, so the buffer ends the launch clean.
  const int down_hi = kBidir && has_down ? frames_hi(g.nblocks, nblocks_down) : -1;
  auto publish_block = [&](int kb) {
    if (has_down && kb >= 0) {
      const int n = kb * kW + (lane - kW);
      // the chunk below takes word n at its step n - edge_shift, which must exist; (single launch)
      // lane 0 sends the block's frame along, in the same instruction
      const bool word = lane >= kW && n >= edge_shift && n - edge_shift < nblocks_down * kW;
      const bool frame = kBidir && lane == 0 && kb >= frames_lo() && kb <= down_hi;
      if (word || frame)
        PublishEdge(word ? edge_out + n : frame_out + kb,
                    word ? reinterpret_cast<const float *>(&lds.fy[kWave - 1][0])[(kb % 3) * kW + (lane - kW)]
                         : lds.frame[kb & (kFrameRing - 1)]);
    }
  };

  // ---- chain wavefront ---------------------------------------------------------------------
  float P = kLogZero;
  const int fx_row = lane == 0 ? kWave : lane;
  auto chain_block = [&](int kb) {
    const int base = (kb % 3) * kQuadsPerBlock;
    P = fmaxf(P, -1.0e36f);  // lanes idling on the stand-in for -inf must never reach -inf itself
    const float into_frame = kBidir ? frame_step(kb) : 0.0f;  // (0 for the chunk's first block)
    float4 nfx = lds.fx[fx_row][base], nfy = lds.fy[lane][base];
    if (kBidir) P -= into_frame;  // into this block's frame (see Frames)
#pragma unroll
    for (int k = 0; k < kQuadsPerBlock; ++k) {
      const float4 fx4 = nfx, fy4 = nfy;
      if (k + 1 < kQuadsPerBlock) {
        nfx = lds.fx[fx_row][base + k + 1];
        nfy = lds.fy[lane][base + k + 1];
      }
      const float fxs[4] = {fx4.x, fx4.y, fx4.z, fx4.w};
      const float fys[4] = {fy4.x, fy4.y, fy4.z, fy4.w};
      float out[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        P = kBidir ? ChainStep2(P, fxs[e], fys[e]) : ChainStep(P, fxs[e], fys[e]);
        out[e] = P;
      }
      lds.fy[lane][base + k] = make_float4(out[0], out[1], out[2], out[3]);
    }
  };

  // the chain wavefront is the critical path: it wins the SIMD's issue arbitration
  if (role == kChain) __builtin_amdgcn_s_setprio(3);
  // ---- prologue: block 0 committed, blocks 1 .. kFwdSets in flight --------------------------
  // A block's loads stay in flight for kFwdSets iterations (~1.2 us each).  Two sets serve the
  // separate forward kernel, whose registers decide whether a second workgroup fits a compute
  // unit.  The single launch has a unit per workgroup, and 2 x 256 of its sweeps read from HBM at
  // once: there two sets leave every iteration waiting for its loads when the inputs are not in
  // the Infinity Cache (1.55 us per block against 1.2).
#ifndef K2AMD_FWD_SETS
#define K2AMD_FWD_SETS 2
#endif
  constexpr int kFwdSets = kBidir ? K2AMD_FWD_SETS : 2;
  FwdRegs sets[kFwdSets];
  if (role == kLoader) {
    float gauge_v = 0.0f;
    if (kBidir) {  // the gauge's sample, in the same trip to memory as block 0
      // (a float that exists, for every lane: the tensor's first one where the lane has no sample)
      const GFloat *src = !gauge_valid ? Global(px)
                          : (lane & kGaugeSample) ? Global(py) + gauge_idx_y + (lane & (kGaugeSample - 1))
                                                  : Global(px) + gauge_idx_x + (lane & (kGaugeSample - 1));
      asm volatile("global_load_dword %0, %1, off" : "=v"(gauge_v) : "v"(src) : "memory");
    }
    load_block(0, sets[0]);
    WaitLoads<0>(sets[0]);
    if (kBidir) {
      // (every load of this wavefront has landed; nothing reads the sample in front of this)
      asm volatile("" : "+v"(gauge_v));
      gauge = GaugeOf(gauge_v, gauge_valid, g.ns);
      if (gauge_out != nullptr && mid == 0) {
        PublishCut(gauge_out, gauge.x);
        PublishCut(gauge_out + 1, gauge.y);
      }
    }
    commit_block(0, sets[0]);
    commit_above(0, sets[0]);
#pragma unroll
    for (int i = 0; i < kFwdSets; ++i) load_block(1 + i, sets[i]);
  } else if (role == kEdge) {
    if (kBidir && g.c > 0) {  // the same sample, the same arithmetic: the same gauge
      const GFloat *src = (lane & kGaugeSample) ? Global(py) + gauge_idx_y : Global(px) + gauge_idx_x;
      float v = 0.0f;
      if (gauge_valid) v = src[lane & (kGaugeSample - 1)];
      gauge = GaugeOf(v, gauge_valid, g.ns);
    }
    take_block(0, edge_px(0));
  }
  K2AMD_TRACE_MARK(half, 4);
  LdsBarrier();
  K2AMD_TRACE_MARK(half, 5);

  // In iteration kb the chain wavefront computes block kb; the loaders commit block kb+1 (loaded
  // kFwdSets iterations ago) and start the loads of block kb+1+kFwdSets; the storers drain block kb-1; the
  // edge wavefront publishes block kb-1 downwards and takes block kb+1 from the chunk above.
  // Every role runs its own loop (same number of barriers), which keeps each loop free of the
  // other roles' code and lets the compiler count outstanding loads exactly.
  if (role == kChain) {
    for (int kb = 0; kb < g.nblocks; ++kb) {
      chain_block(kb);
#ifdef K2AMD_MI_TRACE
      if (kBidir && kb < 24) K2AMD_TRACE_MARK(half, 8 + kb);
#endif
      LdsBarrier();
    }
  } else if (role == kLoader) {
    for (int kb = 0; kb < g.nblocks; kb += kFwdSets) {
#pragma unroll
      for (int i = 0; i < kFwdSets; ++i) {
        if (kb + i >= g.nblocks) break;
        WaitLoads<(kFwdSets - 1) * kFwdLoadsPerBlock>(sets[i]);  // the other sets' loads may stay in flight
        commit_block(kb + i + 1, sets[i]);
        commit_above(kb + i + 1, sets[i]);
        load_block(kb + i + 1 + kFwdSets, sets[i]);
        LdsBarrier();
      }
    }
    // the loads of the blocks past the end are still in flight: they must land before the
    // compiler may give their registers to anything else
#pragma unroll
    for (int i = 0; i < kFwdSets; ++i) WaitLoads<0>(sets[i]);
  } else if (role == kStorer) {
    for (int kb = 0; kb < g.nblocks; ++kb) {
      store_block(kb - 1);
      if (kBidir && wave == 2 + L::kLoaderWaves) choose_frame(kb);
      LdsBarrier();
    }
  } else if (role == kEdge) {
    float px_above = edge_px(1);
    for (int kb = 0; kb < g.nblocks; ++kb) {
      publish_block(kb - 1);
      take_block(kb + 1, px_above);
      LdsBarrier();
      px_above = lds.px_above[(kb + 2) & 3][lane & (kW - 1)];  // committed in this iteration
    }
  }
  K2AMD_TRACE_MARK(half, 6);
  if (role == kStorer) store_block(g.nblocks - 1);
  if (role == kEdge) publish_block(g.nblocks - 1);
  if (kBidir && role == kChain) {
    // What the chain left on the cut diagonal: step n_last of every row, still in the ring.  (A
    // chunk that ran out of columns before the cut has no cell on it; a row whose cell on the cut
    // lies outside the columns holds a stand-in for -inf there already.)  The words validate
    // themselves, so the sequence's join on the cut starts as soon as they land, while the other
    // wavefronts' log-derivatives are still on their way.
    const int at = ((g.nblocks - 1) % 3) * kW + (n_last - (g.nblocks - 1) * kW);
    const bool on_cut = half.dmax - g.row0 * g.skew == n_last && g.row0 + lane <= g.ns;
    PublishCut(cut_out + lane, on_cut ? reinterpret_cast<const float *>(&lds.fy[lane][0])[at] : kLogZero);
    if (lane == 0) PublishCut(cut_frame_out, lds.frame[(g.nblocks - 1) & (kFrameRing - 1)]);
  }
  if (kBidir) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the coherent stores above
}

// One workgroup per chunk; the ticket fixes which (see the file header).
template <bool kKeep, bool kWriteP>
__global__ __launch_bounds__(FwdLayout::kThreads) void MiForwardFastKernel(
    const float *__restrict__ px, const float *__restrict__ py,
    const int64_t *__restrict__ boundary, float *__restrict__ p, float *__restrict__ ans,
    float *__restrict__ log_deriv, FastHeader *hdr, float *edge, int B, int S, int Tn,
    int modified, int nchunks, int edge_stride) {
  __shared__ FwdLds lds;
  if (threadIdx.x == 0) lds.ticket = atomicAdd(&hdr->ticket, 1u);
  __syncthreads();
  const unsigned ticket = lds.ticket;
  MiForwardChunk<kKeep, kWriteP, false>(lds, px, py, LoadBox(boundary, (int)(ticket / nchunks), S, Tn), p,
                                        ans, log_deriv, hdr, edge, B, S, Tn, modified, nchunks,
                                        edge_stride, (int)(ticket / nchunks), (int)(ticket % nchunks),
                                        Half{}, nullptr, nullptr, nullptr);
  if (threadIdx.x == 0) PutTicketsBack(hdr, lds.ticket, gridDim.x);
}

// ------------------------------------------------------------------------------ backward
//
// Mass-flow form of the reference's backward sweep (k2/python/csrc/torch/
// mutual_information_cpu.cu:179-251).  For a destination cell D = (s, t) that holds gradient g:
//     d1 = exp(p[s-1][t+o] + px[s-1][t+o] - p[s][t])        (o = -1 modified, 0 regular)
//     h  = d1 * g        -> px_grad[s-1][t+o], and flows to cell (s-1, t+o)
//     c  = (1 - d1) * g  -> py_grad[s][t-1],   and flows to cell (s, t-1)
// so every cell needs ONE exponential, computed by the loader wavefronts (E = d1, OME = 1 - d1,
// with the reference's guards folded in: first row E = 0, first column of a regular lattice
// E = 1, non-finite d1 -> both 0).  The chain wavefront then does, per position m (descending),
//     h = E * G;  c = OME * G;  G' = c + h(lane + 1) = OME * G + E(lane + 1) * G(lane + 1)
// i.e. two multiplies for the outputs, one DPP multiply and one FMA for the recursion.  Lane l
// handles lattice row row0 + l; lane 63 has no lane below it in the wavefront and receives the h
// of the first row of the chunk below, so here the LOWER chunk runs ahead.
struct BwdLds {
  // rows 0..63: d1 of the row's cells; row 64: the h arriving from the chunk below, laid out like
  // a row so that every lane reads "the row below it" the same way
  float4 e[kWave + 1][kQuadsPerRow];
  float4 ome[kWave][kQuadsPerRow];  // 1 - d1
  // what the chain leaves behind: the gradient of each row AFTER the step at a position, which is
  // the gradient the cell one position to the right saw (the storers multiply it with that cell's
  // d1 and 1 - d1)
  float4 g[kWave][kQuadsPerRow];
  unsigned ticket;
};

struct BwdRegs {
  float4v d[BwdLayout::kLoadItems], s[BwdLayout::kLoadItems], x[BwdLayout::kLoadItems];  // p[dest], p[src], px[src]
};
template <int kYounger>
__device__ __forceinline__ void WaitLoads(BwdRegs &r) {
  static_assert(BwdLayout::kLoadItems == 2, "operand list below");
  asm volatile("s_waitcnt vmcnt(%6)"
               : "+v"(r.d[0]), "+v"(r.s[0]), "+v"(r.x[0]), "+v"(r.d[1]), "+v"(r.s[1]), "+v"(r.x[1])
               : "n"(kYounger));
}
// with kept log-derivatives only r.d is loaded
template <int kYounger>
__device__ __forceinline__ void WaitKeptLoads(BwdRegs &r) {
  static_assert(BwdLayout::kLoadItems == 2, "operand list below");
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(r.d[0]), "+v"(r.d[1]) : "n"(kYounger));
}

// Clears the four columns c..c+3 of array row r of px_grad / py_grad wherever they lie outside
// the region the sweep assigns.
struct ZeroGeom {
  float *gx, *gy;
  int S, T1, Tn;
  int xs0, xs1, xt0, xt1;  // px_grad region assigned by the sweep: rows [xs0,xs1) cols [xt0,xt1)
  int ys1, yt1;            // py_grad region: rows [xs0,ys1) cols [xt0,yt1)
};
__device__ __forceinline__ void ZeroItem(const ZeroGeom &z, int r, int c) {
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  if (r < z.S && c < z.T1) {
    GFloat *dst = Global(z.gx) + (size_t)r * z.T1 + c;
    const bool row_in = r >= z.xs0 && r < z.xs1;
    if (row_in && c >= z.xt0 && c + 3 < z.xt1) {
      // the sweep assigns all four
    } else if (c + 3 < z.T1 && !(row_in && c + 3 >= z.xt0 && c < z.xt1)) {
      StoreQuad(dst, zero);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c + e < z.T1 && !(row_in && c + e >= z.xt0 && c + e < z.xt1)) dst[e] = 0.0f;
    }
  }
  if (r <= z.S && c < z.Tn) {
    GFloat *dst = Global(z.gy) + (size_t)r * z.Tn + c;
    const bool row_in = r >= z.xs0 && r < z.ys1;
    if (row_in && c >= z.xt0 && c + 3 < z.yt1) {
      // the sweep assigns all four
    } else if (c + 3 < z.Tn && !(row_in && c + 3 >= z.xt0 && c < z.yt1)) {
      StoreQuad(dst, zero);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (c + e < z.Tn && !(row_in && c + e >= z.xt0 && c + e < z.yt1)) dst[e] = 0.0f;
    }
  }
}

// kKept: `p` is the log_deriv tensor a kKeep forward launch wrote (same layout as p), px is not
// read, and every cell's d1 is exp() of one loaded value.
// The whole workgroup sweeps chunk `chunk` of sequence `seq`, or (zero_only) clears what the
// sweep leaves unassigned in array rows chunk * 64 .. chunk * 64 + 63 of that sequence.
// kBidir: the sweep covers the half `half` (see Half), whose forward sweep left its
// log-derivatives in `p` (the launch's slab of blocks); it starts on the cut diagonal, where
// every row of the half holds its cell's share of all paths times the gradient of the sequence's
// score (WaveCutJoin, run by the chain wavefront while the loaders fetch the first blocks),
// instead of at the end cell.
template <bool kKept, bool kBidir>
__device__ __forceinline__ void MiBackwardChunk(
    BwdLds &lds, const float *__restrict__ px, const float *__restrict__ p, const Box &box,
    float *__restrict__ ans_grad,
    float *__restrict__ px_grad, float *__restrict__ py_grad, FastHeader *hdr, float *edge, int B,
    int S, int Tn, int modified, int nchunks, int edge_stride, int overwrite_ans_grad, int seq,
    int chunk, bool zero_only, Half half, const BidirJoin *join) {
  static_assert(!kBidir || kKept, "the halves hand over log-derivatives");
  ChunkGeom g;
  g.b = seq;
  g.c = chunk;
  const int T1 = modified ? Tn : Tn + 1;
  const int off = modified ? -1 : 0;
  GFloat *gxb = Global(px_grad) + (size_t)g.b * S * T1;
  GFloat *gyb = Global(py_grad) + (size_t)g.b * (S + 1) * Tn;

  if (zero_only) {
    ZeroGeom zg;
    zg.gx = px_grad + (size_t)g.b * S * T1; zg.gy = py_grad + (size_t)g.b * (S + 1) * Tn; zg.S = S; zg.T1 = T1; zg.Tn = Tn;
    zg.xs0 = box.ok ? box.s0 : 0; zg.xs1 = box.ok ? box.s1 : 0;
    zg.xt0 = box.ok ? box.t0 : 0; zg.xt1 = box.ok ? box.t1 + off + 1 : 0;
    zg.ys1 = box.ok ? box.s1 + 1 : 0; zg.yt1 = box.ok ? box.t1 : 0;
    const int zslices = (T1 + 31) / 32;
    if (threadIdx.x < kRows * 8)
      for (int sl = 0; sl < zslices; ++sl)
        ZeroItem(zg, g.c * kRows + (threadIdx.x >> 3), sl * 32 + 4 * (threadIdx.x & 7));
    return;
  }

  g.s0 = box.s0; g.t0 = box.t0; g.ns = box.s1 - box.s0; g.nt = box.t1 - box.t0;
  g.row0 = g.c * kRows;
  if (!box.ok || g.row0 > g.ns) return;  // nothing to sweep
  g.skew = modified ? 0 : 1;
  const int mirror = kBidir ? half.mirror : 0;
  const int npos_full = g.nt + 2 + (kRows - 1) * g.skew;  // one virtual column right of the end cell
  // positions (and 32-position blocks) of the chunk at local row r0: one past its step on the cut
  auto npos_of = [&](int r0) { return kBidir ? min(npos_full, half.dmax - r0 * g.skew + 2) : npos_full; };
  auto blocks_of = [&](int r0) { return npos_of(r0) >= 2 ? (npos_of(r0) + kW - 1) / kW : 0; };
  const int npos = npos_of(g.row0);
  const int n_last = npos - 2;  // the chunk's position on the cut diagonal (kBidir)
  g.nblocks = blocks_of(g.row0);
  if (kBidir && g.nblocks == 0) return;  // no cell of these rows lies in the half
  const bool has_down = g.row0 + kRows <= g.ns && blocks_of(g.row0 + kRows) > 0;
  const bool has_up = g.c > 0;
  const int nblocks_down = has_down ? blocks_of(g.row0 + kRows) : 0;
  const int nblocks_up = has_up ? blocks_of(g.row0 - kRows) : 0;
  const int LS = Tn + 1;  // floats per row of p / the log-derivatives (the two-kernel pair's tensors)
  const int edge_shift = kRows * g.skew;  // position m here <-> position m - edge_shift one chunk down
  float *edge_out = edge + ((size_t)g.b * nchunks + g.c) * edge_stride;     // read by chunk c-1
  float *edge_in = edge + ((size_t)g.b * nchunks + g.c + 1) * edge_stride;  // from chunk c+1

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  typedef BwdLayout L;
  constexpr int kLoadItems = L::kLoadItems, kRowStep = L::kRowStep;
  const int role = RoleOf<L>(wave);
  const int mid = MoverLane<L>(wave, lane);  // lane id among the loader (or storer) lanes
  const int mq = mid >> 3, mm = mid & 7;     // storers: rows mq and mq + 32, quad mm
  const int lq = mq;                         // loaders: rows lq + kRowStep*it, quad mm

  // ---- loaders ---------------------------------------------------------------------------
  // destination cells with both edges exist only for rows 1..ns and columns 1..nt
  // (kBidir: `p` is the launch's slab, and this chunk of this half has a run of blocks in it)
  const int slab_blocks = SlabBlocks(S, Tn, modified);
  const int4v rsp = kBidir ? MakeResource(p + (size_t)g.b * SlabFloatsPerSequence(S, Tn, modified) +
                                              (size_t)(mirror * nchunks + g.c) * slab_blocks * kSlabBlockFloats,
                                          (size_t)slab_blocks * kSlabBlockFloats)
                           : MakeResource(p, (size_t)B * (S + 1) * LS);
  const int4v rsx = MakeResource(px, (size_t)B * S * T1);
  // float index of destination column 0 of the item's row: p[dest], and p / px of the source
  // cell of the px edge (column jd - 1 + skew of the row above)
  int idx_d[kLoadItems], idx_s[kLoadItems], idx_x[kLoadItems];
#pragma unroll
  for (int it = 0; it < kLoadItems; ++it) {
    const int rc = min(max(g.row0 + lq + kRowStep * it, 1), max(g.ns, 1));  // a row with a row above
    // (kBidir: the item's row inside a block of the slab)
    idx_d[it] = kBidir ? (lq + kRowStep * it) * kW : (g.b * (S + 1) + g.s0 + rc) * LS + g.t0;
    idx_s[it] = (g.b * (S + 1) + g.s0 + rc - 1) * (Tn + 1) + g.t0 + g.skew - 1;
    idx_x[it] = (g.b * S + g.s0 + rc - 1) * T1 + g.t0 + g.skew - 1;
  }
  // every destination cell of block kb has both edges inside the box (and lies in the half)?
  // (uniform)
  auto interior = [&](int kb) {
    return kb * kW - (kRows - 1) * g.skew >= 1 && kb * kW + 31 <= g.nt &&
           (!kBidir || kb * kW + 31 <= n_last);
  };
  // Rows past the sequence's last row never change: their E / OME stay at the zeros written
  // here, the loaders skip them.
  bool row_ok[kLoadItems];
#pragma unroll
  for (int it = 0; it < kLoadItems; ++it) row_ok[it] = g.row0 + lq + kRowStep * it <= g.ns;
  if (g.row0 + kRows - 1 > g.ns) {
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int i = threadIdx.x; i < kWave * kQuadsPerRow; i += L::kThreads) {
      const int q = i / kQuadsPerRow, k = i - q * kQuadsPerRow;
      if (g.row0 + q > g.ns) {
        lds.e[q][k] = zero4;
        lds.ome[q][k] = zero4;
      }
    }
  }
  // One code path for every block: quads that reach outside the valid columns pick up
  // neighbouring floats (or zeros past the tensor's end) that the commit masks.
  // Always issues kLoadsPerBlock loads, so that the counts given to WaitLoads hold in every
  // iteration; for blocks in front of the first one it reads block 0 again, and rows past the
  // sequence's end read its last row (cache hits both).
  constexpr int kLoadsPerBlock = (kKept ? 1 : 3) * kLoadItems;
  auto load_block = [&](int kb, BwdRegs &r) {
    kb = max(kb, 0);
#pragma unroll
    for (int it = 0; it < kLoadItems; ++it) {
      const int jd = kb * kW + 4 * mm - (lq + kRowStep * it) * g.skew;  // destination column of element 0
      r.d[it] = kBidir ? AsyncQuadCoherent(rsp, idx_d[it] + kb * kSlabBlockFloats + 4 * mm)
                       : AsyncQuad(rsp, idx_d[it] + jd);
      if (!kKept) {
        r.s[it] = AsyncQuad(rsp, idx_s[it] + jd);
        r.x[it] = AsyncQuad(rsx, idx_x[it] + jd);
      }
    }
  };
  auto wait_all = [&](BwdRegs &r) {
    if (kKept) WaitKeptLoads<0>(r); else WaitLoads<0>(r);
  };
  // A block's loads stay in flight for kSets iterations.  With kept log-derivatives the
  // loaders' work is light enough for the iteration to drop under half a trip to memory: two
  // sets (as in the forward, whose iterations are twice as long) would make every iteration wait
  // for its loads (measured: 42 us per launch with two sets, 31 us with three or more).  The
  // plain kernel is bound by its movers' instruction issue and gains nothing from a third set.
  constexpr int kSets = kKept ? 4 : 2;
  auto wait_older = [&](BwdRegs &r) {  // the younger sets' loads may stay in flight
    if (kKept) WaitKeptLoads<(kSets - 1) * kLoadsPerBlock>(r); else WaitLoads<(kSets - 1) * kLoadsPerBlock>(r);
  };
  // E / OME of a destination cell that has both edges inside the box; pd, ps, xs = p[dest],
  // p[src], px[src] (k2/python/csrc/torch/mutual_information_cpu.cu:195-211).
  auto flow = [&](float pd, float ps, float xs, float *e_out, float *o_out) {
    const float total = __builtin_isfinite(pd) ? pd : 0.0f;
    const float d1 = kBidir ? __builtin_amdgcn_exp2f(pd) : __expf(kKept ? pd : (ps + xs) - total);
    const bool fin = __builtin_isfinite(d1);
    *e_out = fin ? d1 : 0.0f;
    *o_out = fin ? 1.0f - d1 : 0.0f;
  };
  // The same for a cell on or outside the rim of the box (column j; select-only code).
  auto rim = [&](bool first_row, bool last_row, int j, int m, float *e_io, float *o_io) {
    const bool in = j >= 1 && j <= g.nt;
    const bool col0_up = j == 0 && !modified;  // regular first column flows up
    float e_v = in ? *e_io : (col0_up ? 1.0f : 0.0f);
    float o_v = in ? *o_io : 0.0f;
    // first row: everything flows along py
    e_v = first_row ? 0.0f : e_v;
    o_v = first_row ? (in ? 1.0f : 0.0f) : o_v;
    // virtual cells right of the end cell hand the seed leftwards unchanged; so do, in a half,
    // the positions past the cut diagonal in every row
    const bool virt = kBidir ? m > n_last : last_row && j > g.nt;
    *e_io = virt ? 0.0f : e_v;
    *o_io = virt ? 1.0f : o_v;
  };
  // `inner` is uniform over the workgroup: the rim code below it is a real branch (the empty asm
  // statements keep the compiler from flattening it into selects that every block would pay for).
  auto commit_block = [&](int kb, BwdRegs &r) {
    if (kb < 0) return;
    const bool inner = interior(kb);
#pragma unroll
    for (int it = 0; it < kLoadItems; ++it) {
      if (!row_ok[it]) continue;
      const int q = lq + kRowStep * it;
      float4 qd = AsFloat4(r.d[it]);
      float4 qs = kKept ? qd : AsFloat4(r.s[it]), qx = kKept ? qd : AsFloat4(r.x[it]);
      // (the slab's quads are whole by construction)
      if (!kBidir && !inner) {  // (a quad can start in front of the tensor: see ShiftQuad)
        asm volatile("");
        const int jd0 = kb * kW + 4 * mm - q * g.skew;
        qd = ShiftQuad(qd, idx_d[it] + jd0);
        if (!kKept) {
          qs = ShiftQuad(qs, idx_s[it] + jd0);
          qx = ShiftQuad(qx, idx_x[it] + jd0);
        }
      }
      float ve[4], vo[4];
      flow(qd.x, qs.x, qx.x, &ve[0], &vo[0]);
      flow(qd.y, qs.y, qx.y, &ve[1], &vo[1]);
      flow(qd.z, qs.z, qx.z, &ve[2], &vo[2]);
      flow(qd.w, qs.w, qx.w, &ve[3], &vo[3]);
      if (inner) {
        // only the sequence's first row (lane 0 of chunk 0) differs from the plain formula
        if (it == 0 && g.row0 == 0) {
          const bool first_row = q == 0;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ve[e] = first_row ? 0.0f : ve[e];
            vo[e] = first_row ? 1.0f : vo[e];
          }
        }
      } else {
        asm volatile("");
        const int row_i = g.row0 + q;
        const int jd = kb * kW + 4 * mm - q * g.skew;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          rim(row_i == 0, row_i == g.ns, jd + e, jd + e + q * g.skew, &ve[e], &vo[e]);
      }
      const int pq = (kb % 3) * kQuadsPerBlock + mm;
      lds.e[q][pq] = make_float4(ve[0], ve[1], ve[2], ve[3]);
      lds.ome[q][pq] = make_float4(vo[0], vo[1], vo[2], vo[3]);
    }
  };

  // ---- storers ---------------------------------------------------------------------------
  // The gradient G a cell at position m saw is what the chain left at position m + 1, which for
  // the last position of a block lies in the block to its right (computed one iteration earlier;
  // its slot in g is not written again before the chain reaches the block two to the left).
  // Where a storer lane's two items (rows mq and mq + 32, quad mm) of block 0 go; block kb lies
  // kb * 32 floats further on (back, in the mirrored half).  Worked out once: per block the
  // storers only add.
  //   py_grad[s][t0 + jd - 1 + e]   for destination columns 1..nt
  //   px_grad[s-1][t0 + jd - 1 + skew + e]   for destination columns (1 - skew)..nt
  // The mirrored half's destination cell (row, column) is the lattice's cell (ns - row,
  // nt - column), and what flows into it along its px / py edge is the flow OUT of that lattice
  // cell along px / py: both gradients land at that cell's own index, columns descending.
  // (Set by the storers when their loop starts, and their last block is stored inside their
  // branch: pointers that were live where the roles part would cost every role their registers.)
  GFloat *dy0[2], *dx0[2];
  const ptrdiff_t block_step = mirror ? -kW : kW;
  auto storer_bases = [&]() {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int q = mq + 32 * it;
      const int row_i = g.row0 + q;
      const int jd = 4 * mm - q * g.skew;
      const int s = g.s0 + row_i, sm = g.s0 + g.ns - row_i;
      dy0[it] = mirror ? gyb + (ptrdiff_t)sm * Tn + g.t0 + g.nt - jd - 3 : gyb + (ptrdiff_t)s * Tn + g.t0 + jd - 1;
      dx0[it] = mirror ? gxb + (ptrdiff_t)sm * T1 + g.t0 + g.nt - jd - 3
                       : gxb + (ptrdiff_t)(s - 1) * T1 + g.t0 + jd - 1 + g.skew;
    }
  };
  auto store_block = [&](int kb) {
    if (kb >= g.nblocks) return;
    const bool inner = interior(kb);
    const int ring = __builtin_amdgcn_readfirstlane(kb % 3);
    const int pq = ring * kQuadsPerBlock + mm;
    const int pq_right = mm + 1 < kQuadsPerBlock ? pq + 1 : (ring == 2 ? 0 : ring + 1) * kQuadsPerBlock;
    // Both items' operands are asked for before either is used (one LDS latency per block) where
    // the registers allow it: the plain backward's loaders hold three tensors' loads, and its
    // kernel must stay within the registers that let two workgroups share a compute unit.
    float4 e4[2], o4[2], g4[2], gr[2];
    auto fetch = [&](int it) {
      const int q = mq + 32 * it;
      e4[it] = lds.e[q][pq];
      o4[it] = lds.ome[q][pq];
      g4[it] = lds.g[q][pq];
      gr[it] = lds.g[q][pq_right];
      // Only three floats of g4 and one of gr are used, and the compiler would fetch just those
      // with 4-byte reads: lanes that are whole quads apart then share 16 of the 64 banks (4-way
      // conflicts).  Whole-quad reads are conflict-free.
      asm volatile("" : "+v"(g4[it].x), "+v"(g4[it].y), "+v"(g4[it].z), "+v"(g4[it].w));
      asm volatile("" : "+v"(gr[it].x), "+v"(gr[it].y), "+v"(gr[it].z), "+v"(gr[it].w));
    };
    if (kKept) {
      fetch(0);
      fetch(1);
    }
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int q = mq + 32 * it;
      const int row_i = g.row0 + q;
      if (row_i > g.ns) continue;
      if (!kKept) fetch(it);
      const float gv[4] = {g4[it].y, g4[it].z, g4[it].w, gr[it].x};
      const float hv[4] = {e4[it].x * gv[0], e4[it].y * gv[1], e4[it].z * gv[2], e4[it].w * gv[3]};
      const float cv[4] = {o4[it].x * gv[0], o4[it].y * gv[1], o4[it].z * gv[2], o4[it].w * gv[3]};
      GFloat *dy = dy0[it] + kb * block_step;
      GFloat *dx = dx0[it] + kb * block_step;
      if (inner) {  // uniform: every cell of the block has both edges inside the box
        const float4 c4 = make_float4(cv[0], cv[1], cv[2], cv[3]), h4 = make_float4(hv[0], hv[1], hv[2], hv[3]);
        StoreQuad(dy, kBidir && mirror ? Rev4(c4) : c4);
        if (row_i >= 1) StoreQuad(dx, kBidir && mirror ? Rev4(h4) : h4);
      } else {
        asm volatile("");  // keeps this path a branch of its own
        const int jd = kb * kW + 4 * mm - q * g.skew;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (jd + e >= 1 && jd + e <= g.nt && (!kBidir || jd + e + q * g.skew <= n_last))
            dy[kBidir && mirror ? 3 - e : e] = cv[e];
        if (row_i >= 1) {
          const int lo = 1 - g.skew;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (jd + e >= lo && jd + e <= g.nt && (!kBidir || jd + e + q * g.skew <= n_last))
              dx[kBidir && mirror ? 3 - e : e] = hv[e];
        }
      }
    }
  };

  // ---- edge wavefront ----------------------------------------------------------------------
  auto take_block = [&](int kb) {
    if (lane < kW && kb >= 0) {
      const int mpos = kb * kW + lane;
      float v = 0.0f;
      if (has_down) {
        const int idx = mpos - edge_shift;  // position of the same column in the chunk below
        if (idx >= 0 && idx < nblocks_down * kW) v = TakeEdge(edge_in + idx, hdr, 0.0f);
      }
      reinterpret_cast<float *>(lds.e[kWave])[(kb % 3) * kW + lane] = v;
    }
  };
  // Lanes 32..63 hand the h of the chunk's first row (d1 times the gradient the cell saw, see
  // store_block) to the chunk above.  Only words that chunk will take are published (positions
  // it maps inside its range).
  auto publish_block = [&](int kb) {
    if (has_up && kb < g.nblocks && lane >= kW) {
      const int i = lane - kW;
      const int mpos = kb * kW + i;
      if (mpos + edge_shift < nblocks_up * kW) {
        const float e0 = reinterpret_cast<const float *>(&lds.e[0][0])[(kb % 3) * kW + i];
        const int right = i + 1 < kW ? (kb % 3) * kW + i + 1 : ((kb + 1) % 3) * kW;
        PublishEdge(edge_out + mpos, e0 * reinterpret_cast<const float *>(&lds.g[0][0])[right]);
      }
    }
  };

  // ---- chain wavefront ---------------------------------------------------------------------
  // gradient at the (virtual) right end of each row: the seed on the sequence's last row
  float G = 0.0f;
  if (!kBidir && role == kChain && g.row0 + lane == g.ns) G = ans_grad != nullptr ? ans_grad[g.b] : 1.0f;
  float g_origin = 0.0f;
  // Per position (descending), with OME of the own row and Edn = d1 of the row below (lane + 1):
  //     G' = OME * G + Edn * G(lane + 1)
  // one DPP multiply and one FMA; G' goes to LDS, the storers turn it into px_grad / py_grad.
  // Lane 63 has no lane below it: the DPP multiply leaves its register untouched, and what that
  // register holds is row 64 of the E array, the h arriving from the chunk below.  The DPP read
  // of G needs two wait states after the FMA that wrote it.
  auto chain_block = [&](int kb) {
    const int base = (kb % 3) * kQuadsPerBlock;
    float4 nd = lds.e[lane + 1][base + kQuadsPerBlock - 1], no = lds.ome[lane][base + kQuadsPerBlock - 1];
#pragma unroll
    for (int k = kQuadsPerBlock - 1; k >= 0; --k) {
      const float4 d4 = nd, o4 = no;
      if (k > 0) {
        nd = lds.e[lane + 1][base + k - 1];
        no = lds.ome[lane][base + k - 1];
      }
      float ts[4] = {d4.x, d4.y, d4.z, d4.w};
      const float os[4] = {o4.x, o4.y, o4.z, o4.w};
#pragma unroll
      for (int e = 3; e >= 0; --e) {
        if (kb == 0 && k == 0 && e == 0) g_origin = G;
        asm volatile(
            "s_nop 1\n\t"
            "v_mul_f32_dpp %[t], %[G], %[t] wave_shl:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_fmac_f32 %[t], %[O], %[G]"
            : [t] "+&v"(ts[e])
            : [O] "v"(os[e]), [G] "v"(G));
        G = ts[e];
      }
      lds.g[lane][base + k] = make_float4(ts[0], ts[1], ts[2], ts[3]);
    }
  };

  const int top = g.nblocks - 1;
  BwdRegs sets[kSets];
  unsigned departed_early = 0;  // (chain wavefront, lane 0, single launch)
  auto sh_of = [](const BidirJoin *j) { return j->sh; };
  if (kBidir) {
    // The chain wavefront joins the halves on the cut; the loaders wait for the forward sweeps'
    // last log-derivatives (all of the sequence's: the counter is per sequence) and fetch the
    // first blocks meanwhile.  The edge wavefront asks the chunk below for nothing before the
    // join has said that the halves sweep back at all: where the score is not finite no chunk
    // of the sequence publishes anything.
    CutShared &sh = *join->sh;
    if (role == kChain) {
      float scale;
      K2AMD_TRACE_MARK(half, 7);
      const float total = WaveCutJoin(sh, join->cw, g.ns, modified ? g.nt - g.ns : g.nt, g.row0, mirror, hdr, &G, &scale);
      K2AMD_TRACE_MARK(half, 3);
      if (lane == 0) {
        const bool ok = total > kLogZeroTest;  // a finite score
        sh.total = total;
        sh.scale = scale;
        sh.split_ok = ok;
        if (join->ans != nullptr && ok) *join->ans = GaveUp(hdr) ? __builtin_nanf("") : total;
      }
      K2AMD_TRACE_MARK(half, 1);
    } else if (role == kLoader) {
      const unsigned per_seq = 2u * nchunks;
      if (lane == 0) WaitCount(join->cw.stored, kSentinel + per_seq, hdr);
      load_block(top, sets[0]);
      wait_all(sets[0]);
      commit_block(top, sets[0]);
#pragma unroll
      for (int i = 0; i < kSets; ++i) load_block(top - 1 - i, sets[i]);
    }
    LdsBarrier();
    // This task is through with the sequence's words: the chain has read the cut and, behind the
    // barrier, the loaders have seen the count of the forward sweeps' stores.  Said now, so that
    // the answer is back by the time the sweep ends (it is looked at there; a trip to memory off
    // the launch's tail), and not before the barrier: the task that departs last puts every word
    // of the sequence back, that count included, and a loader still waiting for it to reach its
    // final value would then wait until its bound expires.
    if (role == kChain && lane == 0)
      departed_early = __hip_atomic_fetch_add(Global(join->cw.depart), 1u, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
    if (!sh.split_ok) {
      if (role == kLoader) {
#pragma unroll
        for (int i = 0; i < kSets; ++i) wait_all(sets[i]);
      }
      if (threadIdx.x == 0) {
        sh.departed = departed_early;
        sh.departed_set = 1;
      }
      return;
    }
    // what the cells of the top block's last position saw: the initial gradient
    if (role == kChain) reinterpret_cast<float *>(&lds.g[lane][((top + 1) % 3) * kQuadsPerBlock])[0] = G;
    if (role == kEdge) take_block(top);
    K2AMD_TRACE_MARK(half, 4);
    LdsBarrier();
    K2AMD_TRACE_MARK(half, 5);
  } else {
    // what the cells of the top block's last position saw: the initial gradient
    if (role == kChain)
      reinterpret_cast<float *>(&lds.g[lane][((top + 1) % 3) * kQuadsPerBlock])[0] = G;
    if (role == kLoader) {
      load_block(top, sets[0]);
      wait_all(sets[0]);
      commit_block(top, sets[0]);
#pragma unroll
      for (int i = 0; i < kSets; ++i) load_block(top - 1 - i, sets[i]);
    } else if (role == kEdge) {
      take_block(top);
    }
    LdsBarrier();
  }

  // Descending twin of the forward's loops: in iteration kb the chain computes block kb, the
  // loaders commit block kb-1 and start the loads of block kb-3, the storers drain block kb+1,
  // the edge wavefront publishes block kb+1 upwards and takes block kb-1 from the chunk below.
  if (role == kChain) {
    for (int kb = top; kb >= 0; --kb) {
      chain_block(kb);
      LdsBarrier();
    }
  } else if (role == kLoader) {
    for (int kb = top; kb >= 0; kb -= kSets) {
#pragma unroll
      for (int i = 0; i < kSets; ++i) {
        if (kb - i < 0) break;
        wait_older(sets[i]);
        commit_block(kb - i - 1, sets[i]);
        load_block(kb - i - 1 - kSets, sets[i]);
        LdsBarrier();
      }
    }
    // the loads of the blocks in front of the first one are still in flight: they must land
    // before the compiler may give their registers to anything else
#pragma unroll
    for (int i = 0; i < kSets; ++i) wait_all(sets[i]);
  } else if (role == kStorer) {
    storer_bases();
    for (int kb = top; kb >= 0; --kb) {
      store_block(kb + 1);
      LdsBarrier();
    }
    store_block(0);
  } else if (role == kEdge) {
    for (int kb = top; kb >= 0; --kb) {
      publish_block(kb + 1);
      take_block(kb - 1);
      LdsBarrier();
    }
  }
  K2AMD_TRACE_MARK(half, 6);
  if (kBidir && threadIdx.x == 0) {
    sh_of(join)->departed = departed_early;
    sh_of(join)->departed_set = 1;
  }
  if (role == kEdge) publish_block(0);
  if (overwrite_ans_grad && ans_grad != nullptr && role == kChain && g.c == 0 && lane == 0 && !mirror)
    ans_grad[g.b] = GaveUp(hdr) ? __builtin_nanf("") : g_origin;
}

// The first B * nchunks tickets sweep, lower chunks first; the rest of the grid (as many again)
// clears what the sweep does not assign, one workgroup per (sequence, 64 array rows), on compute
// units the sweep leaves idle and off its critical path.
template <bool kKept>
__global__ __launch_bounds__(BwdLayout::kThreads) void MiBackwardFastKernel(
    const float *__restrict__ px, const float *__restrict__ p,
    const int64_t *__restrict__ boundary, float *__restrict__ ans_grad,
    float *__restrict__ px_grad, float *__restrict__ py_grad, FastHeader *hdr, float *edge, int B,
    int S, int Tn, int modified, int nchunks, int edge_stride, int overwrite_ans_grad) {
  __shared__ BwdLds lds;
  if (threadIdx.x == 0) lds.ticket = atomicAdd(&hdr->ticket, 1u);
  __syncthreads();
  const unsigned ticket = lds.ticket, nsweep = (unsigned)B * nchunks;
  const bool zero_only = ticket >= nsweep;
  const unsigned unit = zero_only ? ticket - nsweep : ticket;
  MiBackwardChunk<kKept, false>(lds, px, p, LoadBox(boundary, (int)(unit / nchunks), S, Tn), ans_grad,
                                px_grad, py_grad, hdr, edge, B, S,
                                Tn, modified, nchunks, edge_stride, overwrite_ans_grad,
                                (int)(unit / nchunks),
                                zero_only ? (int)(unit % nchunks) : nchunks - 1 - (int)(unit % nchunks),
                                zero_only, Half{}, nullptr);
  if (threadIdx.x == 0) PutTicketsBack(hdr, lds.ticket, gridDim.x);
}

// ------------------------------------------------------------------------------ single launch
//
// Forward and backward of every sequence in ONE launch, for callers that want ans and the
// gradients together (the reference's autograd function, k2/python/k2/mutual_information.py:
// 157-169).  Every lattice is split at a cut diagonal half way along its longest path (see Half)
// and swept from both ends at once:
//   1. the first half forward from the origin (alpha), the second half "forward" in its mirrored
//      coordinates from the end cell (beta), each keeping its px-edge log-derivatives;
//   2. on the cut, where every path has exactly one cell, alpha + beta of a cell is the log of
//      the total weight of the paths through it: the score is their log-sum, and a cell's share
//      of the paths, exp(alpha + beta - score), is the gradient that reaches it;
//   3. each half sweeps back from the cut with the ordinary backward chunk sweep, seeded with
//      those shares on every row instead of with the sequence's gradient at the end cell.  In the
//      mirrored half a cell's log-derivative is the log-probability of LEAVING the lattice cell
//      along px given that a path is there, which is what the occupation counts need on that
//      side: the same code yields px_grad / py_grad of the edges that leave each cell.
// So the longest chain of dependent steps is half the lattice's, both ways.
//
// Work is handed out as TASKS through the ticket counter to a fixed set of persistent workgroups
// (one per compute unit): first the forward sweeps of all (sequence, half, 64-row chunk), then the
// backward sweeps, then the clearing of what lies outside the boxes, then one task per sequence
// for the lattices the split cannot serve.  A task only ever waits for tasks with EARLIER
// tickets (a chunk's producer; for the backward sweeps and the last kind of task, all forward
// sweeps of the sequence), and a ticket is only taken by a workgroup that is running, so the
// launch makes progress with any number of resident workgroups: nothing depends on the whole grid
// being resident at once.
//
// A lattice whose end cell no path reaches has no finite score to normalise with; its gradients
// are then DEFINED by the reference's loop order (k2/python/csrc/torch/
// mutual_information_cpu.cu:195-211).  Such a sequence is left to its last task, which runs the
// exact one-workgroup recursion of mi_generic_impl.h on it.
union FusedLds {
  FwdLds fwd;
  BwdLds bwd;
};

// What every task of the single launch needs (the kernel's arguments).
struct BidirArgs {
  const float *px, *py;
  const int64_t *boundary;
  float *ans, *scratch, *ans_grad, *px_grad, *py_grad;
  FastHeader *hdr;
  float *edge0, *edge1, *cut;
  int B, S, Tn, modified, nchunks, edge_stride, overwrite_ans_grad;
#ifdef K2AMD_MI_TRACE
  unsigned long long *trace;  // per ticket: start, cut reached, end (100 MHz clock), compute unit
#endif
};

// The tasks are functions of their own (not inlined into the kernel's loop), so that each gets the
// registers IT needs: the sweeps' loaders keep several blocks of loads in flight in registers and
// count them by hand, which a spill in their loops would upset.  What they need of the kernel's
// arguments and of the sequence's box they read from LDS (a copy made once per workgroup, once per
// task): a reference into any other memory would cost a trip there at the start of every task.
struct TaskShared {
  BidirArgs k;
  Box box;
};
__device__ __attribute__((noinline)) void BidirForwardTask(FwdLds &lds, const TaskShared &t, int seq,
                                                           int chunk, Half half, float *cut_out,
                                                           float *cut_frame_out, float *gauge_out) {
  const BidirArgs &k = t.k;
  MiForwardChunk<true, false, true>(lds, k.px, k.py, t.box, nullptr, k.ans, k.scratch, k.hdr,
                                    half.mirror ? k.edge1 : k.edge0, k.B, k.S, k.Tn, k.modified,
                                    k.nchunks, k.edge_stride, seq, chunk, half, cut_out, cut_frame_out,
                                    gauge_out);
}
// (what the join needs comes as arguments of its own: a structure handed over by address would
// live in scratch memory, a trip there for every field the sweep reads)
__device__ __attribute__((noinline)) void BidirBackwardTask(BwdLds &lds, const TaskShared &t, int seq,
                                                            int chunk, Half half, CutShared *sh,
                                                            float *ans_out) {
  const BidirArgs &k = t.k;
  const BidirJoin join_words{sh, CutOf(k.cut, seq, k.nchunks), ans_out};
  const BidirJoin *join = &join_words;  // (never leaves this function: stays in registers)
  MiBackwardChunk<true, true>(lds, k.px, k.scratch, t.box, k.ans_grad, k.px_grad, k.py_grad, k.hdr,
                              half.mirror ? k.edge1 : k.edge0, k.B, k.S, k.Tn, k.modified, k.nchunks,
                              k.edge_stride, k.overwrite_ans_grad, seq, chunk, false, half, join);
}
__device__ __attribute__((noinline)) void BidirClearTask(BwdLds &lds, const TaskShared &t, int seq, int chunk) {
  const BidirArgs &k = t.k;
  MiBackwardChunk<true, false>(lds, k.px, k.scratch, t.box, k.ans_grad, k.px_grad, k.py_grad, k.hdr,
                               k.edge0, k.B, k.S, k.Tn, k.modified, k.nchunks, k.edge_stride,
                               k.overwrite_ans_grad, seq, chunk, true, Half{}, nullptr);
}
// No path reaches the end cell: the exact recursion, whose loop order defines the result.
__device__ __attribute__((noinline)) void BidirExactTask(CutShared &sh, const TaskShared &t, int seq,
                                                         float seed) {
  const BidirArgs &k = t.k;
  const Box box = t.box;
  float *prev = sh.a, *cur = sh.a + (k.S + 2);
  // p goes where the sequence's blocks would have gone: the sequence's part of the slab is at
  // least (S + 1) rows of Tn + 2 (the exact recursion adds seq * (S + 1) * (Tn + 2) itself)
  float *p_seq = k.scratch + (size_t)seq * (SlabFloatsPerSequence(k.S, k.Tn, k.modified) -
                                            (size_t)(k.S + 1) * (k.Tn + 2));
  static_assert(offsetof(CutShared, b) == sizeof(float) * kCutRows, "a and b are one array here");
  const float end = MiForwardGenericSeq<float>(k.px, k.py, box, p_seq, seq, k.S, k.Tn, k.modified,
                                               k.Tn + 2, prev, cur);
  if (threadIdx.x == 0) k.ans[seq] = GaveUp(k.hdr) ? __builtin_nanf("") : end;
  __syncthreads();
  const float at_origin = MiBackwardGenericSeq<float>(k.px, p_seq, box, seed, k.px_grad, k.py_grad,
                                                      seq, k.S, k.Tn, k.modified, k.Tn + 2, prev, cur);
  if (k.overwrite_ans_grad && k.ans_grad != nullptr && threadIdx.x == 0) k.ans_grad[seq] = at_origin;
}

__global__ __launch_bounds__(FwdLayout::kThreads) void MiBidirKernel(const BidirArgs k) {
  static_assert(FwdLayout::kThreads == BwdLayout::kThreads, "one workgroup shape for both sweeps");
  __shared__ FusedLds lds;
  __shared__ CutShared sh;
  __shared__ TaskShared ts;
  // The boxes of the first sequences, read once per workgroup while its first ticket is on its
  // way: a task then starts without a trip to memory for its box.
  constexpr int kBoxes = 256;
  __shared__ Box boxes[kBoxes];
  if (threadIdx.x == 0) {
    ts.k = k;
    sh.ticket = __hip_atomic_fetch_add(Global(&k.hdr->ticket), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  for (int i = (int)threadIdx.x - kWave; i >= 0 && i < min(k.B, kBoxes); i += blockDim.x - kWave)
    boxes[i] = LoadBox(k.boundary, i, k.S, k.Tn);
  auto box_of = [&](int seq) { return seq < kBoxes ? boxes[seq] : LoadBox(k.boundary, seq, k.S, k.Tn); };
  const int nchunks = k.nchunks;
  const unsigned per_seq = 2u * nchunks, nsweep = (unsigned)k.B * per_seq;
  // Tickets: the forward half-sweeps, the backward half-sweeps, the clearing of what lies outside
  // the boxes, one last task per sequence.  (The clearing writes a fifth as many bytes as the
  // sweeps move, and placed between the two kinds of sweeps, where workgroups whose forward
  // sweeps end early are free for it, it slowed the long sequences' forward sweeps down while
  // their inputs come from HBM: 56.5 us per launch against 54.1 with the clearing behind the
  // backward sweeps, drawn by workgroups whose backward sweeps end early.)
  const unsigned first_bwd = nsweep, first_clear = first_bwd + nsweep;
  const unsigned first_last = first_clear + (unsigned)k.B * nchunks, ntasks = first_last + (unsigned)k.B;
  const int skew = k.modified ? 0 : 1;
  for (bool first = true;; first = false) {
    if (!first) {
      __syncthreads();  // the previous task's last LDS reads are done, its stores complete
      if (threadIdx.x == 0) sh.ticket = __hip_atomic_fetch_add(Global(&k.hdr->ticket), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const unsigned ticket = sh.ticket;
    if (ticket >= ntasks) break;
#ifdef K2AMD_MI_TRACE
    struct Tracer {
      unsigned long long *at;
      __device__ void mark(int i) { if (at != nullptr && threadIdx.x == 0) at[i] = wall_clock64(); }
      __device__ ~Tracer() { mark(2); }
    } tracer{k.trace != nullptr ? k.trace + 32 * (size_t)ticket : nullptr};
    tracer.mark(0);
#endif

    if (ticket >= first_clear && ticket < first_last) {  // what no sweep assigns
      const unsigned unit = ticket - first_clear;
      if (threadIdx.x == 0) ts.box = box_of((int)(unit / nchunks));
      __syncthreads();
      BidirClearTask(lds.bwd, ts, (int)(unit / nchunks), (int)(unit % nchunks));
      continue;
    }

    const bool fwd = ticket < first_bwd, last = ticket >= first_last;
    const unsigned unit = fwd ? ticket : (last ? 0u : ticket - first_bwd);
    const int seq = last ? (int)(ticket - first_last) : (int)(unit / per_seq);
    const int mirror = last ? 0 : (int)((unit % per_seq) / nchunks);
    const int cidx = last ? 0 : (int)(unit % nchunks);
    const int chunk = fwd || last ? cidx : nchunks - 1 - cidx;  // backward: lower chunks first
    if (threadIdx.x == 0) ts.box = box_of(seq);
    __syncthreads();
    const Box box = ts.box;
    const int ns = box.s1 - box.s0, nt = box.t1 - box.t0;
    const int diagonals = nt + ns * skew, dcut = diagonals / 2;
    Half half{};
    half.mirror = mirror;
    half.dmax = mirror ? diagonals - dcut : dcut;
#ifdef K2AMD_MI_TRACE
    half.trace = k.trace != nullptr ? k.trace + 32 * (size_t)ticket : nullptr;
#endif
    const CutWords cw = CutOf(k.cut, seq, nchunks);

    if (fwd) {
      if (!mirror && chunk == 0 && threadIdx.x == 0)
        PublishCut(cw.scale, k.ans_grad != nullptr ? k.ans_grad[seq] : 1.0f);
      BidirForwardTask(lds.fwd, ts, seq, chunk, half, (mirror ? cw.beta : cw.alpha) + chunk * kRows,
                       (mirror ? cw.frame_beta : cw.frame_alpha) + chunk,
                       !mirror && chunk == 0 ? cw.gauge : nullptr);
      // every wavefront has waited for its stores (device-coherent ones, see StoreQuadCoherent)
      // before this barrier: whichever compute unit sweeps this chunk back will see them
      __syncthreads();
      if (threadIdx.x == 0)
        __hip_atomic_fetch_add(Global(cw.stored), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      continue;
    }

    // Backward sweep of a chunk, or the sequence's last task: both start from the cut, whose
    // words they wait for themselves.
    if (threadIdx.x == 0) sh.departed_set = 0;
    if (!last) {
      if (threadIdx.x == 0 && !mirror && chunk == 0 && !box.ok) k.ans[seq] = __builtin_nanf("");
      if (box.ok)
        BidirBackwardTask(lds.bwd, ts, seq, chunk, half, &sh, !mirror && chunk == 0 ? k.ans + seq : nullptr);
    } else {
      // The sequence's last task: the exact recursion where the halves could not be joined (no
      // path reaches the end cell), once no forward sweep has a store on its way into the slab.
      // It waits for the forward sweeps' stores in any case: they include the words of the cut,
      // which the last task to leave the sequence resets, and this task is among those.
      if (threadIdx.x < kWave) {
        float seed, scale = 0.0f;
        const float total = box.ok ? WaveCutJoin(sh, cw, ns, k.modified ? nt - ns : nt, 0, 0, k.hdr, &seed, &scale) : 0.0f;
        if (threadIdx.x == 0) {
          sh.total = total;
          sh.scale = scale;
          WaitCount(cw.stored, kSentinel + per_seq, k.hdr);
        }
      }
      __syncthreads();
      const float seed = sh.scale;
      if (box.ok && !(sh.total > kLogZeroTest)) BidirExactTask(sh, ts, seq, seed);
    }
    // This task is through with the sequence's cut words (where it read them at all).  The last
    // task to say so puts them back into their initial state.
    __syncthreads();
    if (threadIdx.x == 0) {
      const unsigned before = sh.departed_set
                                  ? sh.departed
                                  : __hip_atomic_fetch_add(Global(cw.depart), 1u, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT);
      sh.last = before == kSentinel + per_seq;
    }
    __syncthreads();
    if (sh.last)
      for (int i = threadIdx.x; i < cw.words; i += blockDim.x)
        __hip_atomic_store(Global(reinterpret_cast<unsigned *>(cw.depart) - 1 + i), kSentinel, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
  }
  // (every workgroup draws exactly one ticket past the tasks)
  if (threadIdx.x == 0) PutTicketsBack(k.hdr, sh.ticket, ntasks + gridDim.x);
}

// A sweeping workgroup wants a compute unit to itself (its chain wavefront sets the pace of the
// whole sequence, and a second workgroup on the unit would share its LDS pipe and issue slots).
// Asking for more than half of the unit's 160 KB of LDS makes the dispatcher place one workgroup
// per unit; the bytes beyond the kernels' own structures are never touched.
constexpr size_t kExclusiveLds = 84 * 1024;
static_assert(sizeof(FwdLds) + 16 < kExclusiveLds && sizeof(BwdLds) + 16 < kExclusiveLds, "LDS budget");
// the single launch's own structures already are more than half a unit's LDS
static_assert(sizeof(FusedLds) + sizeof(CutShared) > 80 * 1024 && sizeof(FusedLds) + sizeof(CutShared) < 160 * 1024,
              "one workgroup of the single launch per compute unit");

}  // namespace

// The throughput kernels address each tensor through a buffer resource with 32-bit byte offsets:
// tensors of 2 GiB and more take the exact path.
bool MiFastSupports(int B, int S, int Tn, int modified) {
  (void)modified;
  return S >= 1 && Tn >= 1 && (long long)B * (S + 1) * (Tn + 1) < (1ll << 29);
}

// Two sets of edge rows (the single launch sweeps the two halves of every lattice at once), then
// the words of the cut of every sequence.
size_t MiFastWorkspaceBytes(int B, int S, int Tn) {
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const size_t edge_stride = EdgeStride(Tn);
  const size_t cut_words = CutWordsPerSequence(nchunks);
  return sizeof(FastHeader) + (2 * (size_t)B * (nchunks + 1) * edge_stride + (size_t)B * cut_words) * sizeof(float);
}

int MiFastWorkspaceInit(void *workspace, size_t workspace_bytes, hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < sizeof(FastHeader)) return K2AMD_ERR_WORKSPACE;
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  const size_t n_edge = (workspace_bytes - sizeof(FastHeader)) / sizeof(float);
  hipLaunchKernelGGL(FastWsInitKernel, dim3((unsigned)min((size_t)256, (n_edge + 255) / 256 + 1)),
                     dim3(256), 0, stream, hdr, reinterpret_cast<unsigned *>(hdr + 1), n_edge);
  return LaunchStatus();
}

// Compute units of the current device (asked once per device ordinal), or -1.
static int ComputeUnits() {
  static std::atomic<int> units[64];  // 0 = not asked yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
  int n = units[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
    n = n > 0 ? n : -1;
    units[dev].store(n, std::memory_order_relaxed);  // every thread would store the same value
  }
  return n;
}

// LDS bytes to ask for beyond a kernel's own structure.  While the sweeping workgroups of a launch
// find a compute unit each, every one gets a unit to itself (kExclusiveLds); once there are more
// chunks than units the launch is bound by how many chains the device steps at a time, and two
// workgroups share a unit (K2AMD_MI_SHARE_UNITS=0 in the environment, read once, keeps one to a
// unit: for comparisons).
static size_t LdsPad(size_t own, long long sweepers) {
  static const bool never_share = [] {
    const char *e = getenv("K2AMD_MI_SHARE_UNITS");
    return e != nullptr && e[0] == '0';
  }();
  const int n = ComputeUnits();
  if (!never_share && n > 0 && sweepers > n) return 0;
  return kExclusiveLds - own;
}

int MiForwardFast(const float *px, const float *py, const int64_t *boundary, float *p, float *ans,
                  float *log_deriv, int B, int S, int Tn, int modified, void *workspace,
                  size_t workspace_bytes, hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiFastWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const int edge_stride = EdgeStride(Tn);
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  float *edge = reinterpret_cast<float *>(hdr + 1);
  const dim3 grid((unsigned)(B * nchunks)), block(FwdLayout::kThreads);
  const size_t pad = LdsPad(sizeof(FwdLds), (long long)B * nchunks);
  if (log_deriv == nullptr && p == nullptr) return K2AMD_ERR_INVALID_ARGUMENT;
  if (log_deriv != nullptr && p != nullptr)
    hipLaunchKernelGGL((MiForwardFastKernel<true, true>), grid, block, pad, stream, px, py, boundary, p, ans, log_deriv, hdr, edge, B, S, Tn, modified, nchunks, edge_stride);
  else if (log_deriv != nullptr)
    hipLaunchKernelGGL((MiForwardFastKernel<true, false>), grid, block, pad, stream, px, py, boundary, p, ans, log_deriv, hdr, edge, B, S, Tn, modified, nchunks, edge_stride);
  else
    hipLaunchKernelGGL((MiForwardFastKernel<false, true>), grid, block, pad, stream, px, py, boundary, p, ans, log_deriv, hdr, edge, B, S, Tn, modified, nchunks, edge_stride);
  return LaunchStatus();
}

int MiBackwardFast(const float *px, const float *p, const float *log_deriv,
                   const int64_t *boundary, float *ans_grad, float *px_grad, float *py_grad, int B,
                   int S, int Tn, int modified,
                   int overwrite_ans_grad, void *workspace, size_t workspace_bytes,
                   hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiFastWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const int edge_stride = EdgeStride(Tn);
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  float *edge = reinterpret_cast<float *>(hdr + 1);
  // B * nchunks sweeping workgroups + as many that only clear
  const dim3 grid((unsigned)(2 * B * nchunks)), block(BwdLayout::kThreads);
  const size_t pad = LdsPad(sizeof(BwdLds), (long long)B * nchunks);
  if (log_deriv != nullptr)
    hipLaunchKernelGGL(MiBackwardFastKernel<true>, grid, block, pad, stream, px, log_deriv, boundary, ans_grad, px_grad, py_grad, hdr, edge, B, S, Tn, modified, nchunks, edge_stride, overwrite_ans_grad);
  else
    hipLaunchKernelGGL(MiBackwardFastKernel<false>, grid, block, pad, stream, px, p, boundary, ans_grad, px_grad, py_grad, hdr, edge, B, S, Tn, modified, nchunks, edge_stride, overwrite_ans_grad);
  return LaunchStatus();
}

// The single launch serves what the pipelined kernels serve, up to the number of lattice rows that
// its join on the cut keeps in LDS.  It needs no particular number of resident workgroups.
bool MiFusedSupports(int B, int S, int Tn, int modified) {
  return MiFastSupports(B, S, Tn, modified) && B >= 1 && S + 2 <= kCutRows;
}

// Whether the single launch is the faster way to run both recursions of this shape on the current
// device.  It is, by far, while every forward half-sweep finds a compute unit at once (the launch
// then lasts as long as one sequence's two half-length fronts: B = 32, S = 200, T = 1000 takes 58 us
// against 79 for the pair), and still by a few per cent with up to two half-sweeps per unit.  With
// more of them they queue, one workgroup to a unit, where the pair places two: the pair then wins
// on short lattices (B = 512, S = 100, T = 500: 199 us against 225; T = 700: 474 against 493) and
// the single launch on long ones (B = 512 and 1024, S = 200, T = 1000: 625 against 645 us, 1263
// against 1278).
bool MiFusedAdvised(int B, int S, int Tn) {
  const int units = ComputeUnits();
  const long long nchunks = (S + 1 + kRows - 1) / kRows;
  return units > 0 && (2ll * B * nchunks <= 2ll * units || Tn >= 1000);
}

// Floats of scratch per call of the single launch: the log-derivatives of both halves of every
// sequence, in blocks (SlabBlocks).
size_t MiFusedScratchElems(int B, int S, int Tn, int modified) {
  return (size_t)B * SlabFloatsPerSequence(S, Tn, modified);
}

int MiForwardBackwardFast(const float *px, const float *py, const int64_t *boundary, float *ans,
                          float *scratch, float *ans_grad, float *px_grad, float *py_grad, int B,
                          int S, int Tn, int modified, int overwrite_ans_grad, void *workspace,
                          size_t workspace_bytes, hipStream_t stream) {
  if (workspace == nullptr || workspace_bytes < MiFastWorkspaceBytes(B, S, Tn)) return K2AMD_ERR_WORKSPACE;
  if (scratch == nullptr) return K2AMD_ERR_INVALID_ARGUMENT;
  if (!MiFusedSupports(B, S, Tn, modified)) return K2AMD_ERR_UNSUPPORTED;
  const int units = ComputeUnits();
  if (units <= 0) return K2AMD_ERR_LAUNCH;
  const int nchunks = (S + 1 + kRows - 1) / kRows;
  const int edge_stride = EdgeStride(Tn);
  FastHeader *hdr = static_cast<FastHeader *>(workspace);
  float *edge0 = reinterpret_cast<float *>(hdr + 1);
  float *edge1 = edge0 + (size_t)B * (nchunks + 1) * edge_stride;
  float *cut = edge1 + (size_t)B * (nchunks + 1) * edge_stride;
  // forward sweeps of both halves, clearing, backward sweeps, one last task per sequence
  const long long ntasks = 5ll * B * nchunks + B;
  const dim3 grid((unsigned)std::min<long long>(ntasks, units)), block(FwdLayout::kThreads);
  BidirArgs args{px, py, boundary, ans, scratch, ans_grad, px_grad, py_grad, hdr, edge0, edge1, cut,
                 B, S, Tn, modified, nchunks, edge_stride, overwrite_ans_grad};
#ifdef K2AMD_MI_TRACE
  const char *trace_at = getenv("K2AMD_MI_TRACE_PTR");
  args.trace = trace_at != nullptr ? reinterpret_cast<unsigned long long *>(strtoull(trace_at, nullptr, 0)) : nullptr;
#endif
  hipLaunchKernelGGL(MiBidirKernel, grid, block, 0, stream, args);
  return LaunchStatus();
}

}  // namespace k2amd
