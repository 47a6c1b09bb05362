// The pruned joiner fused with the log-prob builder that consumes its output:
//
//   logits[b,t,k,:] = tanh(am[b,t,:] + lm[b, ranges[b,t,k], :]) . weight^T + bias
//   px, py          = get_rnnt_logprobs_pruned(logits, ...)
//
// i.e. do_rnnt_pruning (k2/python/k2/rnnt_loss.py:913-954), the joiner the reference leaves to the
// caller between it and rnnt_loss_pruned, and get_rnnt_logprobs_pruned (rnnt_loss.py:1180-1348).
// The [B][T][R][C] logits only ever exist as tiles in registers: the forward multiplies a tile of
// rows by the weight on the matrix cores, folds each tile of columns into a running log-sum-exp and
// picks out the two logits a row contributes; the backward multiplies again and forms
// d logits = -softmax (gx + gy) + gx [c == symbol] + gy [c == blank] on the fly, tile of rows by
// tile of rows, for the gradients of am and lm, and leaves the activations and d logits in the
// caller's workspace (in the operand type and in the order a product over the rows consumes them)
// for a second kernel that forms the gradients of the weight and the bias.
//
// One row of the product is (b, t, k); a tile holds whole frames (b, t), R rows each, so the sum
// over k that am's gradient needs stays inside a tile.  Operands: `F32` multiplies fp32 by fp32
// (v_mfma_f32_32x32x2_f32: the products and sums of an fp32 matrix multiply), `Bf16` rounds
// tanh(..), the weight and d logits to bfloat16 and multiplies with v_mfma_f32_32x32x16_bf16; both
// accumulate in fp32, and everything outside the products is fp32.
//
// Data movement: the activations tanh(..) of a tile are formed once and kept in LDS ([row][k], k
// contiguous, rows 16 bytes apart modulo 256 so that 16-byte reads of 32 rows miss each other's
// banks); the weight is read from copies prepared per call in the operand type, padded with zeros
// to whole tiles and stored in the order the multiplies consume them (BOperand), once with k = D
// (for logits) and once with k = C (for d logits . weight); they stay in L2.  A lane's share of an
// operand per step of k is 64 bytes (16 floats or 32 bfloat16): four 16-byte loads.  Which k a lane
// feeds to which multiply is the same for both operands, which is all the instruction needs.
// Workgroups are eight wavefronts, two per SIMD.
#include <cstdlib>

#include "common.h"

namespace k2amd {
namespace {

typedef float Acc16 __attribute__((ext_vector_type(16)));
typedef __bf16 Bf8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 512;   // eight wavefronts: two per SIMD, one computes while the other waits
constexpr int kWaves = kThreads / 64;
constexpr int kNTile = 256;     // columns of a product per pass: 32 per wavefront
constexpr int kMaxD = 512;      // joiner dimension the LDS tiles are sized for
constexpr int kStageCols = 128; // columns of d pre-activation reduced at a time

struct Frag {
  uint4 q[4];
};

__device__ __forceinline__ float AsFloat(unsigned u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ unsigned AsBits(float f) { return __builtin_bit_cast(unsigned, f); }

// float -> bfloat16, round to nearest even (the hardware's conversion)
__device__ __forceinline__ unsigned short ToBf16(float f) {
  return __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
}
__device__ __forceinline__ float FromBf16(unsigned short h) { return AsFloat((unsigned)h << 16); }

// tanh(x) = 1 - 2 / (1 + exp(2 x)): five instructions (the exponential saturates to 0 or inf at
// the ends, which gives -1 and 1); absolute error ~1e-7, which is what the logits (sums of D such
// values times weights) are sensitive to.
__device__ __forceinline__ float Tanh(float x) {
  const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);  // exp(2 x)
  return fmaf(-2.0f, __builtin_amdgcn_rcpf(1.0f + e), 1.0f);
}

struct F32 {
  typedef float Elem;
  static constexpr int kChunk = 32;  // k per step
  static constexpr int kAhead = 1;   // a step is 16 multiplies per block of rows: one step hides a trip to L2
  static constexpr int kPad = 4;     // elements: rows 16 bytes apart modulo 256 (LDS banks)
  static __device__ __forceinline__ Elem From(float f) { return f; }
  static __device__ __forceinline__ float To(Elem e) { return e; }
  static __device__ __forceinline__ void Mma(Acc16 &acc, const Frag &a, const Frag &b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(AsFloat(a.q[i].x), AsFloat(b.q[i].x), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(AsFloat(a.q[i].y), AsFloat(b.q[i].y), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(AsFloat(a.q[i].z), AsFloat(b.q[i].z), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(AsFloat(a.q[i].w), AsFloat(b.q[i].w), acc, 0, 0, 0);
    }
  }
  static __device__ __forceinline__ void Store4(Elem *dst, float4 v) {
    *reinterpret_cast<float4 *>(dst) = v;
  }
};

struct Bf16 {
  typedef unsigned short Elem;
  static constexpr int kChunk = 64;
  static constexpr int kAhead = 1;
  static constexpr int kPad = 8;
  static __device__ __forceinline__ Elem From(float f) { return ToBf16(f); }
  static __device__ __forceinline__ float To(Elem e) { return FromBf16(e); }
  static __device__ __forceinline__ void Mma(Acc16 &acc, const Frag &a, const Frag &b) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(Bf8, a.q[i]),
                                                    __builtin_bit_cast(Bf8, b.q[i]), acc, 0, 0, 0);
  }
  static __device__ __forceinline__ void Store4(Elem *dst, float4 v) {
    uint2 p;
    p.x = (unsigned)ToBf16(v.x) | ((unsigned)ToBf16(v.y) << 16);
    p.y = (unsigned)ToBf16(v.z) | ((unsigned)ToBf16(v.w) << 16);
    *reinterpret_cast<uint2 *>(dst) = p;
  }
};

// 64 bytes of an operand row (16-byte aligned by construction of every caller)
template <typename Elem>
__device__ __forceinline__ Frag LoadFrag(const Elem *p) {
  const uint4 *v = reinterpret_cast<const uint4 *>(p);
  Frag f;
#pragma unroll
  for (int i = 0; i < 4; ++i) f.q[i] = v[i];
  return f;
}

// The weight copies are stored in the order the multiplies consume them: for each block of 32 rows n
// and each step of k, four groups of 64 x 16 bytes, group i holding for lane l the 16 bytes at
// k = step * kChunk + (l >> 5) * kChunk / 2 + i * (16 / sizeof(Elem)) of row n = block * 32 + (l & 31):
// one load instruction of a wavefront then reads 1 KB of consecutive memory.
constexpr int kFragQuads = 4 * 64;  // 16-byte groups per (block of rows, step of k)
// `block` is the same for all lanes (a scalar register), so the loads take the form scalar base +
// lane offset + immediate and need no per-load address registers.
__device__ __forceinline__ Frag LoadFragB(const uint4 *block, int lane) {
  Frag f;
#pragma unroll
  for (int i = 0; i < 4; ++i) f.q[i] = block[i * 64 + lane];
  return f;
}
// groups of block `nb`, step `step0`, in a copy with `ksteps` steps per block (all arguments the
// same for all lanes)
__device__ __forceinline__ const uint4 *BOperand(const void *w, int nb, int ksteps, int step0) {
  return static_cast<const uint4 *>(w) + ((size_t)nb * ksteps + step0) * kFragQuads;
}

struct JoinerArgs {
  const float *am, *lm, *bias;  // bias may be null
  const int64_t *ranges, *symbols, *boundary;
  const void *wk;   // weight copy, rows c (Cpad), k = d: see BOperand
  const void *wc;   // weight copy, rows d (Dpad), k = c (Cpad)
  float *px, *py, *norm;        // forward outputs (norm [B][T][R])
  const float4 *hdr;            // backward: per row {gx, gy, symbol, norm}
  // backward, written by the rows kernel for the weight kernel after it, both as operands of a
  // product over k = row (see BOperand; a step of k is one tile of rows): tanh(..) with rows d,
  // d logits with rows c; and the sums of d logits over each tile's rows, [tile][Cpad]
  void *hs, *dzs;
  float *bias_part;
  int tiles;                    // tiles of rows in the pass at hand: the steps of k of its operands
  int tile0;                    // the pass's first tile (the backward goes through the rows in passes
                                // that fit the workspace)
  float *am_grad, *lm_grad, *weight_grad, *bias_grad;
  int B, S, Tn, R, C, D, blank, rnnt_type;
  int Cpad, Dpad;               // C, D rounded up to whole tiles of kNTile
  int tpt;                      // frames per tile of rows
  long long frames;             // B * Tn
};

struct RowMeta {
  int bt;     // frame b * Tn + t
  int lmrow;  // b * (S + 1) + ranges[b,t,k] (clamped into the sequence's rows)
  int s;      // lattice row (ranges[b,t,0] + k) mod (S + 1)
  int sym;    // symbol whose logit goes to px, or -1
};

// Where row (b, t, k) takes its lm vector from, where it lands in the lattice and which symbol it
// scores (k2/python/k2/rnnt_loss.py:1282-1316).
__device__ __forceinline__ RowMeta MetaOf(const JoinerArgs &a, long long frame, int k) {
  RowMeta m;
  const int b = (int)(frame / a.Tn);
  const int64_t *r = a.ranges + (size_t)frame * a.R;
  const int64_t shift = r[0], src = r[k];
  const int S1 = a.S + 1;
  int ss = (int)((k + shift) % S1);
  if (ss < 0) ss += S1;
  m.bt = (int)frame;
  m.s = ss;
  const int64_t clamped = src < 0 ? 0 : (src > a.S ? a.S : src);
  m.lmrow = b * S1 + (int)clamped;
  if (src >= 0 && src < a.S) m.sym = (int)a.symbols[(size_t)b * a.S + src];
  else if (src == a.S) m.sym = a.blank;
  else m.sym = -1;
  if (m.sym < 0 || m.sym >= a.C) m.sym = -1;
  return m;
}

// The rows of a tile: frames f0 .. f0 + nf - 1, row = (frame - f0) * R + k.
template <int MT>
__device__ __forceinline__ int LoadMeta(const JoinerArgs &a, long long f0, RowMeta *meta) {
  const long long left = a.frames - f0;
  const int nf = (int)(left < a.tpt ? left : a.tpt);
  const int rows = nf * a.R;
  for (int m = threadIdx.x; m < MT; m += kThreads) {
    if (m < rows) {
      meta[m] = MetaOf(a, f0 + m / a.R, m % a.R);
    } else {
      RowMeta z; z.bt = 0; z.lmrow = 0; z.s = 0; z.sym = -1;
      meta[m] = z;
    }
  }
  return rows;
}

// h[m][:] = tanh(am[frame] + lm[lmrow]) for the tile's rows (zeros beyond them), in the operand
// type; kTransposed also keeps a copy ht[d][m] (k = row contiguous, for the weight gradient).
template <typename Mode, int MT, bool kTransposed, int kBatch, int kD>
__device__ __forceinline__ void StageActivations(const JoinerArgs &a, const RowMeta *meta, int rows,
                                                 typename Mode::Elem *h, int ldh,
                                                 typename Mode::Elem *ht, int ldt) {
  // A thread's items in batches of kBatch: all loads of a batch are asked for before the first is
  // used (one trip to memory per batch instead of one per item; the batch is sized to the registers
  // the caller has left).
  // (kD > 0: the joiner dimension is known when compiling, and the divisions below are shifts)
  const int dim = kD > 0 ? kD : a.D;
  const int qpr = dim >> 2, items = MT * qpr;
  for (int base = threadIdx.x; base < items; base += kThreads * kBatch) {
    float4 x[kBatch], y[kBatch];
    int at[kBatch];  // m * qpr + q, or -1 beyond the tile's items
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int idx = base + j * kThreads;
      at[j] = idx < items ? idx : -1;
      x[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      y[j] = x[j];
      if (idx < items) {
        const int m = idx / qpr, q = idx - m * qpr;
        if (m < rows) {
          const RowMeta rm = meta[m];
          x[j] = *reinterpret_cast<const float4 *>(a.am + (size_t)rm.bt * dim + 4 * q);
          y[j] = *reinterpret_cast<const float4 *>(a.lm + (size_t)rm.lmrow * dim + 4 * q);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      if (at[j] < 0) continue;
      const int m = at[j] / qpr, q = at[j] - m * qpr;
      // rows beyond the tile's: tanh(0 + 0) = 0
      const float4 v = make_float4(Tanh(x[j].x + y[j].x), Tanh(x[j].y + y[j].y), Tanh(x[j].z + y[j].z),
                                   Tanh(x[j].w + y[j].w));
      Mode::Store4(h + (size_t)m * ldh + 4 * q, v);
      if (kTransposed) {
        ht[(size_t)(4 * q + 0) * ldt + m] = Mode::From(v.x);
        ht[(size_t)(4 * q + 1) * ldt + m] = Mode::From(v.y);
        ht[(size_t)(4 * q + 2) * ldt + m] = Mode::From(v.z);
        ht[(size_t)(4 * q + 3) * ldt + m] = Mode::From(v.w);
      }
    }
  }
}

// acc[rb] += A[rows rb*32 .. +31][0..K) . B[n][0..K)^T for the wavefront's 32 columns n: A in LDS
// (row stride lda elements), B rows in global memory, both k-contiguous.  kSteps > 0: the number of
// steps of k is known when compiling and the loop is unrolled completely, B asked for Mode::kAhead steps
// ahead of its use (the compiler counts outstanding loads exactly in straight-line code; around a
// loop it waits for all of them at every iteration).  kSteps == 0: any K, that loop.
template <typename Mode, int RB, int kSteps>
__device__ __forceinline__ void TileProduct(Acc16 (&acc)[RB], const typename Mode::Elem *a_lane,
                                            int lda, const uint4 *b_block, int lane, int K) {
  constexpr int kChunk = Mode::kChunk;
  if constexpr (kSteps > 0) {
    constexpr int kAhead = Mode::kAhead;  // steps of k between asking for B and using it
    Frag fb[kAhead + 1], fa[RB];
#pragma unroll
    for (int i = 0; i < kAhead; ++i)
      if (i < kSteps) fb[i] = LoadFragB(b_block + (size_t)i * kFragQuads, lane);
#pragma unroll
    for (int kc = 0; kc < kSteps; ++kc) {
      if (kc + kAhead < kSteps)
        fb[(kc + kAhead) % (kAhead + 1)] = LoadFragB(b_block + (size_t)(kc + kAhead) * kFragQuads, lane);
      // A comes from LDS when its step begins: a second set of its fragments, asked for a step
      // ahead, cost the forward kernel the registers it then spilled (155 -> 132 us in bfloat16
      // without); the SIMD's other wavefront multiplies while this one waits for LDS.
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) fa[rb] = LoadFrag(a_lane + (size_t)rb * 32 * lda + (size_t)kc * kChunk);
      __builtin_amdgcn_sched_barrier(0);  // the requests above stay above the multiplies below
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) Mode::Mma(acc[rb], fa[rb], fb[kc % (kAhead + 1)]);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    const int chunks = K / kChunk, last = chunks - 1;
    Frag f0 = LoadFragB(b_block, lane);
    Frag f1 = LoadFragB(b_block + (size_t)(1 < last ? 1 : last) * kFragQuads, lane);
    for (int kc = 0; kc < chunks; ++kc) {
      const int ahead = kc + 2 < last ? kc + 2 : last;
      const Frag f2 = LoadFragB(b_block + (size_t)ahead * kFragQuads, lane);
      Frag fa[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) fa[rb] = LoadFrag(a_lane + (size_t)rb * 32 * lda + (size_t)kc * kChunk);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) Mode::Mma(acc[rb], fa[rb], f0);
      f0 = f1;
      f1 = f2;
    }
  }
}

// A lane's value as seen by the lane that a DPP control pairs it with (within rows of 16 lanes).
template <int kCtrl>
__device__ __forceinline__ float Dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, true));
}
// (max, sum of exp relative to it) of two sets of logits merged
__device__ __forceinline__ void MergeLse(float &m, float &s, float om, float os) {
  const float d = m - om;
  const float e = __expf(-fabsf(d));
  s = d >= 0 ? s + os * e : s * e + os;
  m = fmaxf(m, om);
}
// accumulator element r of a lane: row (r >> 2) * 8 + half * 4 + (r & 3) of the 32 x 32 block,
// column lane & 31
__device__ __forceinline__ int AccRow(int r, int half) { return (r >> 2) * 8 + half * 4 + (r & 3); }

constexpr float kLowest = -3.0e38f;  // start of a running maximum (finite: -inf - -inf is NaN)

// d logits of one element: -softmax (gx + gy) + gx [n == symbol] + gy [n == blank]; g = {gx, gy,
// symbol, norm}
__device__ __forceinline__ float LogitGrad(float z, int n, const float4 g, int blank) {
  float v = -__expf(z - g.w) * (g.x + g.y);
  if (n == (int)g.z) v += g.x;
  if (n == blank) v += g.y;
  return v;
}

// The same for the hybrid autoregressive transducer (k2/python/k2/rnnt_loss.py:992-1177): column 0
// is the blank with its own sigmoid sg, py = log sg, and the other columns share a softmax whose
// normaliser g.w leaves column 0 out, px = z[symbol] - norm + log(1 - sg):
//   d/d z[0] = gy (1 - sg) - gx sg,   d/d z[n >= 1] = -exp(z[n] - norm) gx,   + gx at the symbol.
__device__ __forceinline__ float LogitGradHat(float z, int n, const float4 g) {
  float v;
  if (n == 0) {
    const float e = __expf(-fabsf(z));
    const float sg = (z >= 0 ? 1.0f : e) / (1.0f + e);
    v = g.y * (1.0f - sg) - g.x * sg;
  } else {
    v = -__expf(z - g.w) * g.x;
  }
  if (n == (int)g.z) v += g.x;
  return v;
}

// ---------------------------------------------------------------------------------- forward
//
// LDS: h [MT][D + pad]; row meta; the two picked logits per row; per wavefront (max, sum) per row.
// kHat: get_hat_logprobs_pruned in place of get_rnnt_logprobs_pruned: the normaliser leaves column 0
// out, py = log sigmoid(z[0]), px = z[symbol] - norm + (py - z[0]) (a.blank is 0).
template <typename Mode, int RB, int kD, bool kHat>
__global__ __launch_bounds__(kThreads) void JoinerForwardKernel(const JoinerArgs a) {
  constexpr int kStepsD = kD / Mode::kChunk;  // 0: D only known at run time
  constexpr int MT = 32 * RB;
  typedef typename Mode::Elem Elem;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int ldh = (kD > 0 ? kD : a.D) + Mode::kPad;  // a constant where D is one: LDS offsets become immediates
  Elem *h = reinterpret_cast<Elem *>(smem);
  RowMeta *meta = reinterpret_cast<RowMeta *>(smem + (size_t)MT * ldh * sizeof(Elem));
  float *zsym = reinterpret_cast<float *>(meta + MT);
  float *zblank = zsym + MT;
  float *part_m = zblank + MT;  // [kWaves][MT]
  float *part_s = part_m + kWaves * MT;

  const long long f0 = (long long)blockIdx.x * a.tpt;
  const int rows = LoadMeta<MT>(a, f0, meta);
  for (int m = threadIdx.x; m < MT; m += kThreads) { zsym[m] = 0.f; zblank[m] = 0.f; }
  __syncthreads();
  StageActivations<Mode, MT, false, 8, kD>(a, meta, rows, h, ldh, nullptr, 0);
  __syncthreads();

  const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in all lanes: a scalar
  const Elem *a_lane = h + (size_t)col * ldh + half * (Mode::kChunk / 2);
  float run_m[RB][16], run_s[RB][16];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int r = 0; r < 16; ++r) { run_m[rb][r] = kLowest; run_s[rb][r] = 0.f; }

  for (int n0 = 0; n0 < a.Cpad; n0 += kNTile) {
    const int n = n0 + wave * 32 + col;
    Acc16 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][r] = 0.f;
    TileProduct<Mode, RB, kStepsD>(acc, a_lane, ldh, BOperand(a.wk, (n0 >> 5) + wave, a.D / Mode::kChunk, 0), lane, a.D);
    const float bn = (n < a.C && a.bias != nullptr) ? a.bias[n] : 0.f;
    if (n0 == 0) {
      // the first tile of columns starts the running pairs: no exponential (a lane whose column
      // lies beyond C keeps the empty pair, and so does the one of column 0 where that column has
      // its own sigmoid)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (n < a.C && !(kHat && n == 0)) { run_m[rb][r] = acc[rb][r] + bn; run_s[rb][r] = 1.0f; }
    } else if (n < a.C) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float z = acc[rb][r] + bn;
          const float m = run_m[rb][r], d = z - m;
          const float e = __expf(-fabsf(d));
          run_s[rb][r] = d > 0 ? run_s[rb][r] * e + 1.0f : run_s[rb][r] + e;
          run_m[rb][r] = d > 0 ? z : m;
        }
    }
    if (n < a.C) {
      // the two logits a row contributes: the lane that holds one parks it
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = rb * 32 + AccRow(r, half);
          if (n == meta[row].sym) zsym[row] = acc[rb][r] + bn;
        }
      if (n == a.blank) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int r = 0; r < 16; ++r) zblank[rb * 32 + AccRow(r, half)] = acc[rb][r] + bn;
      }
    }
  }
  // (max, sum) of a row: over the 32 lanes that hold its columns, then over the wavefronts.  The
  // lanes of a half wavefront hold the same 16 RB rows; at each step a lane keeps one half of the
  // rows it still holds and hands the other half to its partner (xor 1, 2 inside quads on the vector
  // ALU, xor 4, 8, 16 through the LDS crossbar), so every merge is done once, and after five steps
  // (six with RB = 2) each lane holds the merged pair of the rows that the bits of its number select.
  {
    constexpr int kN = 16 * RB;
    float vm[kN], vs[kN];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) { vm[rb * 16 + r] = run_m[rb][r]; vs[rb * 16 + r] = run_s[rb][r]; }
    int mine = 0;  // index rb * 16 + r of the first row this lane ends up with
#define K2AMD_SCATTER_STEP(COUNT, BIT, EXCHANGE)                              \
    {                                                                         \
      const bool up = (col & (BIT)) != 0;                                     \
      _Pragma("unroll") for (int j = 0; j < (COUNT) / 2; ++j) {               \
        float km = up ? vm[j + (COUNT) / 2] : vm[j], ks = up ? vs[j + (COUNT) / 2] : vs[j]; \
        const float sm = up ? vm[j] : vm[j + (COUNT) / 2], ss = up ? vs[j] : vs[j + (COUNT) / 2]; \
        MergeLse(km, ks, EXCHANGE(sm), EXCHANGE(ss));                         \
        vm[j] = km;                                                           \
        vs[j] = ks;                                                           \
      }                                                                       \
      if (up) mine += (COUNT) / 2;                                            \
    }
#define K2AMD_X1(v) Dpp<0xB1>(v)
#define K2AMD_X2(v) Dpp<0x4E>(v)
#define K2AMD_X4(v) __shfl_xor(v, 4, kWave)
#define K2AMD_X8(v) __shfl_xor(v, 8, kWave)
#define K2AMD_X16(v) __shfl_xor(v, 16, kWave)
    K2AMD_SCATTER_STEP(kN, 1, K2AMD_X1)
    K2AMD_SCATTER_STEP(kN / 2, 2, K2AMD_X2)
    K2AMD_SCATTER_STEP(kN / 4, 4, K2AMD_X4)
    K2AMD_SCATTER_STEP(kN / 8, 8, K2AMD_X8)
    if constexpr (RB == 2) {
      K2AMD_SCATTER_STEP(kN / 16, 16, K2AMD_X16)
      const int row = (mine >> 4) * 32 + AccRow(mine & 15, half);
      part_m[wave * MT + row] = vm[0];
      part_s[wave * MT + row] = vs[0];
    } else {
      // RB == 1: one row left per pair of lanes 16 apart; merge it, the lower lane stores
      float km = vm[0], ks = vs[0];
      MergeLse(km, ks, K2AMD_X16(vm[0]), K2AMD_X16(vs[0]));
      if ((col & 16) == 0) {
        const int row = AccRow(mine & 15, half);
        part_m[wave * MT + row] = km;
        part_s[wave * MT + row] = ks;
      }
    }
#undef K2AMD_SCATTER_STEP
#undef K2AMD_X1
#undef K2AMD_X2
#undef K2AMD_X4
#undef K2AMD_X8
#undef K2AMD_X16
  }
  __syncthreads();
  for (int row = threadIdx.x; row < rows; row += kThreads) {
    float m = part_m[row], s = part_s[row];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) MergeLse(m, s, part_m[w * MT + row], part_s[w * MT + row]);
    const float norm = m + logf(s);
    const RowMeta rm = meta[row];
    const int b = rm.bt / a.Tn, t = rm.bt - b * a.Tn;
    a.norm[(size_t)f0 * a.R + row] = norm;
    const int T1 = a.rnnt_type == K2AMD_REGULAR ? a.Tn + 1 : a.Tn;
    const bool has_blank = a.blank >= 0 && a.blank < a.C;
    float shift = 0.f, yv = has_blank ? zblank[row] - norm : Real<float>::NegInf();
    if constexpr (kHat) {
      const float z0 = zblank[row];
      yv = fminf(z0, 0.f) - log1pf(__expf(-fabsf(z0)));  // log sigmoid(z0)
      shift = yv - z0;                                   // log(1 - sigmoid(z0))
    }
    a.py[((size_t)b * (a.S + 1) + rm.s) * a.Tn + t] = yv;
    if (rm.s < a.S) {
      float v = rm.sym >= 0 ? zsym[row] - norm : Real<float>::NegInf();
      if constexpr (kHat) v += shift;  // (-inf stays -inf)
      if (a.rnnt_type == K2AMD_REGULAR && a.boundary != nullptr && a.boundary[4 * b + 3] == t)
        v = Real<float>::NegInf();
      a.px[((size_t)b * a.S + rm.s) * T1 + t] = v;
    }
  }
}

// ------------------------------------------------------------ backward, gradients of am and lm
//
// One tile of MT rows per workgroup.  Per tile of 256 columns c: logits -> d logits into LDS, then
// d h += d logits . weight[c-tile] with d h [MT][D] kept in accumulators over all column tiles
// (wavefront w owns the 32-column blocks w and w + 8 of D).  At the end d pre = d h (1 - h^2) goes
// through LDS 128 columns at a time: am_grad[frame] is the sum over the frame's R rows (plain
// stores: a frame lies in one tile), lm_grad[b, s] collects its rows with atomic adds (runs of
// equal s along t are added up first).
template <typename Mode, int RB, int kD, bool kHat>
__global__ __launch_bounds__(kThreads) void JoinerBackwardRowsKernel(const JoinerArgs a) {
  constexpr int kStepsD = kD / Mode::kChunk;  // 0: D only known at run time
  constexpr int MT = 32 * RB;
  typedef typename Mode::Elem Elem;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int ldh = (kD > 0 ? kD : a.D) + Mode::kPad;  // a constant where D is one: LDS offsets become immediates
  constexpr int ldz = kNTile + Mode::kPad;
  constexpr int kLdStage = kStageCols + 4;
  static_assert((size_t)MT * kLdStage * sizeof(float) <= (size_t)MT * ldz * sizeof(Elem), "stage fits dz");
  Elem *h = reinterpret_cast<Elem *>(smem);
  Elem *dz = h + (size_t)MT * ldh;
  float *stage = reinterpret_cast<float *>(dz);  // after the last column tile
  float4 *hdr = reinterpret_cast<float4 *>(dz + (size_t)MT * ldz);
  RowMeta *meta = reinterpret_cast<RowMeta *>(hdr + MT);
  unsigned long long *run_ends = reinterpret_cast<unsigned long long *>(meta + MT);  // [32]

  const long long f0 = ((long long)a.tile0 + blockIdx.x) * a.tpt;
  const int rows = LoadMeta<MT>(a, f0, meta);
  for (int m = threadIdx.x; m < MT; m += kThreads)
    hdr[m] = m < rows ? a.hdr[(size_t)f0 * a.R + m] : make_float4(0.f, 0.f, -1.f, 3.0e38f);  // padding: exp(. - norm) = 0
  __syncthreads();
  StageActivations<Mode, MT, false, 8, kD>(a, meta, rows, h, ldh, nullptr, 0);
  __syncthreads();
  {  // The tile's activations go to the workspace as an operand with k = row: this tile is step
     // blockIdx.x of k, and a 16-byte group holds consecutive rows of one column d.
    static_assert(MT == Mode::kChunk, "a tile of rows is one step of k");
    constexpr int kPer = 16 / sizeof(Elem);
    uint4 *dst = static_cast<uint4 *>(a.hs);
    const int groups = (a.D / 32) * kFragQuads;
    for (int g = threadIdx.x; g < groups; g += kThreads) {
      const int nb = g / kFragQuads, r = g % kFragQuads, i = r >> 6, l = r & 63;
      const Elem *src = h + (size_t)((l >> 5) * (Mode::kChunk / 2) + i * kPer) * ldh + nb * 32 + (l & 31);
      uint4 out;
      if constexpr (sizeof(Elem) == 4) {
        out = make_uint4(AsBits(Mode::To(src[0])), AsBits(Mode::To(src[ldh])), AsBits(Mode::To(src[2 * ldh])),
                         AsBits(Mode::To(src[3 * ldh])));
      } else {
        unsigned w32[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          w32[e] = (unsigned)(unsigned short)src[(size_t)(2 * e) * ldh] |
                   ((unsigned)(unsigned short)src[(size_t)(2 * e + 1) * ldh] << 16);
        out = make_uint4(w32[0], w32[1], w32[2], w32[3]);
      }
      dst[((size_t)nb * a.tiles + blockIdx.x) * kFragQuads + r] = out;
    }
  }

  const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in all lanes: a scalar
  const int koff = half * (Mode::kChunk / 2);
  Acc16 dh[2][RB];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) dh[i][rb][r] = 0.f;

  for (int n0 = 0; n0 < a.Cpad; n0 += kNTile) {
    const int n = n0 + wave * 32 + col;
    Acc16 acc[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rb][r] = 0.f;
    TileProduct<Mode, RB, kStepsD>(acc, h + (size_t)col * ldh + koff, ldh,
                                   BOperand(a.wk, (n0 >> 5) + wave, a.D / Mode::kChunk, 0), lane, a.D);
    const float bn = (n < a.C && a.bias != nullptr) ? a.bias[n] : 0.f;
    float colsum = 0.f;
    // d logits as an operand with k = row, for the weight kernel: block of columns (n0 >> 5) + wave,
    // step blockIdx.x.  A lane holds runs of four consecutive rows of its column (AccRow), which
    // are half a 16-byte group in bfloat16 and a whole one in fp32.
    unsigned char *zblock = static_cast<unsigned char *>(a.dzs) +
                            ((size_t)((n0 >> 5) + wave) * a.tiles + blockIdx.x) * kFragQuads * 16;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        Elem run[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = j * 4 + e;
          const int row = rb * 32 + AccRow(r, half);
          const float z = acc[rb][r] + bn;
          const float v = n < a.C ? (kHat ? LogitGradHat(z, n, hdr[row]) : LogitGrad(z, n, hdr[row], a.blank)) : 0.f;
          run[e] = Mode::From(v);
          colsum += Mode::To(run[e]);
          dz[(size_t)row * ldz + wave * 32 + col] = run[e];
        }
        const int k = rb * 32 + j * 8 + half * 4;  // the run's first row = its position in the step of k
        constexpr int kHalfChunk = Mode::kChunk / 2, kPer = 16 / (int)sizeof(Elem);
        const int kin = k % kHalfChunk;
        unsigned char *at = zblock + ((size_t)(kin / kPer) * 64 + (k / kHalfChunk) * 32 + col) * 16 +
                            (kin % kPer) * sizeof(Elem);
        if constexpr (sizeof(Elem) == 4) {
          *reinterpret_cast<uint4 *>(at) = make_uint4(AsBits(Mode::To(run[0])), AsBits(Mode::To(run[1])),
                                                      AsBits(Mode::To(run[2])), AsBits(Mode::To(run[3])));
        } else {
          uint2 p;
          p.x = (unsigned)(unsigned short)run[0] | ((unsigned)(unsigned short)run[1] << 16);
          p.y = (unsigned)(unsigned short)run[2] | ((unsigned)(unsigned short)run[3] << 16);
          *reinterpret_cast<uint2 *>(at) = p;
        }
      }
    // the column's sum over the tile's rows (the two halves of the wavefront hold 16 RB rows each)
    colsum += __shfl_xor(colsum, 32, kWave);
    if (half == 0) a.bias_part[(size_t)blockIdx.x * a.Cpad + n] = colsum;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if ((wave + kWaves * i) * 32 < a.D)
        TileProduct<Mode, RB, kNTile / Mode::kChunk>(dh[i], dz + (size_t)col * ldz + koff, ldz,
                                                     BOperand(a.wc, wave + kWaves * i, a.Cpad / Mode::kChunk, n0 / Mode::kChunk), lane, kNTile);
    }
    __syncthreads();
  }

  const int c = threadIdx.x % kStageCols;
  const int part = __builtin_amdgcn_readfirstlane(threadIdx.x / kStageCols);  // the same in a wavefront
  constexpr int kParts = kThreads / kStageCols;
  const int nf = rows / a.R;
  // What the sums below need to know about the tile's rows does not depend on the column: where a
  // run of equal lm rows ends (bit fl of a position's word: after frame fl).  Worked out once per
  // tile, one thread per position k; the loops over the columns are then reads and adds.
  constexpr int kTakes = 2;
  static_assert(MT <= 64, "a bit per frame");
  if ((int)threadIdx.x < a.R) {
    const int k = threadIdx.x;
    unsigned long long ends = 0;
    int key = meta[k].lmrow;
    for (int fl = 0; fl < nf; ++fl) {
      const int next = fl + 1 < nf ? meta[(fl + 1) * a.R + k].lmrow : -1;
      if (next != key) ends |= 1ull << fl;
      key = next;
    }
    run_ends[k] = ends;
  }
  auto ends_of = [&](int k) -> unsigned long long {  // (after the first barrier below)
    const unsigned long long ends = run_ends[k];
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)ends);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(ends >> 32));
    return ((unsigned long long)hi << 32) | lo;
  };
  for (int d0 = 0; d0 < a.D; d0 += kStageCols) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int db = wave + kWaves * i;
      if (db * 32 >= d0 && db * 32 < d0 + kStageCols && db * 32 < a.D) {
        const int d = db * 32 + col;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int row = rb * 32 + AccRow(r, half);
            const float hv = Mode::To(h[(size_t)row * ldh + d]);
            stage[row * kLdStage + d - d0] = dh[i][rb][r] * (1.0f - hv * hv);
          }
      }
    }
    __syncthreads();
    if (d0 + c < a.D) {
      // am_grad[frame] = the sum of the frame's R rows; four values asked for before any is used
      // (one read per iteration, each waiting for the one before it, is what these loops cost).
      const int frame_step = a.R * kLdStage;
      for (int fl = part; fl < nf; fl += kParts) {
        const float *src = stage + fl * frame_step + c;
        float sum = 0.f;
        int k = 0;
        for (; k + 4 <= a.R; k += 4) {
          const float v0 = src[0], v1 = src[kLdStage], v2 = src[2 * kLdStage], v3 = src[3 * kLdStage];
          sum += v0; sum += v1; sum += v2; sum += v3;
          src += 4 * kLdStage;
        }
        for (; k < a.R; ++k, src += kLdStage) sum += *src;
        a.am_grad[(size_t)(f0 + fl) * a.D + d0 + c] = sum;
      }
      // lm_grad[lm row] += the sum of each run of frames that took that row at position k
      for (int kb = part; kb < a.R; kb += kTakes * kParts) {
#pragma unroll
        for (int t = 0; t < kTakes; ++t) {
          const int k = kb + t * kParts;
          if (k >= a.R) break;
          unsigned long long ends = ends_of(k);
          const float *src = stage + k * kLdStage + c;
          float sum = 0.f;
          int fl = 0;
          for (; fl + 4 <= nf; fl += 4) {
            const float v[4] = {src[0], src[frame_step], src[2 * frame_step], src[3 * frame_step]};
            src += 4 * frame_step;
            const unsigned four = (unsigned)(ends >> fl) & 15u;
            if (four == 0) {  // (the common case: the run goes on)
              sum += v[0]; sum += v[1]; sum += v[2]; sum += v[3];
              continue;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              sum += v[j];
              if (four >> j & 1) {
                atomicAdd(a.lm_grad + (size_t)meta[(fl + j) * a.R + k].lmrow * a.D + d0 + c, sum);
                sum = 0.f;
              }
            }
          }
          for (; fl < nf; ++fl, src += frame_step) {
            sum += *src;
            if (ends >> fl & 1) {
              atomicAdd(a.lm_grad + (size_t)meta[fl * a.R + k].lmrow * a.D + d0 + c, sum);
              sum = 0.f;
            }
          }
        }
      }
    }
    __syncthreads();
  }
}

// ------------------------------------------------------- backward, gradients of weight and bias
//
//   weight_grad[c][d] = sum over rows of d logits[row][c] h[row][d]
// is a product over k = row of two operands that the rows kernel has left in the workspace in the
// order the multiplies consume them, so this kernel is nothing but loads and multiplies: no LDS, no
// barrier.  A workgroup of four wavefronts (one per SIMD, so that a wavefront has the registers for
// eight accumulator blocks and two sets of operands) owns 128 columns c x 256 columns d of the
// gradient and one share of the steps of k; wavefront w takes two blocks of c and four of d.  The
// workgroups that share a share of k are eight apart in the grid, which puts them on one XCD: what
// one of them has fetched the others find in that XCD's L2.  The sums meet in weight_grad
// (zeroed by the launcher) through atomic adds; the workgroups of the first block of d also add up
// their tiles' sums of d logits for bias_grad.
constexpr int kWgThreads = 256;
constexpr int kWgCBlocks = 2, kWgDBlocks = 4;  // per wavefront
template <typename Mode>
__global__ __launch_bounds__(kWgThreads) void JoinerWeightGradKernel(const JoinerArgs a, int dtiles, int shares) {
  const int share = blockIdx.x % shares, combo = blockIdx.x / shares;
  const int ct = combo / dtiles, dt = combo - ct * dtiles;
  const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int cb0 = ct * 4 + (wave & 1) * kWgCBlocks, db0 = dt * 8 + (wave >> 1) * kWgDBlocks;
  const int ncb = a.Cpad / 32, ndb = a.D / 32;
  const int t0 = (int)((long long)a.tiles * share / shares), t1 = (int)((long long)a.tiles * (share + 1) / shares);
  bool c_ok[kWgCBlocks], d_ok[kWgDBlocks];
#pragma unroll
  for (int i = 0; i < kWgCBlocks; ++i) c_ok[i] = cb0 + i < ncb;
#pragma unroll
  for (int j = 0; j < kWgDBlocks; ++j) d_ok[j] = db0 + j < ndb;
  Acc16 acc[kWgCBlocks][kWgDBlocks];
#pragma unroll
  for (int i = 0; i < kWgCBlocks; ++i)
#pragma unroll
    for (int j = 0; j < kWgDBlocks; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  struct Operands {
    Frag z[kWgCBlocks], h[kWgDBlocks];
  };
  auto load = [&](Operands &o, int t) {
#pragma unroll
    for (int i = 0; i < kWgCBlocks; ++i)
      if (c_ok[i]) o.z[i] = LoadFragB(BOperand(a.dzs, cb0 + i, a.tiles, t), lane);
#pragma unroll
    for (int j = 0; j < kWgDBlocks; ++j)
      if (d_ok[j]) o.h[j] = LoadFragB(BOperand(a.hs, db0 + j, a.tiles, t), lane);
  };
  auto multiply = [&](const Operands &o) {
#pragma unroll
    for (int i = 0; i < kWgCBlocks; ++i)
#pragma unroll
      for (int j = 0; j < kWgDBlocks; ++j)
        if (c_ok[i] && d_ok[j]) Mode::Mma(acc[i][j], o.z[i], o.h[j]);
  };
  if (t0 < t1 && c_ok[0] && d_ok[0]) {
    Operands o0, o1;
    load(o0, t0);
    for (int t = t0; t < t1; t += 2) {
      load(o1, t + 1 < t1 ? t + 1 : t);
      multiply(o0);
      load(o0, t + 2 < t1 ? t + 2 : t);
      if (t + 1 < t1) multiply(o1);
    }
#pragma unroll
    for (int i = 0; i < kWgCBlocks; ++i)
#pragma unroll
      for (int j = 0; j < kWgDBlocks; ++j) {
        if (!c_ok[i] || !d_ok[j]) continue;
        const int d = (db0 + j) * 32 + col;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c = (cb0 + i) * 32 + AccRow(r, half);
          if (c < a.C) atomicAdd(a.weight_grad + (size_t)c * a.D + d, acc[i][j][r]);
        }
      }
  }
  if (dt == 0 && a.bias_grad != nullptr) {
    const int c = ct * 128 + (int)(threadIdx.x & 127);
    if (c < a.C) {
      float sum = 0.f;
      for (int t = t0 + (int)(threadIdx.x >> 7); t < t1; t += kWgThreads / 128)
        sum += a.bias_part[(size_t)t * a.Cpad + c];
      atomicAdd(a.bias_grad + c, sum);
    }
  }
}

// ---------------------------------------------------------------------------- small kernels

// The weight [C][D] in the operand type and in the order the multiplies read it (see BOperand):
// wk with rows n = c (Cpad of them, zeros beyond C) and k = d; wc with rows n = d (Dpad) and k = c
// (Cpad, zeros beyond C and D).  One thread per 16-byte group.  The same launch fills the tensors
// that the kernels after it only write in part (px, py: -inf) or add to (the sums of atomic adds).
struct Fills {
  float *at[3];
  size_t n[3];
  float value;
};
template <typename Mode>
__global__ void JoinerPrepWeightKernel(const float *__restrict__ weight, uint4 *wk, uint4 *wc, int C,
                                       int D, int Cpad, int Dpad, const Fills fills) {
  typedef typename Mode::Elem Elem;
#pragma unroll
  for (int f = 0; f < 3; ++f) {
    float *at = fills.at[f];
    const size_t n = fills.n[f];
    if (at == nullptr || n == 0) continue;
    // whole 16-byte groups where the tensor's address allows, single floats around them
    const size_t head = ((16 - (reinterpret_cast<size_t>(at) & 15)) & 15) / sizeof(float);
    const size_t lead = head < n ? head : n, quads = (n - lead) / 4;
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
    const float4 four = make_float4(fills.value, fills.value, fills.value, fills.value);
    for (size_t i = first; i < quads; i += stride) reinterpret_cast<float4 *>(at + lead)[i] = four;
    if (first < lead) at[first] = fills.value;
    if (first < n - lead - 4 * quads) at[lead + 4 * quads + first] = fills.value;
  }
  constexpr int kPer = 16 / sizeof(Elem);  // elements per group
  const size_t nk = (size_t)Cpad * D / kPer, nc = wc != nullptr ? (size_t)Dpad * Cpad / kPer : 0;
  for (size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x; g < nk + nc;
       g += (size_t)gridDim.x * blockDim.x) {
    const bool second = g >= nk;
    const size_t j = second ? g - nk : g;
    const int ksteps = (second ? Cpad : D) / Mode::kChunk;
    const int lane = (int)(j & 63), i = (int)((j >> 6) & 3);
    const size_t blockstep = j >> 8;
    const int step = (int)(blockstep % ksteps), nb = (int)(blockstep / ksteps);
    const int n = nb * 32 + (lane & 31);
    const int k0 = step * Mode::kChunk + (lane >> 5) * (Mode::kChunk / 2) + i * kPer;
    Elem v[kPer];
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      const int c = second ? k0 + e : n, d = second ? n : k0 + e;
      v[e] = Mode::From(c < C && d < D ? weight[(size_t)c * D + d] : 0.f);
    }
    uint4 out;
    if (sizeof(Elem) == 4) {
      out = make_uint4(AsBits(Mode::To(v[0])), AsBits(Mode::To(v[1])), AsBits(Mode::To(v[2])), AsBits(Mode::To(v[3])));
    } else {
      unsigned w32[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        w32[e] = (unsigned)(unsigned short)v[(2 * e) % kPer] | ((unsigned)(unsigned short)v[(2 * e + 1) % kPer] << 16);
      out = make_uint4(w32[0], w32[1], w32[2], w32[3]);
    }
    (second ? wc : wk)[j] = out;
  }
}

// px[b,s,t] += py[b,s+1,t] (k2/python/k2/rnnt_loss.py:1345-1346); T1 == Tn here.
__global__ void JoinerConstrainedKernel(float *__restrict__ px, const float *__restrict__ py, int B,
                                        int S, int Tn) {
  const size_t n = (size_t)B * S * Tn;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (size_t)gridDim.x * blockDim.x) {
    const size_t b = i / ((size_t)S * Tn), rem = i - b * (size_t)S * Tn;
    px[i] += py[b * (size_t)(S + 1) * Tn + Tn + rem];
  }
}

// Per row {gx, gy, symbol, norm}: the gradients that reach the row's px and py values, times what
// reaches the sequence's score (one thread per row pays the look-up chain for 64 rows at a time).
__global__ void JoinerRowHeaderKernel(const JoinerArgs a, const float *__restrict__ px_grad,
                                      const float *__restrict__ py_grad,
                                      const float *__restrict__ seq_scale, float4 *__restrict__ hdr) {
  const long long rows = a.frames * a.R;
  const long long row = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= rows) return;
  const long long frame = row / a.R;
  const int k = (int)(row - frame * a.R);
  const RowMeta rm = MetaOf(a, frame, k);
  const int b = rm.bt / a.Tn, t = rm.bt - b * a.Tn;
  const int T1 = a.rnnt_type == K2AMD_REGULAR ? a.Tn + 1 : a.Tn;
  const float scale = seq_scale != nullptr ? seq_scale[b] : 1.0f;
  float gx = 0.f;
  int sym = rm.sym;
  if (rm.s < a.S && sym >= 0) {
    const bool cut = a.rnnt_type == K2AMD_REGULAR && a.boundary != nullptr && a.boundary[4 * b + 3] == t;
    if (!cut) gx = MulRounded(px_grad[((size_t)b * a.S + rm.s) * T1 + t], scale);
  } else {
    sym = -1;
  }
  float gy = MulRounded(py_grad[((size_t)b * (a.S + 1) + rm.s) * a.Tn + t], scale);
  if (a.rnnt_type == K2AMD_CONSTRAINED && rm.s >= 1)
    gy += MulRounded(px_grad[((size_t)b * a.S + (rm.s - 1)) * T1 + t], scale);  // px += py[:, 1:]
  hdr[row] = make_float4(gx, gy, (float)sym, a.norm[row]);
}

// ------------------------------------------------------------------------------- launchers

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }
size_t ElemBytes(int precision) { return precision == K2AMD_JOINER_BF16 ? 2 : 4; }

// A lattice without frames: the regular one still has its px column T, which the reference pads
// with -inf (k2/python/k2/rnnt_loss.py:1310-1319).
__global__ void JoinerFillKernel(float *__restrict__ dst, size_t n, float v) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = v;
}

bool JoinerShapeOk(int B, int S, int T, int R, int C, int D) {
  if (B < 0 || S < 0 || T < 0 || R < 1 || C < 1) return false;
  if (D < 64 || D > kMaxD || D % 64 != 0 || R > 32 || R > S + 1 || C > (1 << 20)) return false;
  const long long rows = (long long)B * T * R;
  return rows * 4 < (1ll << 31) && (long long)B * (S + 1) * (T + 1) < (1ll << 31) &&
         (long long)B * (S + 1) * D < (1ll << 31) && (long long)B * T * D < (1ll << 31);
}

struct WorkspaceLayout {
  size_t wk, wc, hdr, forward_total, hs, dzs, bias_part, total;
};
// rows per tile of the backward's rows kernel, which is one step of k of the weight kernel
int RowsTile(int precision) { return precision == K2AMD_JOINER_BF16 ? 64 : 32; }
// The backward goes through the tiles in passes of equal size whose operands (activations and
// logit gradients of the pass's rows) stay within this many elements (256 MB in bfloat16, 512 MB
// in fp32), so that what it keeps does not grow with B T R x C.  The environment variable
// K2AMD_JOINER_PASS_ELEMS sets another bound (read at every call: the tests use it to go through
// several passes at small shapes).
constexpr size_t kPassElems = (size_t)128 << 20;
size_t PassElems() {
  const char *text = std::getenv("K2AMD_JOINER_PASS_ELEMS");
  const long long given = text != nullptr ? std::atoll(text) : 0;
  return given > 0 ? (size_t)given : kPassElems;
}
size_t TilesPerPass(size_t tiles, int C, int D, int precision) {
  const size_t per_tile = (size_t)RowsTile(precision) * ((size_t)D + RoundUp(C, kNTile));
  const size_t most = PassElems() / per_tile > 0 ? PassElems() / per_tile : 1;
  const size_t passes = (tiles + most - 1) / most;
  return passes > 0 ? (tiles + passes - 1) / passes : 0;
}
WorkspaceLayout LayoutOf(int B, int T, int R, int C, int D, int precision) {
  const size_t e = ElemBytes(precision);
  const size_t Cpad = RoundUp(C, kNTile), Dpad = RoundUp(D, kNTile);
  WorkspaceLayout w;
  w.wk = 0;
  w.wc = (Cpad * D * e + 255) / 256 * 256;
  w.hdr = w.wc + (Dpad * Cpad * e + 255) / 256 * 256;
  w.forward_total = w.wc;  // the forward multiplies by the first copy only
  const size_t tpt = RowsTile(precision) / R;
  const size_t tiles = tpt > 0 ? ((size_t)B * T + tpt - 1) / tpt : 0;
  const size_t pass_tiles = TilesPerPass(tiles, C, D, precision);
  const size_t padded_rows = pass_tiles * RowsTile(precision);
  w.hs = (w.hdr + (size_t)B * T * R * sizeof(float4) + 255) / 256 * 256;
  w.dzs = w.hs + (padded_rows * D * e + 255) / 256 * 256;
  w.bias_part = w.dzs + (padded_rows * Cpad * e + 255) / 256 * 256;
  w.total = w.bias_part + pass_tiles * Cpad * sizeof(float);
  return w;
}

template <typename K>
int AllowLds(K kernel, size_t bytes) {
  if (bytes > 160 * 1024) return K2AMD_ERR_UNSUPPORTED;
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) == hipSuccess
             ? K2AMD_OK
             : K2AMD_ERR_LAUNCH;
}

JoinerArgs MakeArgs(const float *am, const float *lm, const int64_t *ranges, const float *bias,
                    const int64_t *symbols, const int64_t *boundary, int B, int S, int T, int R,
                    int C, int D, int blank, int rnnt_type, int rows_per_tile, void *workspace,
                    int precision) {
  JoinerArgs a{};
  a.am = am; a.lm = lm; a.bias = bias; a.ranges = ranges; a.symbols = symbols; a.boundary = boundary;
  a.B = B; a.S = S; a.Tn = T; a.R = R; a.C = C; a.D = D; a.blank = blank; a.rnnt_type = rnnt_type;
  a.Cpad = RoundUp(C, kNTile); a.Dpad = RoundUp(D, kNTile);
  a.tpt = rows_per_tile / R;
  a.frames = (long long)B * T;
  const WorkspaceLayout w = LayoutOf(B, T, R, C, D, precision);
  unsigned char *ws = static_cast<unsigned char *>(workspace);
  a.wk = ws + w.wk;
  a.wc = ws + w.wc;
  a.hdr = reinterpret_cast<const float4 *>(ws + w.hdr);
  a.hs = ws + w.hs;
  a.dzs = ws + w.dzs;
  a.bias_part = reinterpret_cast<float *>(ws + w.bias_part);
  return a;
}

template <typename Mode>
int PrepWeights(const float *weight, const JoinerArgs &a, bool both, const Fills &fills, hipStream_t st) {
  hipLaunchKernelGGL(JoinerPrepWeightKernel<Mode>, dim3(1024), dim3(256), 0, st, weight,
                     static_cast<uint4 *>(const_cast<void *>(a.wk)),
                     both ? static_cast<uint4 *>(const_cast<void *>(a.wc)) : nullptr, a.C, a.D, a.Cpad,
                     a.Dpad, fills);
  return LaunchStatus();
}

template <typename Mode, int RB>
int ForwardImpl(const float *weight, JoinerArgs a, bool hat, hipStream_t st) {
  constexpr int MT = 32 * RB;
  const size_t npx = (size_t)a.B * a.S * (a.rnnt_type == K2AMD_REGULAR ? a.Tn + 1 : a.Tn);
  const size_t npy = (size_t)a.B * (a.S + 1) * a.Tn;
  const Fills fills{{a.px, a.py, nullptr}, {npx, npy, 0}, Real<float>::NegInf()};
  int rc = PrepWeights<Mode>(weight, a, false, fills, st);
  if (rc != K2AMD_OK) return rc;
  const size_t lds = (size_t)MT * (a.D + Mode::kPad) * sizeof(typename Mode::Elem) +
                     MT * (sizeof(RowMeta) + (2 + 2 * kWaves) * sizeof(float));
  auto kernel = hat ? (a.D == kMaxD ? JoinerForwardKernel<Mode, RB, kMaxD, true> : JoinerForwardKernel<Mode, RB, 0, true>)
                    : (a.D == kMaxD ? JoinerForwardKernel<Mode, RB, kMaxD, false> : JoinerForwardKernel<Mode, RB, 0, false>);
  rc = AllowLds(kernel, lds);
  if (rc != K2AMD_OK) return rc;
  const long long tiles = (a.frames + a.tpt - 1) / a.tpt;
  if (tiles > 0) hipLaunchKernelGGL(kernel, dim3((unsigned)tiles), dim3(kThreads), lds, st, a);
  if (a.rnnt_type == K2AMD_CONSTRAINED && a.S > 0 && a.frames > 0)
    hipLaunchKernelGGL(JoinerConstrainedKernel, dim3(512), dim3(256), 0, st, a.px, a.py, a.B, a.S, a.Tn);
  return LaunchStatus();
}

template <typename Mode>
int BackwardImpl(const float *weight, JoinerArgs a, const float *px_grad, const float *py_grad,
                 const float *seq_scale, bool hat, hipStream_t st) {
  typedef typename Mode::Elem Elem;
  constexpr bool kBf = sizeof(Elem) == 2;
  const Fills fills{{a.lm_grad, a.weight_grad, a.bias_grad},
                    {(size_t)a.B * (a.S + 1) * a.D, (size_t)a.C * a.D, a.bias_grad != nullptr ? (size_t)a.C : 0},
                    0.f};
  int rc = PrepWeights<Mode>(weight, a, true, fills, st);
  if (rc != K2AMD_OK) return rc;
  const long long rows = a.frames * a.R;
  if (rows == 0) return LaunchStatus();
  hipLaunchKernelGGL(JoinerRowHeaderKernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, a,
                     px_grad, py_grad, seq_scale, const_cast<float4 *>(a.hdr));
  // Gradients of am and lm, tile by tile of 32 (fp32) or 64 (bfloat16) rows, and then those of the
  // weight and the bias from what that kernel left in the workspace (blocks of 128 x 256 of the
  // gradient x shares of the rows), pass by pass.
  constexpr int RB = kBf ? 2 : 1, MT = 32 * RB;
  a.tpt = MT / a.R;
  const size_t lds = (size_t)MT * (a.D + Mode::kPad + kNTile + Mode::kPad) * sizeof(Elem) +
                     MT * (sizeof(float4) + sizeof(RowMeta)) + 32 * sizeof(unsigned long long);
  auto kernel = hat ? (a.D == kMaxD ? JoinerBackwardRowsKernel<Mode, RB, kMaxD, true> : JoinerBackwardRowsKernel<Mode, RB, 0, true>)
                    : (a.D == kMaxD ? JoinerBackwardRowsKernel<Mode, RB, kMaxD, false> : JoinerBackwardRowsKernel<Mode, RB, 0, false>);
  rc = AllowLds(kernel, lds);
  if (rc != K2AMD_OK) return rc;
  const long long tiles = (a.frames + a.tpt - 1) / a.tpt;
  const long long pass_tiles = (long long)TilesPerPass((size_t)tiles, a.C, a.D, kBf ? K2AMD_JOINER_BF16 : K2AMD_JOINER_F32);
  const int ctiles = a.Cpad / 128, dtiles = (a.D + 255) / 256;
  int shares = 256 / (ctiles * dtiles) / 8 * 8;  // one workgroup per compute unit; a multiple of the XCDs
  if (shares < 8) shares = 8;
  for (long long first = 0; first < tiles; first += pass_tiles) {
    a.tile0 = (int)first;
    a.tiles = (int)(tiles - first < pass_tiles ? tiles - first : pass_tiles);
    hipLaunchKernelGGL(kernel, dim3((unsigned)a.tiles), dim3(kThreads), lds, st, a);
    hipLaunchKernelGGL(JoinerWeightGradKernel<Mode>, dim3((unsigned)(ctiles * dtiles * shares)),
                       dim3(kWgThreads), 0, st, a, dtiles, shares);
  }
  return LaunchStatus();
}

}  // namespace
}  // namespace k2amd

using namespace k2amd;

extern "C" {

size_t k2amd_rnnt_joiner_pruned_workspace_bytes(int B, int S, int T, int R, int C, int D,
                                                int precision) {
  if (!JoinerShapeOk(B, S, T, R, C, D)) return 0;
  if (precision != K2AMD_JOINER_F32 && precision != K2AMD_JOINER_BF16) return 0;
  return LayoutOf(B, T, R, C, D, precision).total;
}

size_t k2amd_rnnt_joiner_pruned_forward_workspace_bytes(int B, int S, int T, int R, int C, int D,
                                                        int precision) {
  if (!JoinerShapeOk(B, S, T, R, C, D)) return 0;
  if (precision != K2AMD_JOINER_F32 && precision != K2AMD_JOINER_BF16) return 0;
  return LayoutOf(B, T, R, C, D, precision).forward_total;
}

}  // extern "C"

// hat: the hybrid autoregressive transducer's log-probs (column 0 is the blank, termination_symbol 0)
static int JoinerForwardEntry(const void *am, const void *lm, const int64_t *ranges,
                              const void *weight, const void *bias, const int64_t *symbols,
                              const int64_t *boundary, void *px, void *py, void *normalizers,
                              int B, int S, int T, int R, int C, int D, int termination_symbol,
                              int rnnt_type, int precision, bool hat, void *workspace,
                              size_t workspace_bytes, void *stream) {
  if (!JoinerShapeOk(B, S, T, R, C, D)) return K2AMD_ERR_UNSUPPORTED;
  if (hat && C < 2) return K2AMD_ERR_INVALID_ARGUMENT;
  if (precision != K2AMD_JOINER_F32 && precision != K2AMD_JOINER_BF16) return K2AMD_ERR_INVALID_ARGUMENT;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (rnnt_type != K2AMD_REGULAR && T < S) return K2AMD_ERR_INVALID_ARGUMENT;
  if (B == 0) return K2AMD_OK;
  if (T == 0) {  // no frames: py is empty, px is its one -inf column where the lattice is regular
    if (rnnt_type == K2AMD_REGULAR && S > 0) {
      if (!px) return K2AMD_ERR_INVALID_ARGUMENT;
      const size_t n = (size_t)B * S;
      hipLaunchKernelGGL(JoinerFillKernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 1024)), dim3(256), 0,
                         static_cast<hipStream_t>(stream), (float *)px, n, -__builtin_huge_valf());
      return LaunchStatus();
    }
    return K2AMD_OK;
  }
  if (!am || !lm || !ranges || !weight || !px || !py || !normalizers || (!symbols && S > 0))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (workspace == nullptr ||
      workspace_bytes < k2amd_rnnt_joiner_pruned_forward_workspace_bytes(B, S, T, R, C, D, precision))
    return K2AMD_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool bf = precision == K2AMD_JOINER_BF16;
  JoinerArgs a = MakeArgs((const float *)am, (const float *)lm, ranges, (const float *)bias, symbols,
                          boundary, B, S, T, R, C, D, termination_symbol, rnnt_type, 64, workspace,
                          precision);
  a.px = (float *)px; a.py = (float *)py; a.norm = (float *)normalizers;
  return bf ? ForwardImpl<Bf16, 2>((const float *)weight, a, hat, st)
            : ForwardImpl<F32, 2>((const float *)weight, a, hat, st);
}

static int JoinerBackwardEntry(const void *am, const void *lm, const int64_t *ranges,
                               const void *weight, const void *bias, const int64_t *symbols,
                               const int64_t *boundary, const void *normalizers,
                               const void *px_grad, const void *py_grad, const void *seq_scale,
                               void *am_grad, void *lm_grad, void *weight_grad, void *bias_grad,
                               int B, int S, int T, int R, int C, int D, int termination_symbol,
                               int rnnt_type, int precision, bool hat, void *workspace,
                               size_t workspace_bytes, void *stream) {
  if (!JoinerShapeOk(B, S, T, R, C, D)) return K2AMD_ERR_UNSUPPORTED;
  if (hat && C < 2) return K2AMD_ERR_INVALID_ARGUMENT;
  if (precision != K2AMD_JOINER_F32 && precision != K2AMD_JOINER_BF16) return K2AMD_ERR_INVALID_ARGUMENT;
  if (rnnt_type != K2AMD_REGULAR && rnnt_type != K2AMD_MODIFIED && rnnt_type != K2AMD_CONSTRAINED)
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (!weight_grad || (!lm_grad && B > 0)) return K2AMD_ERR_INVALID_ARGUMENT;
  if (B > 0 && T > 0 &&
      (!am || !lm || !ranges || !weight || !normalizers || !px_grad || !py_grad || !am_grad ||
       (!symbols && S > 0)))
    return K2AMD_ERR_INVALID_ARGUMENT;
  if (workspace == nullptr ||
      workspace_bytes < k2amd_rnnt_joiner_pruned_workspace_bytes(B, S, T, R, C, D, precision))
    return K2AMD_ERR_WORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool bf = precision == K2AMD_JOINER_BF16;
  JoinerArgs a = MakeArgs((const float *)am, (const float *)lm, ranges, (const float *)bias, symbols,
                          boundary, B, S, T, R, C, D, termination_symbol, rnnt_type, 32, workspace,
                          precision);
  a.norm = (float *)const_cast<void *>(normalizers);
  a.am_grad = (float *)am_grad; a.lm_grad = (float *)lm_grad;
  a.weight_grad = (float *)weight_grad; a.bias_grad = (float *)bias_grad;
  return bf ? BackwardImpl<Bf16>((const float *)weight, a, (const float *)px_grad,
                                 (const float *)py_grad, (const float *)seq_scale, hat, st)
            : BackwardImpl<F32>((const float *)weight, a, (const float *)px_grad,
                                (const float *)py_grad, (const float *)seq_scale, hat, st);
}

extern "C" {

int k2amd_rnnt_joiner_pruned_forward(const void *am, const void *lm, const int64_t *ranges,
                                     const void *weight, const void *bias, const int64_t *symbols,
                                     const int64_t *boundary, void *px, void *py, void *normalizers,
                                     int B, int S, int T, int R, int C, int D, int termination_symbol,
                                     int rnnt_type, int precision, void *workspace,
                                     size_t workspace_bytes, void *stream) {
  return JoinerForwardEntry(am, lm, ranges, weight, bias, symbols, boundary, px, py, normalizers, B, S, T, R, C, D,
                            termination_symbol, rnnt_type, precision, false, workspace, workspace_bytes, stream);
}

int k2amd_rnnt_joiner_pruned_backward(const void *am, const void *lm, const int64_t *ranges,
                                      const void *weight, const void *bias, const int64_t *symbols,
                                      const int64_t *boundary, const void *normalizers,
                                      const void *px_grad, const void *py_grad, const void *seq_scale,
                                      void *am_grad, void *lm_grad, void *weight_grad, void *bias_grad,
                                      int B, int S, int T, int R, int C, int D, int termination_symbol,
                                      int rnnt_type, int precision, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  return JoinerBackwardEntry(am, lm, ranges, weight, bias, symbols, boundary, normalizers, px_grad, py_grad,
                             seq_scale, am_grad, lm_grad, weight_grad, bias_grad, B, S, T, R, C, D,
                             termination_symbol, rnnt_type, precision, false, workspace, workspace_bytes, stream);
}

int k2amd_rnnt_joiner_hat_pruned_forward(const void *am, const void *lm, const int64_t *ranges,
                                         const void *weight, const void *bias, const int64_t *symbols,
                                         const int64_t *boundary, void *px, void *py, void *normalizers,
                                         int B, int S, int T, int R, int C, int D, int rnnt_type,
                                         int precision, void *workspace, size_t workspace_bytes, void *stream) {
  return JoinerForwardEntry(am, lm, ranges, weight, bias, symbols, boundary, px, py, normalizers, B, S, T, R, C, D,
                            0, rnnt_type, precision, true, workspace, workspace_bytes, stream);
}

int k2amd_rnnt_joiner_hat_pruned_backward(const void *am, const void *lm, const int64_t *ranges,
                                          const void *weight, const void *bias, const int64_t *symbols,
                                          const int64_t *boundary, const void *normalizers,
                                          const void *px_grad, const void *py_grad, const void *seq_scale,
                                          void *am_grad, void *lm_grad, void *weight_grad, void *bias_grad,
                                          int B, int S, int T, int R, int C, int D, int rnnt_type, int precision,
                                          void *workspace, size_t workspace_bytes, void *stream) {
  return JoinerBackwardEntry(am, lm, ranges, weight, bias, symbols, boundary, normalizers, px_grad, py_grad,
                             seq_scale, am_grad, lm_grad, weight_grad, bias_grad, B, S, T, R, C, D, 0, rnnt_type,
                             precision, true, workspace, workspace_bytes, stream);
}

}  // extern "C"
