// A stand-in for <hip/hip_runtime.h> that runs HIP kernels on host threads, for tests only: the
// same kernel source is compiled with g++ and every launch runs its workgroups one after the
// other, each workgroup's work-items as threads of their own, so that barriers and wavefront
// exchanges keep their meaning, and a host sanitizer or a CPU debugger sees the kernels' indexing.
//
// What it has: launches with static and dynamic LDS, __syncthreads, the __shfl family, atomics
// (also the agent-scope builtins), vector types, __half as storage, and of the gfx9 builtins
// readlane / readfirstlane, the DPP moves that the kernels use (quad permutations, mirrored rows,
// the two whole-wavefront shifts), the matrix instructions v_mfma_f32_32x32x2_f32 and
// v_mfma_f32_32x32x16_bf16 (from their documented operand layouts), exp2 / log2 / rcp,
// wave_barrier and fences at wavefront scope (real barriers here: the lanes are free-running
// threads, not in lockstep), s_barrier, s_sleep, and no-ops for other fences and scheduling hints;
// helpers that do what three instructions do which the kernels spell in assembly (the host build
// compiles copies of those sources with calls to the helpers in the assembly's place).  What it
// does not have: inline assembly, other DPP controls, bfloat16 arithmetic.  Workgroups do not
// overlap unless hip_threads::concurrent_workgroups asks for it (then every workgroup is a child
// process): a kernel whose workgroups wait for one another must only ever wait for workgroups that
// started earlier, as on the device, where a later one may not be resident yet.  Slow by design:
// sizes stay small.
#ifndef K2_AMD_TESTS_CPU_BUILD_HIP_RUNTIME_H_
#define K2_AMD_TESTS_CPU_BUILD_HIP_RUNTIME_H_

#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <sys/wait.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <barrier>
#include <cmath>
#include <memory>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static
// dynamic LDS, as HIP spells it
#define HIP_DYNAMIC_SHARED(type, var) type *var = reinterpret_cast<type *>(hip_threads::state().dynamic_lds);

typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
typedef void *hipStream_t;
inline hipError_t hipGetLastError() { return hipSuccess; }
// "device" memory is the host's; a launch has finished when the call returns
#define __align__(n) alignas(n)
#define HIP_SYMBOL(x) (&(x))
enum hipMemcpyKind { hipMemcpyHostToHost, hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice };
inline hipError_t hipGetDevice(int *device) { *device = 0; return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void **address, const void *symbol) {
  *address = const_cast<void *>(symbol);
  return hipSuccess;
}
inline hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind, hipStream_t) {
  memcpy(dst, src, bytes);
  return hipSuccess;
}
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

namespace hip_threads {

constexpr int kWaveSize = 64;

struct Wave {
  std::unique_ptr<std::barrier<>> barrier;
  int lanes;
  // one exchange value per lane, two sets used in turn: a lane that is already writing for the
  // next exchange cannot disturb one that still reads the last (each exchange has a barrier, so
  // no lane is ever two exchanges ahead of another)
  alignas(8) unsigned char slot[2][kWaveSize][8];
  float matrix_a[2][kWaveSize], matrix_b[2][kWaveSize];  // the operands of a matrix instruction, likewise
  float matrix_a8[2][kWaveSize][8], matrix_b8[2][kWaveSize][8];
};

struct State {
  unsigned char *dynamic_lds = nullptr;
  std::barrier<> *block_barrier = nullptr;
  std::vector<Wave> *waves = nullptr;
};

inline State &state() {
  static State s;
  return s;
}

struct Index {
  unsigned x, y, z;
};
inline thread_local Index thread_idx, block_idx;
inline thread_local int flat_thread;
inline thread_local unsigned exchanges;  // this work-item's count of wavefront exchanges in the workgroup
inline Index block_dim, grid_dim;

inline Wave &my_wave() { return (*state().waves)[flat_thread / kWaveSize]; }

template <typename T>
inline T exchange(T v, int src_lane) {
  static_assert(sizeof(T) <= 8, "");
  Wave &w = my_wave();
  const int lane = flat_thread % kWaveSize;
  const unsigned set = exchanges++ & 1;
  memcpy(w.slot[set][lane], &v, sizeof(T));
  w.barrier->arrive_and_wait();
  T r = v;  // a source outside the wavefront gives the lane's own value back; kernels must not rely on it
  if (src_lane >= 0 && src_lane < w.lanes) memcpy(&r, w.slot[set][src_lane], sizeof(T));
  return r;
}

// 0: the workgroups of a launch run one after the other in this process.  n > 0: every workgroup
// runs in a child process of its own (its threads, its own copy of the kernel's static LDS
// variables), n of them at a time, started in the order of their indices: workgroups then really
// overlap, as on the device, and what they hand to each other goes through whatever memory the
// caller has mapped as shared between processes (every buffer a kernel writes has to be; the
// kernels' arguments are copied at the fork).  For tests of what workgroups say to each other.
inline int concurrent_workgroups = 0;

template <typename Kernel, typename... Args>
void run_workgroups(Kernel kernel, dim3 grid, dim3 block, size_t dynamic_lds_bytes, size_t first, size_t last,
                    Args... args) {
  const int threads = (int)(block.x * block.y * block.z);
  // exactly the bytes asked for, on the heap: a sanitizer sees an access beyond them
  std::unique_ptr<unsigned char[]> lds(new unsigned char[std::max<size_t>(dynamic_lds_bytes, 1)]);
  state().dynamic_lds = lds.get();
  // One set of threads for all of them.  A work-item that leaves the kernel drops out of its
  // wavefront's and its workgroup's barriers, as exited lanes and wavefronts do on the hardware, so
  // those barriers are made anew for every workgroup.
  std::unique_ptr<std::barrier<>> block_barrier;
  std::vector<Wave> waves((threads + kWaveSize - 1) / kWaveSize);
  auto fresh = [&] {
    block_barrier.reset(new std::barrier<>(threads));
    for (size_t w = 0; w < waves.size(); ++w) {
      waves[w].lanes = std::min(kWaveSize, threads - (int)w * kWaveSize);
      waves[w].barrier.reset(new std::barrier<>(waves[w].lanes));
    }
    state().block_barrier = block_barrier.get();
  };
  fresh();
  state().waves = &waves;
  auto renew = [&]() noexcept { fresh(); };  // runs once all have arrived, before any goes on
  std::barrier<decltype(renew)> between(threads, renew);
  std::vector<std::thread> pool;
  pool.reserve(threads);
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&, t] {
      flat_thread = t;
      thread_idx = {t % block.x, (t / block.x) % block.y, t / (block.x * block.y)};
      for (size_t k = first; k < last; ++k) {
        exchanges = 0;
        block_idx = {(unsigned)(k % grid.x), (unsigned)((k / grid.x) % grid.y), (unsigned)(k / ((size_t)grid.x * grid.y))};
        kernel(args...);
        my_wave().barrier->arrive_and_drop();
        state().block_barrier->arrive_and_drop();
        between.arrive_and_wait();
      }
    });
  for (auto &th : pool) th.join();
  state().dynamic_lds = nullptr;
  state().block_barrier = nullptr;
  state().waves = nullptr;
}

template <typename Kernel, typename... Args>
void launch(Kernel kernel, dim3 grid, dim3 block, size_t dynamic_lds_bytes, Args... args) {
  const int threads = (int)(block.x * block.y * block.z);
  const size_t blocks = (size_t)grid.x * grid.y * grid.z;
  if (threads == 0 || blocks == 0) return;
  block_dim = {block.x, block.y, block.z};
  grid_dim = {grid.x, grid.y, grid.z};
  if (concurrent_workgroups <= 0) {
    run_workgroups(kernel, grid, block, dynamic_lds_bytes, 0, blocks, args...);
    return;
  }
  size_t started = 0, alive = 0;
  while (started < blocks || alive > 0) {
    while (started < blocks && alive < (size_t)concurrent_workgroups) {
      const pid_t child = fork();
      if (child < 0) abort();
      if (child == 0) {
        run_workgroups(kernel, grid, block, dynamic_lds_bytes, started, started + 1, args...);
        _exit(0);
      }
      ++started;
      ++alive;
    }
    int status = 0;
    if (wait(&status) < 0 || !WIFEXITED(status) || WEXITSTATUS(status) != 0) abort();
    --alive;
  }
}

}  // namespace hip_threads

#define threadIdx hip_threads::thread_idx
#define blockIdx hip_threads::block_idx
#define blockDim hip_threads::block_dim
#define gridDim hip_threads::grid_dim

#define hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, ...) \
  hip_threads::launch(kernel, grid, block, lds_bytes, __VA_ARGS__)

inline void __syncthreads() { hip_threads::state().block_barrier->arrive_and_wait(); }

template <typename T>
inline T __shfl_xor(T v, int mask, int width = hip_threads::kWaveSize) {
  (void)width;
  return hip_threads::exchange(v, (hip_threads::flat_thread % hip_threads::kWaveSize) ^ mask);
}
template <typename T>
inline T __shfl(T v, int src_lane, int width = hip_threads::kWaveSize) {
  (void)width;
  return hip_threads::exchange(v, src_lane);
}
// ---- what the fp32 matrix-core products of rnnt_simple.hip use --------------------------------
// clang's ext_vector_type for FLOAT vectors (the only ones in the files of the host build)
#define ext_vector_type(n) vector_size(4 * (n))
// A fence orders one thread's accesses, which the sequentially consistent atomics and the barriers
// of this stand-in do already; at wavefront scope the kernels use it where the lanes of one
// wavefront hand values to each other through LDS and rely on running in lockstep, so here it is
// a barrier over the wavefront (every live lane has to reach it, as it does on the hardware).
inline void hip_threads_fence(int, const char *scope, const char * = nullptr);
#define __builtin_amdgcn_fence(...) hip_threads_fence(__VA_ARGS__)
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)
inline void __builtin_amdgcn_s_barrier() { __syncthreads(); }

// v_mfma_f32_32x32x2_f32: D = A (32 x 2) * B (2 x 32) + C over the wavefront.  Lane l supplies
// A[l % 32][l / 32] and B[l / 32][l % 32] and holds, in element v of its 16, D[i][l % 32] with
// i = 8 (v / 4) + 4 (l / 32) + v % 4.
typedef float hip_threads_float16 __attribute__((vector_size(64)));
inline hip_threads_float16 __builtin_amdgcn_mfma_f32_32x32x2f32(float a, float b, hip_threads_float16 c, int, int,
                                                               int) {
  hip_threads::Wave &w = hip_threads::my_wave();
  const int lane = hip_threads::flat_thread % hip_threads::kWaveSize;
  const unsigned set = hip_threads::exchanges++ & 1;
  w.matrix_a[set][lane] = a;
  w.matrix_b[set][lane] = b;
  w.barrier->arrive_and_wait();
  const int j = lane % 32;
  for (int v = 0; v < 16; ++v) {
    const int i = 8 * (v / 4) + 4 * (lane / 32) + v % 4;
    c[v] += w.matrix_a[set][i] * w.matrix_b[set][j] + w.matrix_a[set][i + 32] * w.matrix_b[set][j + 32];
  }
  return c;
}

// ---- what the fused joiner (joiner.hip) uses besides ------------------------------------------------
// bfloat16: eight of them as one 16-byte value, and the hardware's conversion (round to nearest
// even; NaN stays NaN).  The host compiler has no such type; the test's build replaces the two
// places of the source that spell it (tests/cpu_kernels.py).
struct hip_threads_bf16x8 { unsigned short v[8]; };
inline unsigned short hip_threads_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
  return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
// v_mfma_f32_32x32x16_bf16: as the fp32 one above with sixteen k per step: lane l supplies eight
// consecutive k of row / column l % 32, the lower half of the wavefront the first eight.
inline hip_threads_float16 __builtin_amdgcn_mfma_f32_32x32x16_bf16(hip_threads_bf16x8 a, hip_threads_bf16x8 b,
                                                                   hip_threads_float16 c, int, int, int) {
  hip_threads::Wave &w = hip_threads::my_wave();
  const int lane = hip_threads::flat_thread % hip_threads::kWaveSize;
  const unsigned set = hip_threads::exchanges++ & 1;
  for (int e = 0; e < 8; ++e) {
    uint32_t ua = (uint32_t)a.v[e] << 16, ub = (uint32_t)b.v[e] << 16;
    memcpy(&w.matrix_a8[set][lane][e], &ua, 4);
    memcpy(&w.matrix_b8[set][lane][e], &ub, 4);
  }
  w.barrier->arrive_and_wait();
  const int j = lane % 32;
  for (int v = 0; v < 16; ++v) {
    const int i = 8 * (v / 4) + 4 * (lane / 32) + v % 4;
    float sum = 0;
    for (int half = 0; half < 2; ++half)
      for (int e = 0; e < 8; ++e) sum += w.matrix_a8[set][i + 32 * half][e] * w.matrix_b8[set][j + 32 * half][e];
    c[v] += sum;
  }
  return c;
}
inline float __builtin_amdgcn_exp2f(float x) { return exp2f(x); }
inline float __builtin_amdgcn_logf(float x) { return log2f(x); }
inline void __builtin_amdgcn_s_setprio(int) {}
inline unsigned __float_as_uint(float f) { unsigned u; memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(unsigned u) { float f; memcpy(&f, &u, 4); return f; }
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount };
// (the compute units of the device that the library is written for: the single launch sizes its
// grid with it and the kernel selection compares with it)
inline hipError_t hipDeviceGetAttribute(int *value, hipDeviceAttribute_t, int) { *value = 256; return hipSuccess; }
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize };
inline hipError_t hipFuncSetAttribute(const void *, hipFuncAttribute, int) { return hipSuccess; }

// ---- what the fp64 wave kernels (mi_wave.hip) use ------------------------------------------------
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_load(address, order, scope) hip_threads::atomic_load(address)
#define __hip_atomic_store(address, value, order, scope) hip_threads::atomic_store(address, value)
#define __hip_atomic_fetch_add(address, value, order, scope) std::atomic_ref(*(address)).fetch_add(value)
namespace hip_threads {
template <typename T>
inline T atomic_load(T *address) { return std::atomic_ref<T>(*address).load(std::memory_order_seq_cst); }
template <typename T, typename V>
inline void atomic_store(T *address, V value) { std::atomic_ref<T>(*address).store((T)value, std::memory_order_seq_cst); }
}  // namespace hip_threads
// (a poll loop's pause; with workgroups in processes of their own the poller sleeps, so that the
// hundreds of threads of the workgroup it waits for get the cores, and a bounded wait of a million
// polls does not run out while they are still being scheduled)
inline void __builtin_amdgcn_s_sleep(int) {
  if (hip_threads::concurrent_workgroups > 0) usleep(20); else std::this_thread::yield();
}
inline float __builtin_amdgcn_rcpf(float x) { return 1.0f / x; }
template <typename T>
inline T __builtin_amdgcn_readlane(T v, int lane) { return hip_threads::exchange(v, lane); }
template <typename T>
inline T __builtin_amdgcn_readfirstlane(T v) { return hip_threads::exchange(v, 0); }  // (lane 0 is live wherever it is used)
// DPP moves: within quads (quad_perm), and over the whole wavefront wave_shr:1 (0x138: lane l
// takes lane l - 1, lane 0 keeps `old`) and wave_shl:1 (0x130: lane l takes lane l + 1, lane 63
// keeps `old`), mirrored rows; all rows and banks enabled, as the kernels ask for.  Other controls
// are not emulated.
inline int hip_threads_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  const int lane = hip_threads::flat_thread % hip_threads::kWaveSize;
  if (ctrl >= 0 && ctrl < 0x100) {  // quad_perm: lane 4 q + i takes lane 4 q + ((ctrl >> 2 i) & 3); always in range
    if (row_mask != 0xf || bank_mask != 0xf) abort();
    return hip_threads::exchange(src, (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3));
  }
  if (ctrl == 0x140 || ctrl == 0x141) {  // row_mirror, row_half_mirror: lane i of a row of 16 (8) takes lane 15 - i (7 - i)
    if (row_mask != 0xf || bank_mask != 0xf) abort();
    const int width = ctrl == 0x140 ? 16 : 8;
    return hip_threads::exchange(src, (lane & ~(width - 1)) | (width - 1 - (lane & (width - 1))));
  }
  if ((ctrl != 0x138 && ctrl != 0x130) || row_mask != 0xf || bank_mask != 0xf || bound_ctrl) abort();
  const int from = ctrl == 0x138 ? lane - 1 : lane + 1;
  const int got = hip_threads::exchange(src, std::min(std::max(from, 0), hip_threads::kWaveSize - 1));
  return from < 0 || from >= hip_threads::my_wave().lanes ? old : got;
}

template <typename T>  // int or unsigned
inline T __builtin_amdgcn_update_dpp(T old, T src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  static_assert(sizeof(T) == 4, "");
  return (T)hip_threads_update_dpp((int)old, (int)src, ctrl, row_mask, bank_mask, bound_ctrl);
}

// The two DPP instructions that the pipelined kernels spell in assembly, for the copy of
// mi_fast.hip that the host build compiles (tests/cpu_kernels.py puts these calls in the place of
// the assembly blocks):
//   v_add_f32_dpp inc, P, inc wave_shr:1   inc = P(lane - 1) + inc; lane 0 has no source lane and
//                                          is left alone
//   v_mul_f32_dpp t, G, t wave_shl:1       t = G(lane + 1) * t; lane 63 likewise
inline float hip_threads_add_from_lane_above(float P, float inc) {
  const int lane = hip_threads::flat_thread % hip_threads::kWaveSize;
  const float above = hip_threads::exchange(P, std::max(lane - 1, 0));
  return lane == 0 ? inc : above + inc;
}
inline float hip_threads_mul_from_lane_below(float G, float t) {
  const int lane = hip_threads::flat_thread % hip_threads::kWaveSize;
  const float below = hip_threads::exchange(G, std::min(lane + 1, hip_threads::kWaveSize - 1));
  return lane == hip_threads::kWaveSize - 1 ? t : below * t;
}
// buffer_load_dwordx4 ... offen through a raw buffer resource (words 0 and 1: the base address,
// word 2: the size in bytes): every dword is range-checked by itself and reads as 0 when any of
// its bytes lies at or beyond the size.
struct hip_threads_int4 { int x, y, z, w; };
struct hip_threads_float4 { float x, y, z, w; };
inline hip_threads_float4 hip_threads_buffer_load4(hip_threads_int4 resource, int byte_offset) {
  const unsigned long long base = (unsigned long long)(unsigned)resource.x | ((unsigned long long)(unsigned)resource.y << 32);
  const unsigned size = (unsigned)resource.z;
  float out[4];
  for (int i = 0; i < 4; ++i) {
    const unsigned long long at = (unsigned long long)(unsigned)byte_offset + 4ull * i;
    out[i] = 0.0f;
    if (at + 4 <= size) memcpy(&out[i], reinterpret_cast<const void *>(base + at), 4);
  }
  return {out[0], out[1], out[2], out[3]};
}

// On the hardware a scheduling fence that emits nothing (a wavefront's lanes run in lockstep);
// here the lanes are free-running threads, so it has to be a real barrier over the wavefront.
inline void __builtin_amdgcn_wave_barrier() { hip_threads::my_wave().barrier->arrive_and_wait(); }
// (HIP_THREADS_FENCES_ARE_NOT_BARRIERS: for the thread sanitizer's test of itself, which has to
// report the race that this barrier prevents)
inline void hip_threads_fence(int, const char *scope, const char *) {
  std::atomic_thread_fence(std::memory_order_seq_cst);
#ifndef HIP_THREADS_FENCES_ARE_NOT_BARRIERS
  if (strcmp(scope, "wavefront") == 0) __builtin_amdgcn_wave_barrier();
#else
  (void)scope;
#endif
}
inline int __any(int predicate) {
  int r = predicate != 0;
  for (int off = 32; off > 0; off >>= 1) r |= __shfl_xor(r, off);
  return r;
}

using std::max;
using std::min;

// ---- vector types (no alignment beyond the element's: host buffers need not be 16-byte aligned) --
struct float2 { float x, y; };
struct float4 { float x, y, z, w; };
struct double2 { double x, y; };
struct uint2 { unsigned x, y; };
struct uint4 { unsigned x, y, z, w; };
struct int2 { int x, y; };
struct int4 { int x, y, z, w; };
inline float2 make_float2(float x, float y) { return {x, y}; }
inline float4 make_float4(float x, float y, float z, float w) { return {x, y, z, w}; }
inline double2 make_double2(double x, double y) { return {x, y}; }
inline uint2 make_uint2(unsigned x, unsigned y) { return {x, y}; }
inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return {x, y, z, w}; }
inline int2 make_int2(int x, int y) { return {x, y}; }
inline int4 make_int4(int x, int y, int z, int w) { return {x, y, z, w}; }

// ---- atomics: work-items of one workgroup are threads, so these have to be real ----------------
template <typename T>
inline T atomicAdd(T *address, T value) { return std::atomic_ref<T>(*address).fetch_add(value); }
template <typename T>
inline T unsafeAtomicAdd(T *address, T value) { return atomicAdd(address, value); }
template <typename T>
inline T atomicMax(T *address, T value) {
  std::atomic_ref<T> a(*address);
  T old = a.load();
  while (old < value && !a.compare_exchange_weak(old, value)) {}
  return old;
}

inline float __expf(float x) { return expf(x); }
inline float __logf(float x) { return logf(x); }

// ---- IEEE half, as storage with a conversion (hip_fp16.h's __half) -----------------------------
struct __half { uint16_t bits; };
inline float __half2float(__half h) {
  const uint32_t sign = (uint32_t)(h.bits & 0x8000u) << 16, exponent = (h.bits >> 10) & 0x1fu, mantissa = h.bits & 0x3ffu;
  uint32_t u;
  if (exponent == 0) {
    if (mantissa == 0) {
      u = sign;
    } else {  // subnormal: value = mantissa * 2^-24
      float f = (float)mantissa * 5.9604644775390625e-8f;
      memcpy(&u, &f, 4);
      u |= sign;
    }
  } else if (exponent == 31) {
    u = sign | 0x7f800000u | (mantissa << 13);
  } else {
    u = sign | ((exponent + 112) << 23) | (mantissa << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

#endif  // K2_AMD_TESTS_CPU_BUILD_HIP_RUNTIME_H_
