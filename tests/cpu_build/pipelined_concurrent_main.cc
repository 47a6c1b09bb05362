// The pipelined fp32 mutual-information kernels (the host copy of k2_amd/csrc/mi_fast.hip, linked
// in) with workgroups that really overlap: every workgroup of a launch runs in a child process of
// its own (hip_threads::concurrent_workgroups), a few at a time, and everything they hand to each
// other (the edge words between chunks, the cut's words and counters, the log-derivatives of the
// single launch, the tickets) goes through memory that the processes share.  What a launch
// computes does not depend on how its workgroups interleave: every word handed over is waited for,
// and the arithmetic is the same in any order.  So each route is run once with the workgroups one
// after the other and then `repeats` times with them overlapping, and every output has to come
// out with the same bits, the workspace clean and no wait expired.
//
//   program rounds repeats window seed
//
// Random small shapes (one to three chunks, one to four blocks, boxes, both lattice types), the
// pair of launches with the log-derivative tensor, the single launch, and the fp64 pair
// (k2_amd/csrc/mi_wave.hip: one wavefront per chunk, the same hand-over between chunks).
#include <sys/mman.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/k2_amd.h"
#include "hip/hip_runtime.h"

namespace {

template <typename T>
T *Shared(size_t n) {
  void *m = mmap(nullptr, std::max<size_t>(n, 1) * sizeof(T), PROT_READ | PROT_WRITE, MAP_SHARED | MAP_ANONYMOUS, -1, 0);
  if (m == MAP_FAILED) abort();
  return static_cast<T *>(m);
}
template <typename T>
void Release(T *p, size_t n) { munmap(p, std::max<size_t>(n, 1) * sizeof(T)); }

struct Outputs {
  float *p, *log_deriv, *ans, *seed, *px_grad, *py_grad;
};

bool Clean(const unsigned *ws, size_t words) {
  for (size_t i = 0; i < 3; ++i)
    if (ws[i] != 0) return false;
  for (size_t i = 64; i < words; ++i)
    if (ws[i] != 0x7fc5a5a5u) return false;
  return true;
}

template <typename T>
bool SameBits(const char *what, const T *a, const T *b, size_t n) {
  if (memcmp(a, b, n * sizeof(T)) == 0) return true;
  for (size_t i = 0; i < n; ++i)
    if (memcmp(a + i, b + i, sizeof(T)) != 0) {
      printf("%s differs at %zu: %.17g against %.17g\n", what, i, (double)a[i], (double)b[i]);
      break;
    }
  return false;
}

// the fp64 pair, in order and `repeats` times overlapping
bool DoublePair(const float *px32, const float *py32, const int64_t *boundary, int B, int S, int T, int modified,
                size_t nx, size_t ny, size_t np, int repeats, int window) {
  const size_t ws_bytes = k2amd_mi_workspace_bytes(B, S, T, modified, K2AMD_F64);
  if (ws_bytes == 0) return true;  // (not served: the exact kernels have no hand-over)
  double *px = Shared<double>(nx), *py = Shared<double>(ny);
  for (size_t i = 0; i < nx; ++i) px[i] = px32[i];
  for (size_t i = 0; i < ny; ++i) py[i] = py32[i];
  unsigned *ws = Shared<unsigned>(ws_bytes / 4);
  bool ok = k2amd_mi_workspace_init(ws, ws_bytes, nullptr) == K2AMD_OK;
  double *p[2], *ans[2], *seed[2], *gx[2], *gy[2];
  for (int i = 0; i < 2; ++i) {
    p[i] = Shared<double>(np); ans[i] = Shared<double>(B); seed[i] = Shared<double>(B);
    gx[i] = Shared<double>(nx); gy[i] = Shared<double>(ny);
  }
  for (int run = 0; ok && run <= repeats; ++run) {
    const int o = run == 0 ? 0 : 1;
    hip_threads::concurrent_workgroups = run == 0 ? 0 : window;
    memset(p[o], 0, np * 8); memset(gx[o], 0, nx * 8); memset(gy[o], 0, ny * 8);
    for (int b = 0; b < B; ++b) { ans[o][b] = 0.0; seed[o][b] = 0.5 + 0.25 * b; }
    int status = k2amd_mi_forward(px, py, boundary, p[o], ans[o], B, S, T, modified, K2AMD_F64, ws, ws_bytes, nullptr);
    if (status == K2AMD_OK)
      status = k2amd_mi_backward(px, py, boundary, p[o], seed[o], gx[o], gy[o], B, S, T, modified, K2AMD_F64, 1, ws,
                                 ws_bytes, nullptr);
    hip_threads::concurrent_workgroups = 0;
    if (status == K2AMD_OK) status = k2amd_mi_workspace_status(ws, nullptr);
    ok = status == K2AMD_OK && Clean(ws, ws_bytes / 4);
    if (!ok) printf("fp64 pair run %d: status %d or workspace not clean\n", run, status);
    if (ok && run > 0) {
      ok = SameBits("ans", ans[0], ans[1], B) && SameBits("ans_grad", seed[0], seed[1], B) && SameBits("p", p[0], p[1], np) &&
           SameBits("px_grad", gx[0], gx[1], nx) && SameBits("py_grad", gy[0], gy[1], ny);
      if (!ok) printf("fp64 pair run %d: not the bits of the run in order\n", run);
    }
  }
  for (int i = 0; i < 2; ++i) {
    Release(p[i], np); Release(ans[i], B); Release(seed[i], B); Release(gx[i], nx); Release(gy[i], ny);
  }
  Release(ws, ws_bytes / 4); Release(px, nx); Release(py, ny);
  return ok;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc != 5) return 64;
  const int rounds = atoi(argv[1]), repeats = atoi(argv[2]), window = atoi(argv[3]);
  std::mt19937 rng((unsigned)atoi(argv[4]));
  for (int round = 0; round < rounds; ++round) {
    const int modified = rng() % 2, B = 1 + rng() % 3;
    const int S = 1 + rng() % 150;
    int T = 1 + rng() % 120;
    if (modified && T < S) T = S + rng() % 5;
    const int T1 = modified ? T : T + 1;
    const size_t nx = (size_t)B * S * T1, ny = (size_t)B * (S + 1) * T, np = (size_t)B * (S + 1) * (T + 1);
    float *px = Shared<float>(nx), *py = Shared<float>(ny);
    int64_t *boundary = Shared<int64_t>(4 * (size_t)B);
    std::normal_distribution<float> normal(-1.0f, 1.0f);
    for (size_t i = 0; i < nx; ++i) px[i] = normal(rng);
    for (size_t i = 0; i < ny; ++i) py[i] = normal(rng);
    for (int b = 0; b < B; ++b) {
      const int s0 = rng() % 3 ? 0 : rng() % (S + 1), t0 = rng() % 3 ? 0 : rng() % (T + 1);
      int s1 = rng() % 3 ? S : s0 + rng() % (S - s0 + 1), t1 = rng() % 3 ? T : t0 + rng() % (T - t0 + 1);
      boundary[4 * b] = s0; boundary[4 * b + 1] = t0; boundary[4 * b + 2] = s1; boundary[4 * b + 3] = t1;
    }
    const size_t ws_bytes = k2amd_mi_workspace_bytes(B, S, T, modified, K2AMD_F32);
    if (ws_bytes == 0) return 65;
    unsigned *ws = Shared<unsigned>(ws_bytes / 4);
    if (k2amd_mi_workspace_init(ws, ws_bytes, nullptr) != K2AMD_OK) return 66;
    const bool single = k2amd_mi_forward_backward_supported(B, S, T, modified, K2AMD_F32, 1) != 0;
    const size_t scratch_bytes = single ? k2amd_mi_forward_backward_scratch_bytes(B, S, T, modified, K2AMD_F32) : 0;
    float *scratch = Shared<float>(scratch_bytes / 4 + 1);
    Outputs out[2];
    for (Outputs &o : out)
      o = Outputs{Shared<float>(np), Shared<float>(np), Shared<float>(B), Shared<float>(B), Shared<float>(nx), Shared<float>(ny)};
    printf("round %d: modified=%d B=%d S=%d T=%d single=%d\n", round, modified, B, S, T, (int)single);
    fflush(stdout);
    for (int route = 0; route < (single ? 2 : 1); ++route) {
      for (int run = 0; run <= repeats; ++run) {
        Outputs &o = out[run == 0 ? 0 : 1];
        hip_threads::concurrent_workgroups = run == 0 ? 0 : window;
        memset(o.p, 0, np * 4); memset(o.log_deriv, 0, np * 4); memset(o.px_grad, 0, nx * 4); memset(o.py_grad, 0, ny * 4);
        for (int b = 0; b < B; ++b) { o.ans[b] = 0.0f; o.seed[b] = 0.5f + 0.25f * b; }
        int status;
        if (route == 0) {
          status = k2amd_mi_forward_keep(px, py, boundary, o.p, o.ans, o.log_deriv, B, S, T, modified, K2AMD_F32, ws,
                                         ws_bytes, nullptr);
          if (status == K2AMD_OK)
            status = k2amd_mi_backward_kept(px, py, boundary, o.p, o.log_deriv, o.seed, o.px_grad, o.py_grad, B, S, T,
                                            modified, K2AMD_F32, 1, ws, ws_bytes, nullptr);
        } else {
          status = k2amd_mi_forward_backward(px, py, boundary, o.ans, scratch, scratch_bytes, o.seed, o.px_grad,
                                             o.py_grad, B, S, T, modified, K2AMD_F32, 1, ws, ws_bytes, nullptr);
        }
        hip_threads::concurrent_workgroups = 0;
        if (status == K2AMD_OK) status = k2amd_mi_workspace_status(ws, nullptr);
        if (status != K2AMD_OK) { printf("route %d run %d: status %d\n", route, run, status); return 1; }
        if (!Clean(ws, ws_bytes / 4)) { printf("route %d run %d: workspace not clean\n", route, run); return 1; }
        if (run == 0) continue;
        bool same = SameBits("ans", out[0].ans, out[1].ans, B) && SameBits("ans_grad", out[0].seed, out[1].seed, B) &&
                    SameBits("px_grad", out[0].px_grad, out[1].px_grad, nx) &&
                    SameBits("py_grad", out[0].py_grad, out[1].py_grad, ny);
        if (route == 0) same = same && SameBits("p", out[0].p, out[1].p, np);
        if (!same) { printf("route %d run %d: not the bits of the run in order\n", route, run); return 1; }
      }
    }
    if (!DoublePair(px, py, boundary, B, S, T, modified, nx, ny, np, repeats, window)) return 1;
    for (Outputs &o : out) {
      Release(o.p, np); Release(o.log_deriv, np); Release(o.ans, B); Release(o.seed, B); Release(o.px_grad, nx); Release(o.py_grad, ny);
    }
    Release(scratch, scratch_bytes / 4 + 1); Release(ws, ws_bytes / 4); Release(boundary, 4 * (size_t)B);
    Release(px, nx); Release(py, ny);
  }
  printf("all rounds done\n");
  return 0;
}
