// Runs, over the thread stand-in of hip/hip_runtime.h, the forms of the exact recursion kernels
// (k2_amd/csrc/mi_generic.hip) and of the prune ranges' finishing kernel (k2_amd/csrc/prune.hip)
// that keep no rows in LDS, and the kernel of get_rnnt_prune_ranges_deprecated, on random inputs in
// heap buffers of exactly the documented sizes.  Built with -fsanitize=thread (every work-item a
// thread: a value read back from p, px_grad, py_grad or ranges must have been stored before the
// workgroup's barrier in between) or -fsanitize=address,undefined.  It checks no values
// (tests/test_cpu_build_kernels.py does).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "common.h"
#include "mi_internal.h"

namespace {

template <typename T>
int Recursion(int B, int S, int Tn, int modified, unsigned seed) {
  std::mt19937 rng(seed);
  std::normal_distribution<double> normal(-1.0, 1.0);
  const int T1 = modified ? Tn : Tn + 1;
  std::vector<T> px((size_t)B * S * T1), py((size_t)B * (S + 1) * Tn);
  for (T &v : px) v = (T)normal(rng);
  for (T &v : py) v = (T)normal(rng);
  std::vector<int64_t> boundary(4 * (size_t)B);
  for (int b = 0; b < B; ++b) {
    boundary[4 * b] = std::min(b % 2, S);
    boundary[4 * b + 1] = std::min(b % 3, Tn);
    boundary[4 * b + 2] = std::max(S - b % 2, (int)boundary[4 * b]);
    boundary[4 * b + 3] = std::max(Tn - b % 2, (int)boundary[4 * b + 1]);
  }
  std::vector<T> p((size_t)B * (S + 1) * (Tn + 1)), ans(B), seeds(B, (T)1), px_grad(px.size()), py_grad(py.size());
  int status = k2amd::MiForwardGeneric<T>(px.data(), py.data(), boundary.data(), p.data(), ans.data(), B, S, Tn,
                                          modified, nullptr);
  if (status != K2AMD_OK) return status;
  return k2amd::MiBackwardGeneric<T>(px.data(), p.data(), boundary.data(), seeds.data(), px_grad.data(),
                                     py_grad.data(), B, S, Tn, modified, 1, nullptr);
}

template <typename T>
int Ranges(int B, int S, int Tn, int modified, int R, bool deprecated, unsigned seed) {
  std::mt19937 rng(seed);
  std::uniform_real_distribution<double> uniform(0.0, 1.0);
  const int T1 = modified ? Tn : Tn + 1;
  std::vector<T> px_grad((size_t)B * S * T1), py_grad((size_t)B * (S + 1) * Tn);
  for (T &v : px_grad) v = (T)uniform(rng);
  for (T &v : py_grad) v = (T)uniform(rng);
  std::vector<int64_t> boundary(4 * (size_t)B, 0);
  for (int b = 0; b < B; ++b) {
    boundary[4 * b + 2] = std::max(S - b % 2, 0);
    boundary[4 * b + 3] = std::max(Tn - b % 3, 0);
  }
  std::vector<int64_t> ranges((size_t)B * Tn * R);
  const int dtype = sizeof(T) == 4 ? K2AMD_F32 : K2AMD_F64;
  return deprecated ? k2amd_rnnt_prune_ranges_deprecated(px_grad.data(), py_grad.data(), boundary.data(),
                                                         ranges.data(), B, S, Tn, modified, R, dtype, nullptr)
                    : k2amd_rnnt_prune_ranges(px_grad.data(), py_grad.data(), boundary.data(), ranges.data(), B, S,
                                              Tn, modified, R, dtype, nullptr);
}

}  // namespace

int main() {
  setenv("K2AMD_MI_GENERIC_ROWS", "global", 1);
  setenv("K2AMD_PRUNE_SCAN_ROWS", "global", 1);
  const int shapes[][3] = {{2, 5, 9}, {3, 40, 41}, {1, 1, 1}, {2, 300, 7}, {2, 7, 300}};
  unsigned seed = 1;
  for (const auto &s : shapes)
    for (int modified = 0; modified < 2; ++modified) {
      if (modified && s[2] < s[1]) continue;
      if (Recursion<float>(s[0], s[1], s[2], modified, seed++) != K2AMD_OK) return 1;
      if (Recursion<double>(s[0], s[1], s[2], modified, seed++) != K2AMD_OK) return 2;
      for (int R : {1, 2, 5}) {
        if (R > s[1] + 1 || (!modified && R < 2)) continue;
        if (Ranges<float>(s[0], s[1], s[2], modified, R, false, seed++) != K2AMD_OK) return 3;
        if (Ranges<double>(s[0], s[1], s[2], modified, R, true, seed++) != K2AMD_OK) return 4;
        if (Ranges<float>(s[0], s[1], s[2], modified, R, true, seed++) != K2AMD_OK) return 5;
      }
    }
  printf("all shapes done\n");
  return 0;
}
