// Runs the smoothed builder's kernels (k2_amd/csrc/rnnt_smoothed.hip, compiled into this program
// over the thread stand-in of hip/hip_runtime.h) on random inputs in heap buffers of exactly the
// documented sizes.  Built with -fsanitize=address,undefined: an access outside a buffer or an
// LDS array ends the program.  It checks no values (tests/test_cpu_build_smoothed.py does).
#include "../../k2_amd/csrc/rnnt_smoothed.hip"

#include <cstdio>
#include <random>

namespace {

template <typename T>
std::unique_ptr<T[]> Random(size_t n, std::mt19937 &rng, double lo, double hi) {
  std::unique_ptr<T[]> a(new T[n]);
  std::uniform_real_distribution<double> d(lo, hi);
  for (size_t i = 0; i < n; ++i) a[i] = (T)d(rng);
  return a;
}

template <typename T>
int RunShape(int B, int S, int Tn, int C, int rnnt_type, bool with_boundary, bool odd_symbols, unsigned seed) {
  std::mt19937 rng(seed);
  const int dtype = sizeof(T) == 4 ? K2AMD_F32 : K2AMD_F64;
  const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
  const size_t lm_n = (size_t)B * (S + 1) * C, am_n = (size_t)B * Tn * C;
  const size_t px_n = (size_t)B * S * T1, py_n = (size_t)B * (S + 1) * Tn;
  auto lm = Random<T>(lm_n, rng, -2, 2), am = Random<T>(am_n, rng, -2, 2);
  auto lm_probs = Random<T>(lm_n, rng, 0.01, 1), am_probs = Random<T>(am_n, rng, 0.01, 1);
  auto lm_max = Random<T>((size_t)B * (S + 1), rng, 0, 2), am_max = Random<T>((size_t)B * Tn, rng, 0, 2);
  auto px_joint = Random<T>(px_n, rng, -5, 0), py_joint = Random<T>(py_n, rng, -5, 0);
  std::unique_ptr<int64_t[]> symbols(new int64_t[(size_t)B * S]);
  for (size_t i = 0; i < (size_t)B * S; ++i) symbols[i] = rng() % C;
  if (odd_symbols)  // outside the vocabulary: such an edge is -inf and takes no part in any sum
    for (size_t i = 0; i < (size_t)B * S; i += 3) symbols[i] = (i % 2) ? -1 : C + 5;
  std::unique_ptr<int64_t[]> boundary(new int64_t[(size_t)B * 4]);
  for (int b = 0; b < B; ++b) {
    boundary[4 * b] = 0; boundary[4 * b + 1] = 0;
    boundary[4 * b + 2] = S - (S > 0 ? (int)(rng() % 2) : 0);
    boundary[4 * b + 3] = Tn - (Tn > 0 ? (int)(rng() % 2) : 0);
  }
  const int64_t *bd = with_boundary ? boundary.get() : nullptr;
  std::unique_ptr<T[]> px(new T[px_n]), py(new T[py_n]), lm_norm(new T[(size_t)B * (S + 1)]),
      am_norm(new T[(size_t)B * Tn]), unigram(new T[2 * (size_t)C]);
  const size_t scratch_n = k2amd_rnnt_smoothed_scratch_elements(B, S, Tn, C);
  std::unique_ptr<T[]> scratch(new T[scratch_n]);
  int status = k2amd_rnnt_smoothed_forward(lm.get(), am.get(), symbols.get(), bd, lm_probs.get(), am_probs.get(),
                                           lm_max.get(), am_max.get(), px_joint.get(), py_joint.get(), px.get(),
                                           py.get(), lm_norm.get(), am_norm.get(), unigram.get(), scratch.get(),
                                           scratch_n, 0.25, 0.1, B, S, Tn, C, C - 1, rnnt_type, dtype, nullptr);
  if (status != K2AMD_OK) return status;
  auto px_grad = Random<T>(px_n, rng, 0, 1), py_grad = Random<T>(py_n, rng, 0, 1);
  auto seq_scale = Random<T>((size_t)B, rng, 0.5, 1.5);
  auto lm_grad = Random<T>(lm_n, rng, -1, 1), am_grad = Random<T>(am_n, rng, -1, 1);
  return k2amd_rnnt_smoothed_backward(px_grad.get(), py_grad.get(), seed % 2 ? seq_scale.get() : nullptr,
                                      symbols.get(), bd, lm_probs.get(), am_probs.get(), lm_max.get(),
                                      am_max.get(), lm_norm.get(), am_norm.get(), unigram.get(), lm_grad.get(),
                                      am_grad.get(), scratch.get(), scratch_n, 0.25, 0.1, B, S, Tn, C, C - 1,
                                      rnnt_type, dtype, nullptr);
}

}  // namespace

int main() {
  const int shapes[][4] = {  // B, S, T, C
      {1, 1, 1, 1},  {1, 0, 1, 2},  {2, 3, 0, 5},  {3, 6, 11, 70}, {1, 16, 17, 64},
      {2, 5, 5, 65}, {1, 70, 75, 3}, {17, 0, 3, 7}, {2, 15, 16, 129},
  };
  unsigned seed = 1;
  int shape_index = 0;
  for (const auto &sh : shapes) {
    ++shape_index;
    for (int rnnt_type = 0; rnnt_type < 3; ++rnnt_type)
      {
        if (rnnt_type != K2AMD_REGULAR && (shape_index + rnnt_type) % 2 != 0) continue;  // every other shape
        if (rnnt_type != K2AMD_REGULAR && sh[2] < sh[1]) continue;
        const int variant = (int)(seed % 4);  // boundary or not, symbols outside the vocabulary or not
        const bool with_boundary = variant & 1, odd_symbols = variant & 2;
        int status = (seed & 2) ? RunShape<float>(sh[0], sh[1], sh[2], sh[3], rnnt_type, with_boundary, odd_symbols, seed)
                                : RunShape<double>(sh[0], sh[1], sh[2], sh[3], rnnt_type, with_boundary, odd_symbols, seed);
        if (status != K2AMD_OK) {
          std::printf("status %d at B=%d S=%d T=%d C=%d type %d variant %d\n", status, sh[0], sh[1], sh[2], sh[3],
                      rnnt_type, variant);
          return 1;
        }
        ++seed;
      }
  }
  std::printf("all shapes done (%u runs)\n", seed - 1);
  return 0;
}
