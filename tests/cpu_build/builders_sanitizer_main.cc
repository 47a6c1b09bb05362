// Runs get_rnnt_logprobs' kernels (k2_amd/csrc/rnnt_simple.hip) and the fused joiner's (the host
// copy of k2_amd/csrc/joiner.hip, linked in) through the C-ABI, forward and backward, on random
// inputs in heap buffers of exactly the documented sizes.  It checks no values (the tests that
// load the host library do); it is the program that the sanitizers get to see:
//   -fsanitize=thread: the work-items are threads, ordered by the barriers of a workgroup and of
//     a wavefront and by atomics; two wavefronts that touch the same LDS or device word without
//     one of those between them are reported as a data race;
//   -fsanitize=address,undefined: an access outside a buffer or a workgroup's LDS ends it.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "../../include/k2_amd.h"

namespace {

std::mt19937 rng(3);

template <typename T>
std::vector<T> Random(size_t n, double lo, double hi) {
  std::vector<T> a(std::max<size_t>(n, 1));
  std::uniform_real_distribution<double> d(lo, hi);
  for (T &v : a) v = (T)d(rng);
  return a;
}

std::vector<int64_t> Boundary(int B, int S, int T) {
  std::vector<int64_t> bd(4 * (size_t)B);
  for (int b = 0; b < B; ++b) {
    bd[4 * b] = 0;
    bd[4 * b + 1] = 0;
    bd[4 * b + 2] = S - (S > 1 ? b % 2 : 0);
    bd[4 * b + 3] = T - (T > S + 1 ? b % 2 : 0);
  }
  return bd;
}

template <typename T>
int Simple(int B, int S, int Tn, int C, int rnnt_type, bool with_boundary) {
  const int dtype = sizeof(T) == 4 ? K2AMD_F32 : K2AMD_F64;
  const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
  const size_t lm_n = (size_t)B * (S + 1) * C, am_n = (size_t)B * Tn * C;
  auto lm = Random<T>(lm_n, -2, 2), am = Random<T>(am_n, -2, 2);
  std::vector<int64_t> symbols(std::max<size_t>((size_t)B * S, 1));
  for (int64_t &s : symbols) s = rng() % C;
  auto bd = Boundary(B, S, Tn);
  const int64_t *boundary = with_boundary ? bd.data() : nullptr;
  std::vector<T> px(std::max<size_t>((size_t)B * S * T1, 1)), py(std::max<size_t>((size_t)B * (S + 1) * Tn, 1)), lm_probs(lm_n),
      am_probs(std::max<size_t>(am_n, 1)), lm_max((size_t)B * (S + 1)), am_max(std::max<size_t>((size_t)B * Tn, 1)),
      denom(std::max<size_t>((size_t)B * (S + 1) * Tn, 1));
  int status = k2amd_rnnt_logprobs_simple_forward(lm.data(), am.data(), symbols.data(), boundary, px.data(), py.data(),
                                                  lm_probs.data(), am_probs.data(), lm_max.data(), am_max.data(),
                                                  denom.data(), B, S, Tn, C, 0, rnnt_type, dtype, nullptr);
  if (status != K2AMD_OK) return status;
  auto px_grad = Random<T>(px.size(), 0, 1), py_grad = Random<T>(py.size(), 0, 1), seq_scale = Random<T>(B, 0.5, 1.5);
  std::vector<T> lm_grad(lm_n), am_grad(std::max<size_t>(am_n, 1));
  const size_t scratch_n = k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, Tn);
  std::vector<T> scratch(std::max<size_t>(scratch_n, 1));
  return k2amd_rnnt_logprobs_simple_backward(px_grad.data(), py_grad.data(), seq_scale.data(), symbols.data(), boundary,
                                             lm_probs.data(), am_probs.data(), denom.data(), lm_grad.data(),
                                             am_grad.data(), scratch.data(), scratch_n, B, S, Tn, C, 0, rnnt_type,
                                             dtype, nullptr);
}

int Joiner(int B, int S, int Tn, int R, int C, int D, int rnnt_type, int precision, bool hat, bool with_bias) {
  const int T1 = rnnt_type == K2AMD_REGULAR ? Tn + 1 : Tn;
  auto am = Random<float>((size_t)B * Tn * D, -1, 1), lm = Random<float>((size_t)B * (S + 1) * D, -1, 1);
  auto weight = Random<float>((size_t)C * D, -0.2, 0.2), bias = Random<float>(C, -0.5, 0.5);
  std::vector<int64_t> ranges((size_t)B * Tn * R), symbols(std::max<size_t>((size_t)B * S, 1));
  for (int64_t &s : symbols) s = hat ? 1 + rng() % (C - 1) : rng() % C;
  for (int b = 0; b < B; ++b)
    for (int t = 0; t < Tn; ++t) {
      const int start = std::min<int>(S + 1 - R, (int)((long long)t * (S + 2 - R) / std::max(Tn, 1)));
      for (int k = 0; k < R; ++k) ranges[((size_t)b * Tn + t) * R + k] = start + k;
    }
  auto bd = Boundary(B, S, Tn);
  std::vector<float> px(std::max<size_t>((size_t)B * S * T1, 1)), py(std::max<size_t>((size_t)B * (S + 1) * Tn, 1)),
      normalizers((size_t)B * Tn * R);
  const size_t ws_bytes = k2amd_rnnt_joiner_pruned_workspace_bytes(B, S, Tn, R, C, D, precision);
  if (ws_bytes == 0 || k2amd_rnnt_joiner_pruned_forward_workspace_bytes(B, S, Tn, R, C, D, precision) > ws_bytes) return -1;
  std::vector<unsigned char> ws(ws_bytes);
  const float *b_ptr = with_bias ? bias.data() : nullptr;
  int status = hat ? k2amd_rnnt_joiner_hat_pruned_forward(am.data(), lm.data(), ranges.data(), weight.data(), b_ptr,
                                                          symbols.data(), bd.data(), px.data(), py.data(),
                                                          normalizers.data(), B, S, Tn, R, C, D, rnnt_type, precision,
                                                          ws.data(), ws_bytes, nullptr)
                   : k2amd_rnnt_joiner_pruned_forward(am.data(), lm.data(), ranges.data(), weight.data(), b_ptr,
                                                      symbols.data(), bd.data(), px.data(), py.data(),
                                                      normalizers.data(), B, S, Tn, R, C, D, 0, rnnt_type, precision,
                                                      ws.data(), ws_bytes, nullptr);
  if (status != K2AMD_OK) return status;
  auto px_grad = Random<float>(px.size(), 0, 1), py_grad = Random<float>(py.size(), 0, 1), seq_scale = Random<float>(B, 0.5, 1.5);
  std::vector<float> am_grad(am.size()), lm_grad(lm.size()), weight_grad(weight.size()), bias_grad(C);
  float *bg = with_bias ? bias_grad.data() : nullptr;
  return hat ? k2amd_rnnt_joiner_hat_pruned_backward(am.data(), lm.data(), ranges.data(), weight.data(), b_ptr,
                                                     symbols.data(), bd.data(), normalizers.data(), px_grad.data(),
                                                     py_grad.data(), seq_scale.data(), am_grad.data(), lm_grad.data(),
                                                     weight_grad.data(), bg, B, S, Tn, R, C, D, rnnt_type, precision,
                                                     ws.data(), ws_bytes, nullptr)
             : k2amd_rnnt_joiner_pruned_backward(am.data(), lm.data(), ranges.data(), weight.data(), b_ptr,
                                                 symbols.data(), bd.data(), normalizers.data(), px_grad.data(),
                                                 py_grad.data(), seq_scale.data(), am_grad.data(), lm_grad.data(),
                                                 weight_grad.data(), bg, B, S, Tn, R, C, D, 0, rnnt_type, precision,
                                                 ws.data(), ws_bytes, nullptr);
}

}  // namespace

int main() {
  int runs = 0;
  const int simple[][4] = {{2, 5, 9, 70}, {1, 40, 70, 33}, {3, 0, 4, 5}, {2, 6, 0, 7}, {1, 33, 65, 130}};  // B, S, T, C
  for (const auto &sh : simple)
    for (int rnnt_type = 0; rnnt_type < 3; ++rnnt_type) {
      if (rnnt_type != K2AMD_REGULAR && sh[2] < sh[1]) continue;
      const int status = (runs % 2) ? Simple<float>(sh[0], sh[1], sh[2], sh[3], rnnt_type, runs % 3 != 0)
                                    : Simple<double>(sh[0], sh[1], sh[2], sh[3], rnnt_type, runs % 3 != 0);
      if (status != K2AMD_OK) {
        std::printf("simple builder: status %d at B=%d S=%d T=%d C=%d type %d\n", status, sh[0], sh[1], sh[2], sh[3], rnnt_type);
        return 1;
      }
      ++runs;
    }
  const int joiner[][6] = {{2, 6, 9, 3, 37, 64}, {1, 9, 14, 5, 130, 128}, {2, 4, 7, 2, 11, 64}};  // B, S, T, R, C, D
  for (const auto &sh : joiner)
    for (int variant = 0; variant < 6; ++variant) {
      const int rnnt_type = variant % 3, precision = variant % 2;
      const bool hat = variant >= 3;
      const int status = Joiner(sh[0], sh[1], sh[2], sh[3], sh[4], sh[5], rnnt_type, precision, hat, variant != 1);
      if (status != K2AMD_OK) {
        std::printf("fused joiner: status %d at B=%d S=%d T=%d R=%d C=%d D=%d variant %d\n", status, sh[0], sh[1], sh[2],
                    sh[3], sh[4], sh[5], variant);
        return 1;
      }
      ++runs;
    }
  std::printf("all shapes done (%d runs)\n", runs);
  return 0;
}
