// Runs the pipelined fp32 mutual-information kernels (the host copy of k2_amd/csrc/mi_fast.hip,
// linked in) through the C-ABI once: program B S T modified route, route 0 = the pair of launches,
// 1 = the pair with the log-derivative tensor and no p, 2 = the single launch; heap buffers of
// exactly the documented sizes.  It checks no values (tests/test_cpu_build_pipelined.py does); it
// prints the first score so that a run can be compared with another.  Built
//   with -fsanitize=thread: the work-items are threads, the barriers of a workgroup and of a
//     wavefront and the atomics are what orders them, so two wavefronts that touch the same LDS or
//     device word without one of those between them are reported as a data race;
//   with -fsanitize=address,undefined: an access outside a buffer or outside a workgroup's LDS
//     structure, and an index beyond the bounds of an array inside it, end the program.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "../../include/k2_amd.h"

int main(int argc, char **argv) {
  if (argc != 6) return 64;
  const int B = atoi(argv[1]), S = atoi(argv[2]), T = atoi(argv[3]), modified = atoi(argv[4]), route = atoi(argv[5]);
  const int T1 = modified ? T : T + 1;
  std::mt19937 rng(7);
  std::normal_distribution<float> normal(-1.0f, 1.0f);
  std::vector<float> px((size_t)B * S * T1), py((size_t)B * (S + 1) * T);
  for (float &v : px) v = normal(rng);
  for (float &v : py) v = normal(rng);
  std::vector<int64_t> boundary(4 * (size_t)B);
  for (int b = 0; b < B; ++b) {
    boundary[4 * b] = std::min(b % 2, S);
    boundary[4 * b + 1] = std::min(b % 3, T);
    boundary[4 * b + 2] = std::max(S - b % 2, (int)boundary[4 * b]);
    boundary[4 * b + 3] = std::max(T - b % 2, (int)boundary[4 * b + 1]);
  }
  const size_t ws_bytes = k2amd_mi_workspace_bytes(B, S, T, modified, K2AMD_F32);
  if (ws_bytes == 0) return 65;
  std::vector<unsigned char> ws(ws_bytes);
  if (k2amd_mi_workspace_init(ws.data(), ws_bytes, nullptr) != K2AMD_OK) return 66;
  std::vector<float> p((size_t)B * (S + 1) * (T + 1)), log_deriv(p.size()), ans(B), seed(B, 1.0f), px_grad(px.size()),
      py_grad(py.size());
  int status;
  if (route == 0) {
    status = k2amd_mi_forward(px.data(), py.data(), boundary.data(), p.data(), ans.data(), B, S, T, modified, K2AMD_F32,
                              ws.data(), ws_bytes, nullptr);
    if (status == K2AMD_OK)
      status = k2amd_mi_backward(px.data(), py.data(), boundary.data(), p.data(), seed.data(), px_grad.data(),
                                 py_grad.data(), B, S, T, modified, K2AMD_F32, 1, ws.data(), ws_bytes, nullptr);
  } else if (route == 1) {
    status = k2amd_mi_forward_keep(px.data(), py.data(), boundary.data(), nullptr, ans.data(), log_deriv.data(), B, S,
                                   T, modified, K2AMD_F32, ws.data(), ws_bytes, nullptr);
    if (status == K2AMD_OK)
      status = k2amd_mi_backward_kept(px.data(), py.data(), boundary.data(), nullptr, log_deriv.data(), seed.data(),
                                      px_grad.data(), py_grad.data(), B, S, T, modified, K2AMD_F32, 1, ws.data(),
                                      ws_bytes, nullptr);
  } else {
    const size_t scratch_bytes = k2amd_mi_forward_backward_scratch_bytes(B, S, T, modified, K2AMD_F32);
    std::vector<float> scratch(scratch_bytes / 4 + 1);
    status = k2amd_mi_forward_backward(px.data(), py.data(), boundary.data(), ans.data(), scratch.data(), scratch_bytes,
                                       seed.data(), px_grad.data(), py_grad.data(), B, S, T, modified, K2AMD_F32, 1,
                                       ws.data(), ws_bytes, nullptr);
  }
  if (status == K2AMD_OK) status = k2amd_mi_workspace_status(ws.data(), nullptr);
  printf("status %d score %.6g\n", status, ans[0]);
  return status == K2AMD_OK ? 0 : 1;
}
