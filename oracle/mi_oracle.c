/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of k2's mutual-information
 * recursion, used as the checker for the HIP kernels and as the timed CPU
 * baseline.  Nothing in the product path may call into this file.
 *
 * Follows (reference file:line):
 *   log-add            k2/csrc/utils.h:511-563
 *   forward recursion  k2/python/csrc/torch/mutual_information_cpu.cu:50-124
 *   backward recursion k2/python/csrc/torch/mutual_information_cpu.cu:128-255
 *
 * Layout (all row-major, T axis contiguous):
 *   px [B][S][T1]   T1 = T (modified) or T+1 (regular)
 *   py [B][S+1][T]
 *   p  [B][S+1][T+1]   cells outside the boundary box are left untouched
 *   boundary [B][4] int64 = (s_begin, t_begin, s_end, t_end), or NULL for
 *   (0, 0, S, T).
 *
 * Parity status: pinned against the compiled reference (oracle/_ref) on the
 * committed fixtures (bit-exact), and against closed forms / brute-force path
 * enumeration / invariants in tests/test_oracle_mi.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MIN_LOG_DIFF_F (-15.9423847198486328125f)                       /* logf(FLT_EPSILON) */
#define MIN_LOG_DIFF_D (-36.0436533891171535515240975655615329742431640625) /* log(DBL_EPSILON) */

static inline float log_add_f(float x, float y) {
  float diff;
  if (x < y) { diff = x - y; x = y; } else { diff = y - x; }
  if (diff >= MIN_LOG_DIFF_F) return x + log1pf(expf(diff));
  return x;
}

static inline double log_add_d(double x, double y) {
  double diff;
  if (x < y) { diff = x - y; x = y; } else { diff = y - x; }
  if (diff >= MIN_LOG_DIFF_D) return x + log1p(exp(diff));
  return x;
}

float k2o_log_add_f32(float x, float y) { return log_add_f(x, y); }
double k2o_log_add_f64(double x, double y) { return log_add_d(x, y); }

#define DEFINE_MI(SUFFIX, REAL, LOGADD, EXP, NEG_INF)                                      \
  void k2o_mi_forward_##SUFFIX(const REAL *px, const REAL *py, const int64_t *boundary,    \
                               REAL *p, REAL *ans, int B, int S, int T, int modified) {    \
    const int T1 = modified ? T : T + 1;                                                    \
    const int off = modified ? -1 : 0;                                                      \
    for (int b = 0; b < B; ++b) {                                                           \
      const REAL *pxb = px + (size_t)b * S * T1;                                            \
      const REAL *pyb = py + (size_t)b * (S + 1) * T;                                       \
      REAL *pb = p + (size_t)b * (S + 1) * (T + 1);                                         \
      int s0 = 0, t0 = 0, s1 = S, t1 = T;                                                   \
      if (boundary) {                                                                       \
        s0 = (int)boundary[4 * b + 0]; t0 = (int)boundary[4 * b + 1];                       \
        s1 = (int)boundary[4 * b + 2]; t1 = (int)boundary[4 * b + 3];                       \
      }                                                                                     \
      pb[(size_t)s0 * (T + 1) + t0] = 0;                                                    \
      for (int s = s0 + 1; s <= s1; ++s) {                                                  \
        if (modified)                                                                       \
          pb[(size_t)s * (T + 1) + t0] = NEG_INF;                                           \
        else                                                                                \
          pb[(size_t)s * (T + 1) + t0] =                                                    \
              pb[(size_t)(s - 1) * (T + 1) + t0] + pxb[(size_t)(s - 1) * T1 + t0];          \
      }                                                                                     \
      for (int t = t0 + 1; t <= t1; ++t)                                                    \
        pb[(size_t)s0 * (T + 1) + t] =                                                      \
            pb[(size_t)s0 * (T + 1) + t - 1] + pyb[(size_t)s0 * T + t - 1];                 \
      for (int s = s0 + 1; s <= s1; ++s) {                                                  \
        REAL left = pb[(size_t)s * (T + 1) + t0];                                           \
        for (int t = t0 + 1; t <= t1; ++t) {                                                \
          REAL up = pb[(size_t)(s - 1) * (T + 1) + t + off] +                               \
                    pxb[(size_t)(s - 1) * T1 + t + off];                                    \
          left = LOGADD(up, left + pyb[(size_t)s * T + t - 1]);                             \
          pb[(size_t)s * (T + 1) + t] = left;                                               \
        }                                                                                   \
      }                                                                                     \
      ans[b] = pb[(size_t)s1 * (T + 1) + t1];                                               \
    }                                                                                       \
  }                                                                                         \
                                                                                            \
  /* px_grad / py_grad: caller passes them zero-filled when a boundary tensor is given     \
     (that is what the reference allocates); every in-box element is assigned.  p_grad is  \
     scratch of shape [B][S+1][T+1], zero-filled here.  Returns the number of sequences    \
     whose start-cell gradient differs from ans_grad by more than 1 % (the reference only  \
     logs a warning for those). */                                                          \
  int k2o_mi_backward_##SUFFIX(const REAL *px, const REAL *py, const int64_t *boundary,    \
                               const REAL *p, const REAL *ans_grad, REAL *p_grad,          \
                               REAL *px_grad, REAL *py_grad, int B, int S, int T,          \
                               int modified) {                                             \
    (void)py;                                                                               \
    const int T1 = modified ? T : T + 1;                                                    \
    const int off = modified ? -1 : 0;                                                      \
    int warnings = 0;                                                                       \
    memset(p_grad, 0, sizeof(REAL) * (size_t)B * (S + 1) * (T + 1));                        \
    for (int b = 0; b < B; ++b) {                                                           \
      const REAL *pxb = px + (size_t)b * S * T1;                                            \
      const REAL *pb = p + (size_t)b * (S + 1) * (T + 1);                                   \
      REAL *gb = p_grad + (size_t)b * (S + 1) * (T + 1);                                    \
      REAL *gx = px_grad + (size_t)b * S * T1;                                              \
      REAL *gy = py_grad + (size_t)b * (S + 1) * T;                                         \
      int s0 = 0, t0 = 0, s1 = S, t1 = T;                                                   \
      if (boundary) {                                                                       \
        s0 = (int)boundary[4 * b + 0]; t0 = (int)boundary[4 * b + 1];                       \
        s1 = (int)boundary[4 * b + 2]; t1 = (int)boundary[4 * b + 3];                       \
      }                                                                                     \
      gb[(size_t)s1 * (T + 1) + t1] = ans_grad[b];                                          \
      for (int s = s1; s > s0; --s) {                                                       \
        for (int t = t1; t > t0; --t) {                                                     \
          REAL term1 = pb[(size_t)(s - 1) * (T + 1) + t + off] +                            \
                       pxb[(size_t)(s - 1) * T1 + t + off];                                 \
          REAL total = pb[(size_t)s * (T + 1) + t];                                         \
          if (total - total != 0) total = 0;                                                \
          REAL d1 = EXP(term1 - total), d2 = (REAL)1.0 - d1;                                \
          REAL g = gb[(size_t)s * (T + 1) + t], g1, g2;                                     \
          if (d1 - d1 == 0) { g1 = d1 * g; g2 = d2 * g; } else { g1 = g2 = 0; }             \
          gx[(size_t)(s - 1) * T1 + t + off] = g1;                                          \
          gb[(size_t)(s - 1) * (T + 1) + t + off] = g1;                                     \
          gy[(size_t)s * T + t - 1] = g2;                                                   \
          gb[(size_t)s * (T + 1) + t - 1] += g2;                                            \
        }                                                                                   \
      }                                                                                     \
      for (int t = t1; t > t0; --t) {                                                       \
        REAL g = gb[(size_t)s0 * (T + 1) + t];                                              \
        gb[(size_t)s0 * (T + 1) + t - 1] += g;                                              \
        gy[(size_t)s0 * T + t - 1] = g;                                                     \
      }                                                                                     \
      if (!modified) {                                                                      \
        for (int s = s1; s > s0; --s) {                                                     \
          REAL g = gb[(size_t)s * (T + 1) + t0];                                            \
          gb[(size_t)(s - 1) * (T + 1) + t0] += g;                                          \
          gx[(size_t)(s - 1) * T1 + t0] = g;                                                \
        }                                                                                   \
      }                                                                                     \
      if (ans_grad[b] != 0) {                                                               \
        float ratio = (float)(gb[(size_t)s0 * (T + 1) + t0] / ans_grad[b]);                 \
        if (fabs(ratio - 1.0) > 0.01) ++warnings;                                           \
      }                                                                                     \
    }                                                                                       \
    return warnings;                                                                        \
  }

DEFINE_MI(f32, float, log_add_f, expf, (-INFINITY))
DEFINE_MI(f64, double, log_add_d, exp, (-INFINITY))
