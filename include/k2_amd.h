/*
 * C-ABI of libk2amd.so: the MI355X (gfx950) implementation of k2's RNN-T
 * mutual-information path.  Plain pointers and sizes only; every pointer is a
 * DEVICE pointer unless stated otherwise; tensors are dense row-major with the
 * last axis contiguous.  Every function returns K2AMD_OK (0) or a K2AMD_ERR_*
 * code and never throws; launches are asynchronous on `stream` (a hipStream_t,
 * NULL = the default stream).  No function synchronises the device.
 *
 * Each declaration cites the reference interface it replaces.
 */
#ifndef K2_AMD_H_
#define K2_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define K2AMD_VERSION 100
#define K2AMD_API __attribute__((visibility("default")))

enum k2amd_status {
  K2AMD_OK = 0,
  K2AMD_ERR_INVALID_ARGUMENT = 1, /* bad shape / null pointer / unknown enum */
  K2AMD_ERR_UNSUPPORTED = 2,      /* valid request this build cannot serve (size limit) */
  K2AMD_ERR_WORKSPACE = 3,        /* workspace missing or too small */
  K2AMD_ERR_LAUNCH = 4,           /* HIP reported a launch error */
  K2AMD_ERR_TIMEOUT = 5,          /* a bounded in-kernel wait expired; re-initialise the workspace */
  K2AMD_ERR_SCRATCH_LIMIT = 6     /* k2amd_mi_forward_noalloc: shape beyond its static scratch array */
};

enum k2amd_dtype { K2AMD_F32 = 0, K2AMD_F64 = 1, K2AMD_F16 = 2 /* lattice scores only */ };

/* rnnt_type of k2/python/k2/rnnt_loss.py:70 ("regular" | "modified" | "constrained") */
enum k2amd_rnnt_type { K2AMD_REGULAR = 0, K2AMD_MODIFIED = 1, K2AMD_CONSTRAINED = 2 };

K2AMD_API int k2amd_version(void);
K2AMD_API const char *k2amd_status_string(int status);

/* ------------------------------------------------------------------ MI recursion
 *
 * Shapes (k2/python/csrc/torch/mutual_information.h:30-79):
 *   px [B][S][T1]  with T1 = T (modified != 0) or T+1 (modified == 0)
 *   py [B][S+1][T]
 *   p  [B][S+1][T+1]   written inside each sequence's boundary box only
 *   boundary [B][4] int64 = (s_begin, t_begin, s_end, t_end) or NULL for (0,0,S,T)
 *   ans, ans_grad [B]
 *
 * Workspace (throughput paths): k2amd_mi_workspace_bytes() tells how many bytes of device
 * scratch the pipelined kernels want for a shape and dtype (fp32: chunks of 64 rows as workgroups
 * of specialised wavefronts; fp64: one wavefront per chunk; 0 = no pipelined kernel serves the
 * shape).  The layout and the initial state are the same for both.  The caller owns the buffer and
 * must run k2amd_mi_workspace_init() on it ONCE before its first use (and again after a
 * K2AMD_ERR_TIMEOUT); the kernels leave it ready for the next call, so a buffer sized for the
 * largest shape can be reused for any smaller one.  One workspace serves one stream at a time.
 * Passing workspace == NULL selects the exact one-workgroup-per-sequence kernels instead, which
 * take any S and T with (S + 1) (T + 1) < 2^31.
 */
K2AMD_API size_t k2amd_mi_workspace_bytes(int B, int S, int T, int modified, int dtype);
K2AMD_API int k2amd_mi_workspace_init(void *workspace, size_t workspace_bytes, void *stream);
/* Synchronises `stream` and returns K2AMD_ERR_TIMEOUT if a pipelined kernel that used this
 * workspace gave up waiting for a neighbouring workgroup.  Its results are then invalid, and so
 * are those of every later call until the workspace is initialised again; the kernels make that
 * visible without this call by writing NaN to ans (and to the ans_grad they hand back). */
K2AMD_API int k2amd_mi_workspace_status(const void *workspace, void *stream);
/* The same question without the wait: queues, on `stream`, a copy of the workspace's error flag
 * into *host_flag (4 bytes of pinned host memory that must stay valid until the stream has passed
 * this point) and returns at once.  Once the stream has passed it, *host_flag != 0 says what
 * K2AMD_ERR_TIMEOUT says above.  For hosts that wait on the stream anyway (the reference's Python
 * layer reads `boundary` on the host in every call, k2/python/k2/mutual_information.py:287): the
 * flag rides along with that read, and a launch that gave up is reported at the caller's next
 * call instead of as NaN scores from then on.  No counterpart in the reference. */
K2AMD_API int k2amd_mi_workspace_status_async(const void *workspace, unsigned *host_flag, void *stream);

/* Replaces _k2.mutual_information_forward (k2/python/csrc/torch/mutual_information.cu:26-44,
 * CPU semantics of k2/python/csrc/torch/mutual_information_cpu.cu:50-124):
 *   p[b,s_begin,t_begin] = 0
 *   p[b,s,t] = log_add(p[b,s-1,t+o] + px[b,s-1,t+o], p[b,s,t-1] + py[b,s,t-1]),  o = modified ? -1 : 0
 *   ans[b] = p[b,s_end,t_end]                                                                     */
K2AMD_API int k2amd_mi_forward(const void *px, const void *py, const int64_t *boundary, void *p, void *ans,
                     int B, int S, int T, int modified, int dtype, void *workspace,
                     size_t workspace_bytes, void *stream);

/* k2amd_mi_forward for callers that cannot allocate or bring a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, results and kernels as k2amd_mi_forward, except that the scratch of
 * the pipelined fp32 kernels is a static device array of K2AMD_MI_NOALLOC_SCRATCH_BYTES inside the
 * library (each GPU the library runs on holds its own copy until the process ends); the call
 * itself allocates and frees nothing and synchronises nothing.  A shape whose
 * k2amd_mi_workspace_bytes(...) exceeds that size is refused with K2AMD_ERR_SCRATCH_LIMIT (the
 * headline shape B=32, S=200, T=1000 needs 1.5 MB in fp32, 1.4 MB in fp64).  Every call re-initialises the part of the array it uses with a fill kernel in front of
 * the recursion, so a call never inherits anything from the one before it.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race
 * and must be serialised by the caller.  The first call on a device looks up the array's address;
 * a call with B == 0 does only that.                                                             */
#define K2AMD_MI_NOALLOC_SCRATCH_BYTES (8u << 20)
K2AMD_API int k2amd_mi_forward_noalloc(const void *px, const void *py, const int64_t *boundary,
                                       void *p, void *ans, int B, int S, int T, int modified,
                                       int dtype, void *stream);
/* k2amd_mi_workspace_status for the static array of the current device: synchronises `stream` and
 * returns K2AMD_ERR_TIMEOUT if the last k2amd_mi_forward_noalloc on this device gave up a wait
 * (its ans then holds NaN).  Ask before the next such call: every call starts by clearing the flag
 * with the rest of the array.  No counterpart in the reference.                                  */
K2AMD_API int k2amd_mi_noalloc_status(void *stream);

/* Replaces _k2.mutual_information_backward (k2/python/csrc/torch/mutual_information.cu:46-67,
 * semantics of k2/python/csrc/torch/mutual_information_cpu.cu:128-255).  Writes EVERY element of
 * px_grad [B][S][T1] and py_grad [B][S+1][T] (zeros outside the boundary box).  If
 * overwrite_ans_grad != 0, ans_grad[b] is replaced by the gradient that reached
 * p[b,s_begin,t_begin], which equals the incoming ans_grad[b] when the recursion is consistent
 * (k2/python/csrc/torch/mutual_information_cuda.cu:661-663).                                     */
K2AMD_API int k2amd_mi_backward(const void *px, const void *py, const int64_t *boundary, const void *p,
                      void *ans_grad, void *px_grad, void *py_grad, int B, int S, int T,
                      int modified, int dtype, int overwrite_ans_grad, void *workspace,
                      size_t workspace_bytes, void *stream);

/* The pair below is k2amd_mi_forward / k2amd_mi_backward with one more tensor between them, for
 * callers that run the backward right after the forward, as the reference's autograd function
 * does (k2/python/k2/mutual_information.py:159-164).  It has no counterpart in the reference.
 *   log_deriv [B][S+1][T+1], dtype as p: written by the forward, read by the backward.  It holds
 *   (p[b,s-1,t+o] + px[b,s-1,t+o]) - p[b,s,t], the logarithm of the px edge's derivative at cell
 *   (s,t) exactly as the backward sweep forms it (mutual_information_cpu.cu:195-211), so the
 *   backward reads one tensor where it otherwise reads p twice and px once; the gradients are the
 *   same bits either way.  Elements of a sequence's first row and first column are undefined.
 * log_deriv == NULL makes each call identical to the plain entry point.  Where the pair uses the
 * tensor, p may be NULL in both calls: the forward then does not store p at all (ans and the
 * gradients are all that such a caller gets, which is all the reference's autograd function
 * keeps, k2/python/k2/mutual_information.py:157-169).  Only the pipelined fp32
 * kernels use the tensor: k2amd_mi_keeps_log_deriv(...) tells whether the pair will (1) or will
 * leave it untouched (0) for a shape, so that a host can skip the allocation.  Give the backward
 * the tensor only if the forward call with the same shape, dtype and workspace wrote it.        */
K2AMD_API int k2amd_mi_keeps_log_deriv(int B, int S, int T, int modified, int dtype, int has_workspace);
K2AMD_API int k2amd_mi_forward_keep(const void *px, const void *py, const int64_t *boundary, void *p,
                          void *ans, void *log_deriv, int B, int S, int T, int modified, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream);
K2AMD_API int k2amd_mi_backward_kept(const void *px, const void *py, const int64_t *boundary, const void *p,
                           const void *log_deriv, void *ans_grad, void *px_grad, void *py_grad,
                           int B, int S, int T, int modified, int dtype, int overwrite_ans_grad,
                           void *workspace, size_t workspace_bytes, void *stream);

/* Forward and backward recursion in ONE launch: what the reference's autograd function does with
 * two native calls when gradients are wanted (k2/python/k2/mutual_information.py:157-169).  It has
 * no counterpart in the reference.
 *   ans [B] out; ans_grad [B] in (and out if overwrite_ans_grad), or NULL for the reference's
 *   torch.ones(B) (mutual_information.py:163); px_grad, py_grad out, every element written;
 *   scratch: k2amd_mi_forward_backward_scratch_bytes(...) bytes of device memory that the launch
 *   writes and then reads (nothing in it is an output).
 * Every lattice is swept from both ends at once: the first half of its diagonals forward from
 * the origin, the second half backward from the end cell (the same recursion on px / py read in
 * reverse); where the two meet, alpha + beta of a cell is the log-weight of all paths through
 * it, which gives the score and the gradient that each half then carries back to its own end.
 * The results are those of the two calls to within fp32 rounding of p (not the same bits: the
 * second half's occupation counts come from beta instead of alpha).  A sequence whose end cell no
 * path reaches (score -inf) gets the reference's result for that case from the exact kernels'
 * code inside the same launch.
 * Work is handed to a fixed set of workgroups in an order in which every wait is for work handed
 * out earlier, so the launch needs no particular number of resident workgroups and is safe next
 * to other streams' kernels.  It serves fp32 with a workspace and S + 2 <= 2056:
 * k2amd_mi_forward_backward_supported(...) says whether a call will be served (1) or returns
 * K2AMD_ERR_UNSUPPORTED (0; use the two calls).  k2amd_mi_forward_backward_advised(...) says
 * whether it is also the faster way on the current device (1): it is while the device has a compute
 * unit for every two of the 2 * B * ceil((S+1)/64) half-sweeps, and on long lattices (T >= 1000) at
 * any batch size; otherwise the two calls, whose kernels share compute units, take less time (by
 * up to a fifth), and a host that has the choice makes them. */
K2AMD_API int k2amd_mi_forward_backward_supported(int B, int S, int T, int modified, int dtype,
                                        int has_workspace);
K2AMD_API int k2amd_mi_forward_backward_advised(int B, int S, int T, int modified, int dtype,
                                      int has_workspace);
K2AMD_API size_t k2amd_mi_forward_backward_scratch_bytes(int B, int S, int T, int modified, int dtype);
K2AMD_API int k2amd_mi_forward_backward(const void *px, const void *py, const int64_t *boundary, void *ans,
                              void *scratch, size_t scratch_bytes, void *ans_grad, void *px_grad,
                              void *py_grad, int B, int S, int T, int modified, int dtype,
                              int overwrite_ans_grad, void *workspace, size_t workspace_bytes,
                              void *stream);

/* The split of a joint score over the N inputs of joint_mutual_information_recursion
 * (k2/python/k2/mutual_information.py:404-417, torch ops there: stack, clamp, product, sum):
 *   prods[n][b] = sum_k px_grad[b][k] * max(px_n[b][k], lowest) + the same over py_grad, py_n,
 * lowest = the most negative finite value of the type (an input of -inf carries no occupation).
 * px, py: HOST arrays of N device pointers, each tensor [B][kx] resp. [B][ky] elements, dense;
 * N <= 8 (else K2AMD_ERR_UNSUPPORTED); prods [N][B]; partial: device scratch of
 * k2amd_mi_joint_products_scratch_elements(N, B) elements of the type.                          */
K2AMD_API size_t k2amd_mi_joint_products_scratch_elements(int N, int B);
K2AMD_API int k2amd_mi_joint_products(const void *const *px, const void *const *py, int N,
                                      const void *px_grad, const void *py_grad, void *prods,
                                      void *partial, int B, long long kx, long long ky, int dtype,
                                      void *stream);

/* ------------------------------------------------------------------ RNN-T log-prob builders
 *
 * Common conventions: symbols [B][S] int64 in [0,C); boundary [B][4] int64 or NULL;
 * px [B][S][T1] with T1 = T+1 for K2AMD_REGULAR (column T is -inf) and T otherwise;
 * py [B][S+1][T].  "constrained" adds py[b,s+1,t] to px[b,s,t]; "regular" with a boundary sets
 * px[b,:,t_end[b]] = -inf (k2/python/k2/rnnt_loss.py:25-43,220-223).  The *_backward functions
 * take the gradients w.r.t. the px / py that the matching forward returned, and seq_scale [B]
 * (dtype as the gradients) or NULL: px_grad[b] and py_grad[b] count as multiplied by seq_scale[b].
 * That is the product the reference's autograd function forms with two elementwise kernels
 * (k2/python/k2/mutual_information.py:177-182: the occupation probabilities times the gradient
 * that reaches the sequence's score); here it rides in the kernels that read the gradients.
 */

/* Replaces get_rnnt_logprobs (k2/python/k2/rnnt_loss.py:65-225):
 *   N[b,s,t]  = log(sum_c exp(lm[b,s,c]-lm_max[b,s]) * exp(am[b,t,c]-am_max[b,t]) + tiny) + lm_max + am_max
 *   px[b,s,t] = am[b,t,sym[b,s]] + lm[b,s,sym[b,s]] - N[b,s,t];  py[b,s,t] = am[b,t,blank] + lm[b,s,blank] - N[b,s,t]
 * lm [B][S+1][C], am [B][T][C].  The caller provides the buffers that the backward re-uses:
 * lm_probs [B][S+1][C], am_probs [B][T][C] (the max-shifted exponentials), lm_max [B][S+1],
 * am_max [B][T] and denom [B][S+1][T] (= the matmul + tiny).                                    */
K2AMD_API int k2amd_rnnt_logprobs_simple_forward(
    const void *lm, const void *am, const int64_t *symbols, const int64_t *boundary, void *px,
    void *py, void *lm_probs, void *am_probs, void *lm_max, void *am_max, void *denom, int B, int S,
    int T, int C, int termination_symbol, int rnnt_type, int dtype, void *stream);

/* Gradient of the above w.r.t. lm and am (what torch autograd derives from
 * k2/python/k2/rnnt_loss.py:172-223).  q_scratch is device scratch of q_scratch_elements
 * elements of the tensors' type, at least
 * k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T)
 * (= B * ((S+1) * T + ceil((S+1) / 32) * T + 2 * (S+1) * ceil(T / 64)): the [B][S+1][T] operand
 * of the two products, then the gradients' sums along s ([B][T] per 32 rows) and along t
 * ([B][S+1] per 64 frames, for px_grad and for py_grad)); less is refused with
 * K2AMD_ERR_WORKSPACE before anything is launched.                                               */
K2AMD_API size_t k2amd_rnnt_logprobs_simple_backward_scratch_elements(int B, int S, int T);
K2AMD_API int k2amd_rnnt_logprobs_simple_backward(
    const void *px_grad, const void *py_grad, const void *seq_scale, const int64_t *symbols,
    const int64_t *boundary,
    const void *lm_probs, const void *am_probs, const void *denom, void *lm_grad, void *am_grad,
    void *q_scratch, size_t q_scratch_elements, int B, int S, int T, int C, int termination_symbol,
    int rnnt_type, int dtype, void *stream);

/* The terms that get_rnnt_logprobs_smoothed (k2/python/k2/rnnt_loss.py:1471-1704) adds to
 * get_rnnt_logprobs, and the mix of the three:
 *   px[b,s,t] = joint_scale * px_joint[b,s,t] + lm_only_scale * log softmax(lm[b,s])[sym[b,s]]
 *                                             + am_only_scale * log softmax(am[b,t] + log unigram)[sym[b,s]]
 * and py alike with the termination symbol; joint_scale = 1 - lm_only_scale - am_only_scale,
 * unigram = the mean over all B (S+1) rows of softmax(lm) + tiny, a scale of exactly 0 counts as
 * 1e-20 as in the reference.  After the mix: px[b,:,T] = px[b,:,boundary[b,3]] = -inf on a regular
 * lattice, px[b,s,t] += py[b,s+1,t] on a constrained one.
 * Inputs besides lm and am: what k2amd_rnnt_logprobs_simple_forward wrote for the same lm and am
 * on a REGULAR (if rnnt_type is regular) or MODIFIED (otherwise) lattice with a null boundary:
 * px_joint, py_joint, lm_probs, am_probs, lm_max, am_max.  Outputs: px [B][S][T+1 or T],
 * py [B][S+1][T] (neither may overlap px_joint / py_joint), and for the backward lm_norm [B][S+1]
 * (log sum_c exp lm), am_norm [B][T] (log sum_c exp(am) unigram[c]) and unigram [2][C] (the
 * unigram, then its log).  scratch: k2amd_rnnt_smoothed_scratch_elements(B, S, T, C) elements of
 * the tensors' type (row sums of the lattice's gradients, per-row weights and the partial column
 * sums over chunks of rows: 4 B (S+1) + 3 B T + C (ceil(B T / 64) + ceil(B (S+1) / 64) + 1) at
 * most, chunks capped at 64 each); less is refused with K2AMD_ERR_WORKSPACE before anything is
 * launched.  No limit on the vocabulary; k2amd_rnnt_smoothed_supported tells whether the row
 * counts fit the kernels' 32-bit indexing.                                                         */
K2AMD_API size_t k2amd_rnnt_smoothed_scratch_elements(int B, int S, int T, int C);
K2AMD_API int k2amd_rnnt_smoothed_supported(int B, int S, int T, int C, int dtype);
K2AMD_API int k2amd_rnnt_smoothed_forward(
    const void *lm, const void *am, const int64_t *symbols, const int64_t *boundary,
    const void *lm_probs, const void *am_probs, const void *lm_max, const void *am_max,
    const void *px_joint, const void *py_joint, void *px, void *py, void *lm_norm, void *am_norm,
    void *unigram, void *scratch, size_t scratch_elements, double lm_only_scale, double am_only_scale,
    int B, int S, int T, int C, int termination_symbol, int rnnt_type, int dtype, void *stream);

/* Gradient of the two marginal terms above (what torch autograd derives from
 * k2/python/k2/rnnt_loss.py:1608-1690), ADDED to lm_grad [B][S+1][C] and am_grad [B][T][C].  The
 * joint term's gradient is k2amd_rnnt_logprobs_simple_backward's on the same px_grad / py_grad,
 * boundary and rnnt_type with seq_scale[b] * joint_scale in place of seq_scale[b]; it writes
 * lm_grad and am_grad and so has to run first.  px_grad / py_grad are the gradients that reach
 * the mixed px / py.                                                                              */
K2AMD_API int k2amd_rnnt_smoothed_backward(
    const void *px_grad, const void *py_grad, const void *seq_scale, const int64_t *symbols,
    const int64_t *boundary, const void *lm_probs, const void *am_probs, const void *lm_max,
    const void *am_max, const void *lm_norm, const void *am_norm, const void *unigram, void *lm_grad,
    void *am_grad, void *scratch, size_t scratch_elements, double lm_only_scale, double am_only_scale,
    int B, int S, int T, int C, int termination_symbol, int rnnt_type, int dtype, void *stream);

/* Replaces get_rnnt_logprobs_joint (k2/python/k2/rnnt_loss.py:341-447): logits [B][T][S+1][C];
 * normalizers [B][T][S+1] = logsumexp over C is written for the backward.                        */
K2AMD_API int k2amd_rnnt_logprobs_joint_forward(
    const void *logits, const int64_t *symbols, const int64_t *boundary, void *px, void *py,
    void *normalizers, int B, int S, int T, int C, int termination_symbol, int rnnt_type, int dtype,
    void *stream);
K2AMD_API int k2amd_rnnt_logprobs_joint_backward(
    const void *logits, const void *normalizers, const void *px_grad, const void *py_grad,
    const void *seq_scale, const int64_t *symbols, const int64_t *boundary, void *logits_grad, int B, int S, int T, int C,
    int termination_symbol, int rnnt_type, int dtype, void *stream);

/* Replaces get_rnnt_logprobs_pruned (k2/python/k2/rnnt_loss.py:1180-1348): logits [B][T][R][C],
 * ranges [B][T][R] int64 with values in [0,S]; row k of frame t lands on
 * s = (ranges[b,t,0] + k) mod (S+1) (k2/python/k2/rnnt_loss.py:957-989), every other element of
 * px / py is -inf.  normalizers [B][T][R] is written for the backward.                           */
K2AMD_API int k2amd_rnnt_logprobs_pruned_forward(
    const void *logits, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary,
    void *px, void *py, void *normalizers, int B, int S, int T, int R, int C,
    int termination_symbol, int rnnt_type, int dtype, void *stream);
K2AMD_API int k2amd_rnnt_logprobs_pruned_backward(
    const void *logits, const void *normalizers, const void *px_grad, const void *py_grad,
    const void *seq_scale, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary, void *logits_grad,
    int B, int S, int T, int R, int C, int termination_symbol, int rnnt_type, int dtype,
    void *stream);

/* Replaces get_hat_logprobs_pruned (k2/python/k2/rnnt_loss.py:992-1177), the hybrid autoregressive
 * transducer variant that rnnt_loss_pruned(use_hat_loss=True) selects (rnnt_loss.py:1439-1447):
 * the blank is column 0 and py = log sigmoid(logits[...,0]); normalizers [B][T][R] = logsumexp
 * over columns 1..C-1; px = logits[..., symbol] - normalizers + log(1 - sigmoid(logits[...,0])).
 * Placement, -inf fill, boundary fix and the "constrained" add are those of the pruned builder. */
K2AMD_API int k2amd_rnnt_hat_logprobs_pruned_forward(
    const void *logits, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary,
    void *px, void *py, void *normalizers, int B, int S, int T, int R, int C, int rnnt_type,
    int dtype, void *stream);
K2AMD_API int k2amd_rnnt_hat_logprobs_pruned_backward(
    const void *logits, const void *normalizers, const void *px_grad, const void *py_grad,
    const void *seq_scale, const int64_t *symbols, const int64_t *ranges, const int64_t *boundary, void *logits_grad,
    int B, int S, int T, int R, int C, int rnnt_type, int dtype, void *stream);

/* ------------------------------------------------------------------ pruning
 *
 * Replaces the device work of get_rnnt_prune_ranges (k2/python/k2/rnnt_loss.py:730-780):
 * window sum of s_range rows of py_grad (added first row to last), minus px_grad shifted down one
 * row, first arg-max over the window start, frames t >= t_end-1 pinned to max(s_end-s_range+1, 0),
 * then the two reverse running minima of _adjust_pruning_lower_bound
 * (k2/python/k2/rnnt_loss.py:580-630).  s_range is the final value (the caller applies the
 * adjustments of k2/python/k2/rnnt_loss.py:694-729).  ranges [B][T][s_range] int64.              */
K2AMD_API int k2amd_rnnt_prune_ranges(const void *px_grad, const void *py_grad,
                                      const int64_t *boundary, int64_t *ranges, int B, int S, int T,
                                      int modified, int s_range, int dtype, void *stream);

/* Replaces the device work of get_rnnt_prune_ranges_deprecated (k2/python/k2/rnnt_loss.py:853-908):
 * per frame the first arg-max over w of prefix[w + s_range] - prefix[w], where prefix[k] is the sum
 * over rows i < k of px_grad[b,i,t] + py_grad[b,i,t] (px_grad's row S counts as 0), each prefix
 * accumulated in double and rounded once to the input type (torch.cumsum on the CPU), the
 * difference taken in the input type; then the padding and the running minima of
 * k2amd_rnnt_prune_ranges.  s_range is the final value (min(s_range, S + 1), rnnt_loss.py:842-843).
 * ranges [B][T][s_range] int64.                                                                  */
K2AMD_API int k2amd_rnnt_prune_ranges_deprecated(const void *px_grad, const void *py_grad,
                                                 const int64_t *boundary, int64_t *ranges, int B,
                                                 int S, int T, int modified, int s_range, int dtype,
                                                 void *stream);

/* Replaces the gather of do_rnnt_pruning (k2/python/k2/rnnt_loss.py:947-953):
 * lm_pruned[b,t,k,:] = lm[b, ranges[b,t,k], :]; lm [B][S1][D].  Indices outside [0,S1) yield 0.  */
K2AMD_API int k2amd_rnnt_prune_gather(const void *lm, const int64_t *ranges, void *lm_pruned, int B,
                                      int S1, int T, int R, int D, int dtype, void *stream);
/* Its gradient: lm_grad[b,s,:] = sum over (t,k) with ranges[b,t,k] == s of grad[b,t,k,:], every
 * element of lm_grad written.  Which terms meet in which partial sum is fixed by ranges alone, so
 * the result is the same in every run, while T * R <= 10240; beyond that the sums are formed with
 * floating-point atomic adds and their last bits vary.                                           */
K2AMD_API int k2amd_rnnt_prune_gather_backward(const void *grad, const int64_t *ranges,
                                               void *lm_grad, int B, int S1, int T, int R, int D,
                                               int dtype, void *stream);

/* ------------------------------------------------------------------ pruned joiner, fused
 *
 * What stands between do_rnnt_pruning (k2/python/k2/rnnt_loss.py:913-954) and rnnt_loss_pruned
 * (rnnt_loss.py:1351-1468) in the reference's recipes is the caller's joiner; these two calls run
 * the usual one, logits = tanh(am_pruned + lm_pruned) . weight^T + bias, TOGETHER with the gather
 * before it and get_rnnt_logprobs_pruned (rnnt_loss.py:1180-1348) after it, so that the
 * [B][T][R][C] logits never exist in memory (the reference has no such call; its torch-op chain
 * do_rnnt_pruning -> tanh -> linear -> get_rnnt_logprobs_pruned is what they are checked against).
 *   am [B][T][D], lm [B][S+1][D], ranges [B][T][R] int64, weight [C][D] (torch.nn.Linear's
 *   layout), bias [C] or NULL, symbols [B][S]; all floating tensors fp32.
 *   px, py, normalizers [B][T][R]: as k2amd_rnnt_logprobs_pruned_forward.
 *   precision: K2AMD_JOINER_F32 multiplies in fp32 on the matrix cores; K2AMD_JOINER_BF16 rounds the
 *   activations, the weight and the logits' gradients to bfloat16 for the products (fp32 sums).
 *   workspace: device memory, k2amd_rnnt_joiner_pruned_forward_workspace_bytes(...) bytes for the
 *   forward (the weight in the operand type) and k2amd_rnnt_joiner_pruned_workspace_bytes(...)
 *   for the backward (the weight twice, and what its first kernel hands its second: the
 *   activations and the logits' gradients in the operand type, B T R x (D + C) elements or, where
 *   that is more than 128 Mi elements, as many; the backward then goes through the rows in
 *   passes; the environment variable K2AMD_JOINER_PASS_ELEMS, read at every call, sets another
 *   bound); 0 = shape not served: D a multiple of 64 up to 512, R <= 32 and <= S + 1; any C.  Contents need
 *   not survive between the two calls.
 * The backward takes what the forward took, the normalizers it wrote and the gradients w.r.t. its
 * px / py (seq_scale as for the other builders), and writes am_grad [B][T][D], lm_grad [B][S+1][D],
 * weight_grad [C][D], bias_grad [C] (or NULL).  lm_grad, weight_grad and bias_grad are sums formed
 * with floating-point atomic adds: their last bits vary from run to run.                        */
enum k2amd_joiner_precision { K2AMD_JOINER_F32 = 0, K2AMD_JOINER_BF16 = 1 };
K2AMD_API size_t k2amd_rnnt_joiner_pruned_workspace_bytes(int B, int S, int T, int R, int C, int D,
                                                          int precision);
K2AMD_API size_t k2amd_rnnt_joiner_pruned_forward_workspace_bytes(int B, int S, int T, int R, int C,
                                                                  int D, int precision);
K2AMD_API int k2amd_rnnt_joiner_pruned_forward(
    const void *am, const void *lm, const int64_t *ranges, const void *weight, const void *bias,
    const int64_t *symbols, const int64_t *boundary, void *px, void *py, void *normalizers, int B,
    int S, int T, int R, int C, int D, int termination_symbol, int rnnt_type, int precision,
    void *workspace, size_t workspace_bytes, void *stream);
K2AMD_API int k2amd_rnnt_joiner_pruned_backward(
    const void *am, const void *lm, const int64_t *ranges, const void *weight, const void *bias,
    const int64_t *symbols, const int64_t *boundary, const void *normalizers, const void *px_grad,
    const void *py_grad, const void *seq_scale, void *am_grad, void *lm_grad, void *weight_grad,
    void *bias_grad, int B, int S, int T, int R, int C, int D, int termination_symbol, int rnnt_type,
    int precision, void *workspace, size_t workspace_bytes, void *stream);

/* The same pair with get_hat_logprobs_pruned (k2/python/k2/rnnt_loss.py:992-1177) in place of
 * get_rnnt_logprobs_pruned, i.e. rnnt_loss_pruned(use_hat_loss=True) on the joiner's logits: column 0
 * is the blank, py = log sigmoid(logits[..., 0]), normalizers = logsumexp over columns 1..C-1,
 * px = logits[..., symbol] - normalizers + log(1 - sigmoid(logits[..., 0])).  Arguments, workspace
 * and limits as above, without termination_symbol; C >= 2.  The reference has no such call (its
 * chain is do_rnnt_pruning -> the caller's joiner -> get_hat_logprobs_pruned).                   */
K2AMD_API int k2amd_rnnt_joiner_hat_pruned_forward(
    const void *am, const void *lm, const int64_t *ranges, const void *weight, const void *bias,
    const int64_t *symbols, const int64_t *boundary, void *px, void *py, void *normalizers, int B,
    int S, int T, int R, int C, int D, int rnnt_type, int precision, void *workspace,
    size_t workspace_bytes, void *stream);
K2AMD_API int k2amd_rnnt_joiner_hat_pruned_backward(
    const void *am, const void *lm, const int64_t *ranges, const void *weight, const void *bias,
    const int64_t *symbols, const int64_t *boundary, const void *normalizers, const void *px_grad,
    const void *py_grad, const void *seq_scale, void *am_grad, void *lm_grad, void *weight_grad,
    void *bias_grad, int B, int S, int T, int R, int C, int D, int rnnt_type, int precision,
    void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------ lattice
 *
 * Replaces _k2.pruned_ranges_to_lattice (k2/python/csrc/torch/pruned_ranges_to_lattice.cu:60-263):
 * the pruned band as one lattice per sequence.  ranges [B][T][R] int32, frames [B] int32,
 * symbols [B][S] int64, logits [B][T][R][C] (f32 / f64 / f16) with element strides
 * logits_strides[4] (host memory).  Sequence b has frames[b] * R + 1 states.
 *
 * Step 1 (..._count) fills, on the device,
 *   arc_local  [B][T*R+1]  arcs of sequence b leaving states before the given one (scratch),
 *   seq_arcs   [B]         (scratch),
 *   state_splits [B+1]     row splits sequence -> states (k2's row_splits1),
 *   arc_base   [B+1]       arcs of the sequences before b; arc_base[B] = number of arcs.
 * The caller reads state_splits[B] and arc_base[B] to size the outputs of step 2 (..._fill):
 *   arc_splits [states+1]  row splits state -> arcs (k2's row_splits2),
 *   arcs       [arcs][4]   k2's Arc records {int32 src, int32 dest, int32 label, float score},
 *   arc_map    [arcs]      element index of the arc's score in logits, or -1.                    */
K2AMD_API int k2amd_lattice_count(const int32_t *ranges, const int32_t *frames, int32_t *arc_local,
                                  int32_t *seq_arcs, int32_t *state_splits, int32_t *arc_base,
                                  int B, int T, int R, void *stream);
K2AMD_API int k2amd_lattice_fill(const int32_t *ranges, const int32_t *frames,
                                 const int64_t *symbols, const void *logits,
                                 const int64_t *logits_strides, const int32_t *state_splits,
                                 const int32_t *arc_base, const int32_t *arc_local,
                                 int32_t *arc_splits, void *arcs, int32_t *arc_map, int B, int T,
                                 int R, int S, int C, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* K2_AMD_H_ */
