"""TEST INFRASTRUCTURE ONLY: numpy restatement of the torch-op chains of
k2/python/k2/rnnt_loss.py that surround the mutual-information recursion.

Each function names the reference lines it follows.  Arithmetic is carried out in the dtype of
the inputs (fp32 stays fp32) and in the reference's order of operations where that order is
visible in its source; reductions inside numpy (``max``, ``sum``, ``matmul``) may round
differently from torch's, which is within the stated float tolerances.

Parity status: every function below is pinned.
  * By what the reference's OWN Python chain computes: tests/golden/rnnt_ref_fixtures.npz, written
    by tests/golden/make_rnnt_fixtures.py from k2/python/k2/rnnt_loss.py and mutual_information.py
    loaded by path over the reference's compiled CPU recursion (whole chains simple loss ->
    gradients -> prune ranges -> pruning -> pruned log-probs -> pruned loss for the three lattice
    types, delay penalty, HAT, smoothed, deprecated ranges; cases around arg-max ties and around
    the ``+ tiny`` floor).  tests/test_oracle_rnnt_fixtures.py: integers bit for bit, floats to
    the stated tolerances.  (That comparison is why ``prune_ranges_deprecated`` accumulates its
    cumulative sums in float64: torch's CPU cumsum does.)
  * ``logprobs_simple`` / ``logprobs_joint`` / ``logprobs_pruned`` also by the hand fixture of
    k2/python/tests/rnnt_loss_test.py:127-139 through brute-force enumeration of its alignments,
    by the identities the reference tests assert (simple == joint on am+lm, invariance to
    per-frame constants) and by the no-pruning identity (s_range = S+1 gives the joint loss).
  * ``apply_delay_penalty`` also by brute force over alignments with the per-symbol term.
  * ``roll_by_shifts``, ``monotonic_lower_bound`` also by the doc-test vectors at
    k2/python/k2/rnnt_loss.py:965-976 and :551-565.
  * ``hat_logprobs_pruned`` also by the probability identity of the model, by direct
    probability-space evaluation and by reduction to ``logprobs_pruned``.
  * ``logprobs_smoothed`` also by the identity the reference tests assert (both scales 0 gives
    rnnt_loss_simple, k2/python/tests/rnnt_loss_test.py:167-178) and shift invariance (:436-485).
  * ``joiner_pruned_logits`` (the step the reference leaves to the caller) by torch's own gather /
    tanh / linear on the same numbers and by explicit loops.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this.
"""
import numpy as np

from . import mi as _mi


def _neg_inf(dtype):
    return np.array(-np.inf, dtype=dtype)


def fix_for_boundary(px, boundary):
    """k2/python/k2/rnnt_loss.py:25-43: px[b, :, t_end[b]] = -inf (regular lattice only)."""
    if boundary is None:
        return px
    B = px.shape[0]
    px[np.arange(B), :, boundary[:, 3]] = -np.inf
    return px


def validate_st_lengths(S, T, regular, boundary):
    """k2/python/k2/rnnt_loss.py:46-62."""
    assert S >= 0, S
    if boundary is None:
        assert regular or T >= S, (T, S)
    else:
        assert regular or bool((boundary[:, 3] >= boundary[:, 2]).all())


def logprobs_simple(lm, am, symbols, termination_symbol, rnnt_type="regular", boundary=None):
    """k2/python/k2/rnnt_loss.py:65-225 (get_rnnt_logprobs)."""
    assert lm.ndim == 3 and am.ndim == 3
    assert lm.shape[0] == am.shape[0] and lm.shape[2] == am.shape[2]
    B, T, C = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S)
    assert rnnt_type in ("regular", "modified", "constrained")
    validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    dt = am.dtype
    am_max = am.max(axis=2, keepdims=True)
    lm_max = lm.max(axis=2, keepdims=True)
    am_probs = np.exp(am - am_max)
    lm_probs = np.exp(lm - lm_max)
    normalizers = np.log(np.matmul(lm_probs, am_probs.transpose(0, 2, 1)) + np.finfo(dt).tiny)
    normalizers = (normalizers + lm_max + am_max.transpose(0, 2, 1)).astype(dt)  # [B,S+1,T]

    bi = np.arange(B)[:, None, None]
    px_am = am[bi, np.arange(T)[None, None, :], symbols[:, :, None]]  # [B,S,T]
    if rnnt_type == "regular":
        px_am = np.concatenate([px_am, np.full((B, S, 1), -np.inf, dtype=dt)], axis=2)
    px_lm = lm[bi, np.arange(S)[None, :, None], symbols[:, :, None]]  # [B,S,1]
    px = (px_am + px_lm).astype(dt)
    px[:, :, :T] -= normalizers[:, :S, :]
    py = (am[:, :, termination_symbol][:, None, :] + lm[:, :, termination_symbol][:, :, None]
          - normalizers).astype(dt)
    if rnnt_type == "regular":
        px = fix_for_boundary(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def _logsumexp_last(x):
    m = x.max(axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0).astype(x.dtype)
    return (np.log(np.exp(x - m).sum(axis=-1)) + m[..., 0]).astype(x.dtype)


def logprobs_joint(logits, symbols, termination_symbol, rnnt_type="regular", boundary=None):
    """k2/python/k2/rnnt_loss.py:341-447 (get_rnnt_logprobs_joint)."""
    assert logits.ndim == 4
    B, T, S1, C = logits.shape
    S = S1 - 1
    assert symbols.shape == (B, S)
    assert rnnt_type in ("regular", "modified", "constrained")
    validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    dt = logits.dtype
    normalizers = _logsumexp_last(logits).transpose(0, 2, 1)  # [B,S+1,T]
    bi = np.arange(B)[:, None, None]
    px = logits[bi, np.arange(T)[None, :, None], np.arange(S)[None, None, :],
                symbols[:, None, :]]  # [B,T,S]
    px = px.transpose(0, 2, 1)
    if rnnt_type == "regular":
        px = np.concatenate([px, np.full((B, S, 1), -np.inf, dtype=dt)], axis=2)
    px = np.ascontiguousarray(px)
    px[:, :, :T] -= normalizers[:, :S, :]
    py = np.ascontiguousarray(logits[:, :, :, termination_symbol].transpose(0, 2, 1))
    py -= normalizers
    if rnnt_type == "regular":
        px = fix_for_boundary(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def monotonic_lower_bound(x):
    """k2/python/k2/rnnt_loss.py:543-577: reverse running minimum along the last axis."""
    return np.minimum.accumulate(x[..., ::-1], axis=-1)[..., ::-1]


def adjust_pruning_lower_bound(s_begin, s_range):
    """k2/python/k2/rnnt_loss.py:580-630."""
    T = s_begin.shape[1]
    ramp = (s_range - 1) * np.arange(T, dtype=np.int64)
    s_begin = monotonic_lower_bound(s_begin)
    s_begin = -(s_begin - ramp)
    s_begin = monotonic_lower_bound(s_begin)
    s_begin = np.maximum(s_begin, 0)
    return -(s_begin - ramp)


def effective_s_range(S, T1_is_regular, boundary, s_range):
    """The s_range adjustments at k2/python/k2/rnnt_loss.py:694-729 (the reference prints a
    warning when it changes the value)."""
    if T1_is_regular:
        Ss = boundary[:, 2]
        Ts = boundary[:, 3]
        # trunc division of (S_b - 1) by T_b, then + 2
        q = np.trunc((Ss - 1).astype(np.float64) / Ts.astype(np.float64)).astype(np.int64)
        s_range_min = int((q + 2).max())
        if s_range < s_range_min:
            s_range = s_range_min
    if s_range > S:
        s_range = S + 1
    if T1_is_regular:
        assert s_range >= 2
    else:
        assert s_range >= 1
    return s_range


def prune_ranges(px_grad, py_grad, boundary, s_range):
    """k2/python/k2/rnnt_loss.py:636-780 (get_rnnt_prune_ranges).  The window sum adds the
    s_range rows left to right, then subtracts px_grad, then takes the first maximum."""
    B, S, T1 = px_grad.shape
    T = py_grad.shape[-1]
    regular = T1 != T
    assert T1 in (T, T + 1)
    S1 = S + 1
    assert py_grad.shape == (B, S1, T)
    assert boundary.shape == (B, 4)
    validate_st_lengths(S, T, regular, boundary)
    s_range = effective_s_range(S, regular, boundary, s_range)
    n = S1 - s_range + 1
    blk = py_grad[:, 0:n, :].copy()
    for k in range(1, s_range):
        blk = blk + py_grad[:, k:k + n, :]
    px_pad = np.concatenate([np.zeros((B, 1, T1), dtype=px_grad.dtype), px_grad], axis=1)
    final = blk - px_pad[:, :n, :T]
    s_begin = np.argmax(final, axis=1).astype(np.int64)  # [B,T], first maximum
    mask = np.arange(T)[None, :] < (boundary[:, 3][:, None] - 1)
    pad = np.maximum(boundary[:, 2][:, None] - s_range + 1, 0)
    s_begin = np.where(mask, s_begin, pad)
    s_begin = adjust_pruning_lower_bound(s_begin, 2 if not regular else s_range)
    return (s_begin[:, :, None] + np.arange(s_range, dtype=np.int64)[None, None, :]).astype(np.int64)


def do_pruning(am, lm, ranges):
    """k2/python/k2/rnnt_loss.py:913-954 (do_rnnt_pruning)."""
    B, T, R = ranges.shape
    assert am.shape[0] == B and lm.shape[0] == B and am.shape[1] == T
    am_pruned = np.broadcast_to(am[:, :, None, :], (B, T, R, am.shape[-1]))
    lm_pruned = lm[np.arange(B)[:, None, None], ranges, :]
    return am_pruned, lm_pruned


def joiner_pruned_logits(am, lm, ranges, weight, bias=None):
    """The joiner that the reference's recipes place between do_rnnt_pruning and
    rnnt_loss_pruned (k2/python/k2/rnnt_loss.py:913-954 describes the step: "am_pruned + lm_pruned"
    goes to the joiner): logits = tanh(am_pruned + lm_pruned) . weight^T + bias, [B][T][R][C], with
    weight [C][D] in torch.nn.Linear's layout.  Plain numpy on the arrays' own dtype."""
    am_pruned, lm_pruned = do_pruning(am, lm, ranges)
    logits = np.tanh(am_pruned + lm_pruned) @ weight.T
    if bias is not None:
        logits = logits + bias
    return logits.astype(am.dtype)


def roll_by_shifts(src, shifts):
    """k2/python/k2/rnnt_loss.py:957-989: out[b,t,s] = src[b,t,(s - shifts[b,t]) mod S]."""
    B, T, S = src.shape
    assert shifts.shape == (B, T)
    index = (np.arange(S)[None, None, :] - shifts[:, :, None]) % S
    return np.take_along_axis(src, index, axis=2)


def logprobs_pruned(logits, symbols, ranges, termination_symbol, boundary, rnnt_type="regular"):
    """k2/python/k2/rnnt_loss.py:1180-1348 (get_rnnt_logprobs_pruned)."""
    assert logits.ndim == 4
    B, T, R, C = logits.shape
    assert ranges.shape == (B, T, R)
    S = symbols.shape[1]
    assert symbols.shape == (B, S)
    assert rnnt_type in ("regular", "modified", "constrained")
    validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    dt = logits.dtype
    normalizers = _logsumexp_last(logits)  # [B,T,R]
    sym_ext = np.concatenate(
        [symbols, np.full((B, 1), termination_symbol, dtype=np.int64)], axis=1)
    pruned_symbols = sym_ext[np.arange(B)[:, None, None], ranges]  # [B,T,R]
    px = np.take_along_axis(logits, pruned_symbols[..., None], axis=3)[..., 0] - normalizers
    px = np.concatenate([px, np.full((B, T, S + 1 - R), -np.inf, dtype=dt)], axis=2)
    px = roll_by_shifts(px, ranges[:, :, 0])[:, :, :S]
    px = px.transpose(0, 2, 1)
    if rnnt_type == "regular":
        px = np.concatenate([px, np.full((B, S, 1), -np.inf, dtype=dt)], axis=2)
    px = np.ascontiguousarray(px)
    py = logits[:, :, :, termination_symbol] - normalizers
    py = np.concatenate([py, np.full((B, T, S + 1 - R), -np.inf, dtype=dt)], axis=2)
    py = roll_by_shifts(py, ranges[:, :, 0])
    py = np.ascontiguousarray(py.transpose(0, 2, 1))
    if rnnt_type == "regular":
        px = fix_for_boundary(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def _log_sigmoid(x):
    return (np.minimum(x, 0) - np.log1p(np.exp(-np.abs(x)))).astype(x.dtype)


def hat_logprobs_pruned(logits, symbols, ranges, termination_symbol, boundary,
                        rnnt_type="regular"):
    """k2/python/k2/rnnt_loss.py:992-1177 (get_hat_logprobs_pruned)."""
    assert logits.ndim == 4
    B, T, R, C = logits.shape
    assert ranges.shape == (B, T, R)
    S = symbols.shape[1]
    assert symbols.shape == (B, S)
    assert rnnt_type != "modified" or T >= S
    assert rnnt_type in ("regular", "modified", "constrained")
    assert termination_symbol == 0
    dt = logits.dtype
    logp_b = _log_sigmoid(logits[..., 0])                     # [B,T,R]
    nb_normalizers = _logsumexp_last(logits[..., 1:])         # [B,T,R]
    nb_shift = logp_b - logits[..., 0]
    sym_ext = np.concatenate([symbols, np.zeros((B, 1), dtype=np.int64)], axis=1)
    pruned_symbols = sym_ext[np.arange(B)[:, None, None], ranges]
    px = np.take_along_axis(logits, pruned_symbols[..., None], axis=3)[..., 0]
    px = px - nb_normalizers + nb_shift
    px = np.concatenate([px, np.full((B, T, S + 1 - R), -np.inf, dtype=dt)], axis=2)
    px = roll_by_shifts(px, ranges[:, :, 0])[:, :, :S]
    px = px.transpose(0, 2, 1)
    if rnnt_type == "regular":
        px = np.concatenate([px, np.full((B, S, 1), -np.inf, dtype=dt)], axis=2)
    px = np.ascontiguousarray(px)
    py = np.concatenate([logp_b, np.full((B, T, S + 1 - R), -np.inf, dtype=dt)], axis=2)
    py = roll_by_shifts(py, ranges[:, :, 0])
    py = np.ascontiguousarray(py.transpose(0, 2, 1))
    if rnnt_type == "regular":
        px = fix_for_boundary(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def logprobs_smoothed(lm, am, symbols, termination_symbol, lm_only_scale=0.1, am_only_scale=0.1,
                      boundary=None, rnnt_type="regular"):
    """k2/python/k2/rnnt_loss.py:1471-1704 (get_rnnt_logprobs_smoothed)."""
    B, T, C = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S)
    validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    dt = am.dtype
    tiny = np.finfo(dt).tiny
    am_max = am.max(axis=2, keepdims=True)
    lm_max = lm.max(axis=2, keepdims=True)
    am_probs = np.exp(am - am_max)
    lm_probs = np.exp(lm - lm_max)
    normalizers = np.log(np.matmul(lm_probs, am_probs.transpose(0, 2, 1)) + tiny)
    lmonly = lm_probs.sum(axis=2, keepdims=True)                          # [B,S+1,1]
    unigram = (lm_probs / lmonly).mean(axis=(0, 1), keepdims=True) + tiny  # [1,1,C]
    amonly = np.log(am_probs.reshape(-1, C) @ unigram.reshape(C)).reshape(B, T, 1) + am_max
    amonly = amonly.transpose(0, 2, 1)                                     # [B,1,T]
    unigram = np.log(unigram)
    lmonly = np.log(lmonly) + lm_max
    normalizers = (normalizers + lm_max + am_max.transpose(0, 2, 1)).astype(dt)

    bi = np.arange(B)[:, None, None]
    px_am = am[bi, np.arange(T)[None, None, :], symbols[:, :, None]]
    if rnnt_type == "regular":
        px_am = np.concatenate([px_am, np.full((B, S, 1), -np.inf, dtype=dt)], axis=2)
    px_lm = lm[bi, np.arange(S)[None, :, None], symbols[:, :, None]]       # [B,S,1]
    px_lm_unigram = unigram[0, 0][symbols][:, :, None]                     # [B,S,1]
    px = (px_am + px_lm).astype(dt)
    px[:, :, :T] -= normalizers[:, :S, :]
    px_amonly = (px_am + px_lm_unigram).astype(dt)
    px_amonly[:, :, :T] -= amonly
    px_lmonly = px_lm - lmonly[:, :S, :]
    py_am = am[:, :, termination_symbol][:, None, :]
    py_lm = lm[:, :, termination_symbol][:, :, None]
    py = py_am + py_lm - normalizers
    py_amonly = py_am + unigram[0, 0, termination_symbol] - amonly
    py_lmonly = py_lm - lmonly
    combined = 1.0 - lm_only_scale - am_only_scale
    if lm_only_scale == 0.0:
        lm_only_scale = 1.0e-20
    if am_only_scale == 0.0:
        am_only_scale = 1.0e-20
    with np.errstate(invalid="ignore"):
        px_i = (px * combined + px_lmonly * lm_only_scale + px_amonly * am_only_scale).astype(dt)
        py_i = (py * combined + py_lmonly * lm_only_scale + py_amonly * am_only_scale).astype(dt)
    if rnnt_type == "regular":
        px_i = fix_for_boundary(px_i, boundary)
    elif rnnt_type == "constrained":
        px_i += py_i[:, 1:, :]
    return px_i, py_i


def prune_ranges_deprecated(px_grad, py_grad, boundary, s_range):
    """k2/python/k2/rnnt_loss.py:786-910 (get_rnnt_prune_ranges_deprecated)."""
    B, S, T1 = px_grad.shape
    T = py_grad.shape[-1]
    assert T1 in (T, T + 1)
    if s_range > S:
        s_range = S + 1
    dt = px_grad.dtype
    py_p = py_grad if T1 == T else np.concatenate(
        [py_grad, np.zeros((B, S + 1, 1), dtype=dt)], axis=2)
    tot = np.concatenate([px_grad, np.zeros((B, 1, T1), dtype=dt)], axis=1) + py_p
    tot = np.concatenate([np.zeros((B, 1, T1), dtype=dt), tot], axis=1)
    # torch's CPU cumsum accumulates fp32 input in double and rounds each prefix once
    tot = np.cumsum(tot, axis=1, dtype=np.float64).astype(dt)
    diff = tot[:, s_range:, :] - tot[:, :-s_range, :]
    s_begin = np.argmax(diff, axis=1).astype(np.int64)[:, :T]
    mask = np.arange(T)[None, :] < (boundary[:, 3][:, None] - 1)
    pad = np.maximum(boundary[:, 2][:, None] - s_range + 1, 0)
    s_begin = np.where(mask, s_begin, pad)
    s_begin = adjust_pruning_lower_bound(s_begin, 2 if T1 == T else s_range)
    return (s_begin[:, :, None] + np.arange(s_range, dtype=np.int64)[None, None, :]).astype(np.int64)


def apply_delay_penalty(px, boundary, rnnt_type, delay_penalty):
    """k2/python/k2/rnnt_loss.py:307-322 (same block at :509-528 and :1441-1456)."""
    if not delay_penalty > 0.0:
        return px
    B, S, T0 = px.shape
    T = T0 if rnnt_type != "regular" else T0 - 1
    if boundary is None:
        offset = np.full((B,), (T - 1) / 2, dtype=px.dtype)
    else:
        # integer tensor true-divided by 2: torch yields float32
        offset = ((boundary[:, 3] - 1) / 2).astype(np.float32)
    penalty = offset.reshape(B, 1, 1) - np.arange(T0).reshape(1, 1, T0).astype(offset.dtype)
    penalty = penalty * offset.dtype.type(delay_penalty)
    px += penalty.astype(px.dtype)
    return px


def _reduce(negated_loss, reduction):
    if reduction == "none":
        return -negated_loss
    if reduction == "mean":
        return -np.mean(negated_loss)
    if reduction == "sum":
        return -np.sum(negated_loss)
    raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")


def rnnt_loss_simple(lm, am, symbols, termination_symbol, boundary=None, rnnt_type="regular",
                     delay_penalty=0.0, reduction="mean", return_grad=False):
    """k2/python/k2/rnnt_loss.py:228-338."""
    px, py = logprobs_simple(lm, am, symbols, termination_symbol, rnnt_type, boundary)
    px = apply_delay_penalty(px, boundary, rnnt_type, delay_penalty)
    ans, gx, gy = _mi.mi(px, py, boundary)
    loss = _reduce(ans, reduction)
    return (loss, (gx, gy)) if return_grad else loss


def rnnt_loss(logits, symbols, termination_symbol, boundary=None, rnnt_type="regular",
              delay_penalty=0.0, reduction="mean"):
    """k2/python/k2/rnnt_loss.py:450-540."""
    px, py = logprobs_joint(logits, symbols, termination_symbol, rnnt_type, boundary)
    px = apply_delay_penalty(px, boundary, rnnt_type, delay_penalty)
    ans, _ = _mi.mi_forward(px, py, boundary)
    return _reduce(ans, reduction)


def rnnt_loss_smoothed(lm, am, symbols, termination_symbol, lm_only_scale=0.1, am_only_scale=0.1,
                       boundary=None, rnnt_type="regular", delay_penalty=0.0, reduction="mean"):
    """k2/python/k2/rnnt_loss.py:1707-1829."""
    px, py = logprobs_smoothed(lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale,
                               boundary, rnnt_type)
    px = apply_delay_penalty(px, boundary, rnnt_type, delay_penalty)
    ans, _ = _mi.mi_forward(px, py, boundary)
    return _reduce(ans, reduction)


def rnnt_loss_pruned(logits, symbols, ranges, termination_symbol, boundary=None,
                     rnnt_type="regular", delay_penalty=0.0, reduction="mean",
                     use_hat_loss=False):
    """k2/python/k2/rnnt_loss.py:1351-1468."""
    builder = hat_logprobs_pruned if use_hat_loss else logprobs_pruned
    px, py = builder(logits, symbols, ranges, termination_symbol, boundary, rnnt_type)
    px = apply_delay_penalty(px, boundary, rnnt_type, delay_penalty)
    ans, _ = _mi.mi_forward(px, py, boundary)
    return _reduce(ans, reduction)
