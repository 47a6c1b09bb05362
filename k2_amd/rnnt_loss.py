"""Drop-in for the RNN-T loss functions of k2/python/k2/rnnt_loss.py on MI355X.

Function names, arguments, return values, warnings and exception classes follow the reference.
Where the reference chains 15-25 torch ops per call, each builder here is one fused HIP kernel
(plus its hand-written backward), reached through a torch.autograd.Function so that
``loss.backward()`` works as before.  Tensors must live on a ROCm device.
"""
import os
from typing import Optional, Tuple, Union

import torch
from torch import Tensor

from . import capi, native
from .mutual_information import (begin_boundary_read, boundary_rows, check_recursion_inputs,
                                 mutual_information_recursion, recursion_values)

_RNNT_TYPES = ("regular", "modified", "constrained")


def _dev_i64(t: Optional[Tensor], like: Tensor) -> Optional[Tensor]:
    if t is None:
        return None
    assert t.dtype == torch.int64, t.dtype
    return t.to(like.device).contiguous()


def fix_for_boundary(px: Tensor, boundary: Optional[Tensor] = None) -> Tensor:
    """k2/python/k2/rnnt_loss.py:25-43: px[b, :, boundary[b, 3]] = -inf, in place (the fused
    builders below already do this; kept for callers that build px themselves)."""
    if boundary is None:
        return px
    B, S, T1 = px.shape
    index = boundary[:, 3].reshape(B, 1, 1).expand(B, S, T1)
    return px.scatter_(dim=2, index=index, value=float("-inf"))


def _validate_st_lengths(S: int, T: int, is_rnnt_type_regular: bool,
                         boundary: Optional[Tensor] = None):
    """k2/python/k2/rnnt_loss.py:46-62."""
    assert S >= 0, S
    if boundary is None:
        assert is_rnnt_type_regular or T >= S, \
            f"Modified transducer requires T >= S, but got T={T} and S={S}"
    else:
        assert is_rnnt_type_regular or all(r[3] >= r[2] for r in boundary_rows(boundary)), \
            f"Modified transducer requires T >= S, but got T={boundary[:, 3]} and S={boundary[:, 2]}"


def _trunc_div(a: int, b: int) -> int:
    """Integer quotient rounded towards zero, like torch.div(..., rounding_mode="trunc")."""
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


class _LogprobsSimple(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lm, am, symbols, termination_symbol, rnnt_code, boundary):
        lm_c, am_c = lm.contiguous(), am.contiguous()
        px, py, saved = native.logprobs_simple_forward(lm_c, am_c, symbols, termination_symbol,
                                                     rnnt_code, boundary)
        ctx.save_for_backward(*saved)
        ctx.meta = (symbols, boundary, termination_symbol, rnnt_code)
        return px, py

    @staticmethod
    def backward(ctx, px_grad, py_grad):
        symbols, boundary, termination_symbol, rnnt_code = ctx.meta
        lm_grad, am_grad = native.logprobs_simple_backward(
            px_grad.contiguous(), py_grad.contiguous(), symbols, boundary, ctx.saved_tensors,
            termination_symbol, rnnt_code)
        return lm_grad, am_grad, None, None, None, None


class _LogprobsSmoothed(torch.autograd.Function):
    """get_rnnt_logprobs_smoothed in the library's kernels: the simple builder, then the marginal
    terms and the mix (k2_amd/csrc/rnnt_smoothed.hip)."""

    @staticmethod
    def forward(ctx, lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale, rnnt_code, boundary):
        px, py, saved = native.logprobs_smoothed_forward(lm.contiguous(), am.contiguous(), symbols,
                                                        termination_symbol, lm_only_scale, am_only_scale,
                                                        rnnt_code, boundary)
        ctx.save_for_backward(*saved)
        ctx.meta = (symbols, boundary, termination_symbol, lm_only_scale, am_only_scale, rnnt_code)
        return px, py

    @staticmethod
    def backward(ctx, px_grad, py_grad):
        symbols, boundary, termination_symbol, lm_only_scale, am_only_scale, rnnt_code = ctx.meta
        lm_grad, am_grad = native.logprobs_smoothed_backward(
            px_grad.contiguous(), py_grad.contiguous(), symbols, boundary, ctx.saved_tensors,
            termination_symbol, lm_only_scale, am_only_scale, rnnt_code)
        return lm_grad, am_grad, None, None, None, None, None, None


def smoothed_kernels_enabled() -> bool:
    """The marginal terms of get_rnnt_logprobs_smoothed have two implementations on the device:
    torch ops (the default) and the library's own kernels, which so far have run only in their
    host-thread build (tests/test_cpu_build_smoothed.py), never on a GPU; K2AMD_SMOOTHED_KERNELS=1
    selects them."""
    return os.environ.get("K2AMD_SMOOTHED_KERNELS", "0") == "1"


class _LogprobsJoint(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, symbols, termination_symbol, rnnt_code, boundary):
        logits_c = logits.contiguous()
        px, py, norm = native.logprobs_joint_forward(logits_c, symbols, termination_symbol,
                                                   rnnt_code, boundary)
        ctx.save_for_backward(logits_c, norm)
        ctx.meta = (symbols, boundary, termination_symbol, rnnt_code)
        return px, py

    @staticmethod
    def backward(ctx, px_grad, py_grad):
        symbols, boundary, termination_symbol, rnnt_code = ctx.meta
        logits, norm = ctx.saved_tensors
        grad = native.logprobs_joint_backward(logits, norm, px_grad.contiguous(),
                                            py_grad.contiguous(), symbols, boundary,
                                            termination_symbol, rnnt_code)
        return grad, None, None, None, None


class _LogprobsPruned(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, symbols, ranges, termination_symbol, rnnt_code, boundary, hat=False):
        logits_c = logits.contiguous()
        px, py, norm = native.logprobs_pruned_forward(logits_c, symbols, ranges, termination_symbol,
                                                      boundary, rnnt_code, hat)
        ctx.save_for_backward(logits_c, norm)
        ctx.meta = (symbols, ranges, boundary, termination_symbol, rnnt_code, hat)
        return px, py

    @staticmethod
    def backward(ctx, px_grad, py_grad):
        symbols, ranges, boundary, termination_symbol, rnnt_code, hat = ctx.meta
        logits, norm = ctx.saved_tensors
        grad = native.logprobs_pruned_backward(logits, norm, px_grad.contiguous(),
                                               py_grad.contiguous(), symbols, ranges, boundary,
                                               termination_symbol, rnnt_code, hat)
        return grad, None, None, None, None, None, None


class _Scores(torch.autograd.Function):
    """A builder above and the recursion on its px, py as ONE autograd node, for the loss functions:
    scores [B] straight from lm / am (``kind`` "simple") or logits ("joint", "pruned").  The
    recursion has the occupation probabilities ready when it returns (as the reference's does,
    k2/python/k2/mutual_information.py:162-169); what arrives at the scores in the backward pass
    scales them per sequence inside the builder's gradient kernels (``seq_scale``), where the
    reference runs two elementwise products first (mutual_information.py:177-182).  The node also
    negates and reduces the scores (the reference's last two torch ops, rnnt_loss.py:331-338), so
    that a loss is one graph node instead of three (2-4 us less host time per step, measured on
    one machine against the three-node form; the small configurations are bound by the host).
    Returns (loss, px_grad, py_grad); the last two are None unless asked for or needed."""

    @staticmethod
    def forward(ctx, kind, rnnt_type, delay_penalty, return_grad, reduction, *args):
        if reduction not in ("none", "mean", "sum"):
            raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")
        boundary = {"joint": 4, "joiner": 8}.get(kind, 5)
        boundary = args[boundary]
        begin_boundary_read(boundary)  # for check_recursion_inputs below, behind the builder's kernels
        need = return_grad or any(ctx.needs_input_grad)
        # no zero tensors for the gradients of px_grad / py_grad, which nothing differentiates
        ctx.set_materialize_grads(False)
        if kind == "simple":
            lm, am, symbols, termination_symbol, rnnt_code, _ = args
            px, py, saved = native.logprobs_simple_forward(lm.contiguous(), am.contiguous(), symbols,
                                                         termination_symbol, rnnt_code, boundary)
        elif kind == "smoothed":
            lm, am, symbols, termination_symbol, rnnt_code, _, lm_only_scale, am_only_scale = args
            px, py, saved = native.logprobs_smoothed_forward(lm.contiguous(), am.contiguous(), symbols,
                                                           termination_symbol, lm_only_scale, am_only_scale,
                                                           rnnt_code, boundary)
        elif kind == "joint":
            logits, symbols, termination_symbol, rnnt_code, _ = args
            logits = logits.contiguous()
            px, py, norm = native.logprobs_joint_forward(logits, symbols, termination_symbol,
                                                         rnnt_code, boundary)
            saved = (logits, norm)
        elif kind == "joiner":
            am, lm, ranges, weight, bias, symbols, termination_symbol, rnnt_code, _, precision, hat = args
            am, lm, weight = am.contiguous(), lm.contiguous(), weight.contiguous()
            bias = bias.contiguous() if bias is not None else None
            px, py, norm = native.joiner_pruned_forward(am, lm, ranges, weight, bias, symbols,
                                                        termination_symbol, boundary, rnnt_code, precision, hat)
            saved = (am, lm, weight, norm) + ((bias,) if bias is not None else ())
        else:
            logits, symbols, ranges, termination_symbol, rnnt_code, _, hat = args
            logits = logits.contiguous()
            px, py, norm = native.logprobs_pruned_forward(logits, symbols, ranges,
                                                          termination_symbol, boundary, rnnt_code, hat)
            saved = (logits, norm)
        if delay_penalty > 0.0:
            px = _delay_penalty(px, boundary, rnnt_type, delay_penalty)
        check_recursion_inputs(px, py, boundary)
        scores, px_grad, py_grad = recursion_values(px.contiguous(), py.contiguous(), boundary, need)
        ctx.kind, ctx.args, ctx.n_saved = kind, args, len(saved)
        ctx.reduction, ctx.batch = reduction, scores.shape[0]
        if need:
            ctx.save_for_backward(*saved, px_grad, py_grad)
            ctx.mark_non_differentiable(px_grad, py_grad)
        return _reduce(scores, reduction), px_grad, py_grad

    @staticmethod
    def backward(ctx, loss_grad, _px_grad_grad, _py_grad_grad):
        args = ctx.args
        if loss_grad is None:
            return (None,) * (5 + len(args))
        saved, (px_grad, py_grad) = ctx.saved_tensors[:ctx.n_saved], ctx.saved_tensors[ctx.n_saved:]
        # what reaches each sequence's score: the loss is minus the scores, their sum or their mean
        if ctx.reduction == "none":
            scale = loss_grad.neg()
        else:
            # (a division for the mean, as torch's own backward of it: the same bits; the op on the
            # expanded scalar writes the [B] tensor in one launch)
            scale = loss_grad.expand(ctx.batch)
            scale = (scale.neg() if ctx.reduction == "sum" else scale / float(-ctx.batch)).contiguous()
        if ctx.kind == "simple":
            _, _, symbols, termination_symbol, rnnt_code, boundary = args
            grads = native.logprobs_simple_backward(px_grad, py_grad, symbols, boundary, saved,
                                                    termination_symbol, rnnt_code, scale)
        elif ctx.kind == "smoothed":
            _, _, symbols, termination_symbol, rnnt_code, boundary, lm_only_scale, am_only_scale = args
            grads = native.logprobs_smoothed_backward(px_grad, py_grad, symbols, boundary, saved,
                                                      termination_symbol, lm_only_scale, am_only_scale,
                                                      rnnt_code, scale)
        elif ctx.kind == "joint":
            _, symbols, termination_symbol, rnnt_code, boundary = args
            grads = (native.logprobs_joint_backward(saved[0], saved[1], px_grad, py_grad, symbols,
                                                    boundary, termination_symbol, rnnt_code, scale),)
        elif ctx.kind == "joiner":
            _, _, ranges, _, bias, symbols, termination_symbol, rnnt_code, boundary, precision, hat = args
            am, lm, weight, norm = saved[:4]
            d_am, d_lm, d_w, d_b = native.joiner_pruned_backward(
                am, lm, ranges, weight, saved[4] if bias is not None else None, symbols,
                termination_symbol, boundary, rnnt_code, norm, px_grad, py_grad, scale, precision, hat)
            grads = (d_am, d_lm, None, d_w, d_b)
        else:
            _, symbols, ranges, termination_symbol, rnnt_code, boundary, hat = args
            grads = (native.logprobs_pruned_backward(saved[0], saved[1], px_grad, py_grad, symbols,
                                                     ranges, boundary, termination_symbol, rnnt_code,
                                                     hat, scale),)
        return (None, None, None, None, None) + tuple(grads) + (None,) * (len(args) - len(grads))


class _PruneGather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, lm, ranges):
        ctx.save_for_backward(ranges)
        ctx.S1 = lm.shape[1]
        return native.prune_gather(lm.contiguous(), ranges)

    @staticmethod
    def backward(ctx, grad):
        (ranges,) = ctx.saved_tensors
        return native.prune_gather_backward(grad.contiguous(), ranges, ctx.S1), None


def get_rnnt_logprobs(
    lm: Tensor,
    am: Tensor,
    symbols: Tensor,
    termination_symbol: int,
    rnnt_type: str = "regular",
    boundary: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """k2.get_rnnt_logprobs (k2/python/k2/rnnt_loss.py:65-225): lm [B][S+1][C], am [B][T][C],
    symbols [B][S] -> px [B][S][T+1 or T], py [B][S+1][T] for mutual_information_recursion."""
    return _LogprobsSimple.apply(*_simple_args(lm, am, symbols, termination_symbol, rnnt_type,
                                               boundary))


def _simple_args(lm, am, symbols, termination_symbol, rnnt_type, boundary):
    """The reference's checks (k2/python/k2/rnnt_loss.py:159-170) and the arguments of
    _LogprobsSimple."""
    assert lm.ndim == 3, lm.shape
    assert am.ndim == 3, am.shape
    assert lm.shape[0] == am.shape[0], (lm.shape, am.shape)
    assert lm.shape[2] == am.shape[2], (lm.shape, am.shape)
    (B, T, C) = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S), (symbols.shape, B, S)
    assert rnnt_type in _RNNT_TYPES, rnnt_type
    _validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    return (lm, am, _dev_i64(symbols, am), int(termination_symbol), capi.RNNT_TYPES[rnnt_type],
            _dev_i64(boundary, am))


def _delay_penalty(px: Tensor, boundary: Optional[Tensor], rnnt_type: str,
                   delay_penalty: float) -> Tensor:
    """The penalty block shared by the three losses (k2/python/k2/rnnt_loss.py:307-322):
    px[b,s,t] += ((T_b - 1) / 2 - t) * delay_penalty."""
    B, S, T0 = px.shape
    T = T0 if rnnt_type != "regular" else T0 - 1
    if boundary is None:
        offset = torch.tensor((T - 1) / 2, dtype=px.dtype, device=px.device).expand(B, 1, 1)
    else:
        offset = (boundary[:, 3] - 1) / 2
    penalty = offset.reshape(B, 1, 1) - torch.arange(T0, device=px.device).reshape(1, 1, T0)
    penalty = penalty * delay_penalty
    return px + penalty.to(px.dtype)


def _reduce(negated_loss: Tensor, reduction: Optional[str]) -> Tensor:
    if reduction == "none":
        return -negated_loss
    elif reduction == "mean":
        return -torch.mean(negated_loss)
    elif reduction == "sum":
        return -torch.sum(negated_loss)
    raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")


def rnnt_loss_simple(
    lm: Tensor,
    am: Tensor,
    symbols: Tensor,
    termination_symbol: int,
    boundary: Optional[Tensor] = None,
    rnnt_type: str = "regular",
    delay_penalty: float = 0.0,
    reduction: Optional[str] = "mean",
    return_grad: bool = False,
) -> Union[Tensor, Tuple[Tensor, Tuple[Tensor, Tensor]]]:
    """k2.rnnt_loss_simple (k2/python/k2/rnnt_loss.py:228-338)."""
    args = _simple_args(lm, am, symbols, termination_symbol, rnnt_type, boundary)
    loss, px_grad, py_grad = _Scores.apply("simple", rnnt_type, float(delay_penalty),
                                           bool(return_grad), reduction, *args)
    return (loss, (px_grad, py_grad)) if return_grad else loss


def get_rnnt_logprobs_joint(
    logits: Tensor,
    symbols: Tensor,
    termination_symbol: int,
    rnnt_type: str = "regular",
    boundary: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """k2.get_rnnt_logprobs_joint (k2/python/k2/rnnt_loss.py:341-447): logits [B][T][S+1][C]."""
    return _LogprobsJoint.apply(*_joint_args(logits, symbols, termination_symbol, rnnt_type, boundary))


def _joint_args(logits, symbols, termination_symbol, rnnt_type, boundary):
    """The reference's checks (k2/python/k2/rnnt_loss.py:400-408) and the arguments of
    _LogprobsJoint."""
    assert logits.ndim == 4, logits.shape
    (B, T, S1, C) = logits.shape
    S = S1 - 1
    assert symbols.shape == (B, S), (symbols.shape, B, S)
    assert rnnt_type in _RNNT_TYPES, rnnt_type
    _validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    return (logits, _dev_i64(symbols, logits), int(termination_symbol), capi.RNNT_TYPES[rnnt_type],
            _dev_i64(boundary, logits))


def rnnt_loss(
    logits: Tensor,
    symbols: Tensor,
    termination_symbol: int,
    boundary: Optional[Tensor] = None,
    rnnt_type: str = "regular",
    delay_penalty: float = 0.0,
    reduction: Optional[str] = "mean",
) -> Tensor:
    """k2.rnnt_loss (k2/python/k2/rnnt_loss.py:450-540)."""
    args = _joint_args(logits, symbols, termination_symbol, rnnt_type, boundary)
    return _Scores.apply("joint", rnnt_type, float(delay_penalty), False, reduction, *args)[0]


def get_rnnt_prune_ranges(
    px_grad: Tensor,
    py_grad: Tensor,
    boundary: Tensor,
    s_range: int,
) -> Tensor:
    """k2.get_rnnt_prune_ranges (k2/python/k2/rnnt_loss.py:636-780): int64 [B][T][s_range]."""
    (B, S, T1) = px_grad.shape
    T = py_grad.shape[-1]
    is_regular = T1 != T
    assert T1 in [T, T + 1], (T1, T)
    S1 = S + 1
    assert py_grad.shape == (B, S1, T), (py_grad.shape, B, S1, T)
    assert boundary.shape == (B, 4), (boundary.shape, B)
    _validate_st_lengths(S, T, is_regular, boundary)

    if is_regular:
        # the smallest s_range that lets a path take all S_b symbols in T_b frames, as
        # k2/python/k2/rnnt_loss.py:699-705 has it: max over b of trunc((S_b - 1) / T_b) + 2,
        # from the host copy of the boundary (a sequence without frames asks for nothing)
        s_range_min = max((_trunc_div(r[2] - 1, r[3]) + 2 for r in boundary_rows(boundary) if r[3] != 0),
                          default=2)
        if s_range < s_range_min:
            print(f"Warning: get_rnnt_prune_ranges - got s_range={s_range} "
                  f"for boundaries S={boundary[:, 2]}, T={boundary[:, 3]}. Adjusting to {s_range_min}")
            s_range = s_range_min
    if s_range > S:
        print(f"Warning: get_rnnt_prune_ranges - got s_range={s_range} "
              f"for boundaries S={S}. Adjusting to {S + 1}")
        s_range = S + 1
    if is_regular:
        assert s_range >= 2, \
            f"Pruning range for standard RNN-T should be equal to or greater than 2, " \
            f"or no valid paths could survive pruning. Given {s_range}"
    else:
        assert s_range >= 1, \
            f"Pruning range for modified RNN-T should be equal to or greater than 1, " \
            f"or no valid paths could survive pruning. Given {s_range}"
    return native.prune_ranges(px_grad.detach().contiguous(), py_grad.detach().contiguous(),
                             _dev_i64(boundary, px_grad), int(s_range))


def do_rnnt_pruning(am: Tensor, lm: Tensor, ranges: Tensor) -> Tuple[Tensor, Tensor]:
    """k2.do_rnnt_pruning (k2/python/k2/rnnt_loss.py:913-954): am_pruned is a broadcast view
    [B][T][s_range][E]; lm_pruned[b,t,k,:] = lm[b, ranges[b,t,k], :]."""
    assert ranges.shape[0] == am.shape[0], (ranges.shape, am.shape)
    assert ranges.shape[0] == lm.shape[0], (ranges.shape, lm.shape)
    assert am.shape[1] == ranges.shape[1], (am.shape, ranges.shape)
    (B, T, s_range) = ranges.shape
    (B, S1, decoder_dim) = lm.shape
    encoder_dim = am.shape[-1]
    assert am.shape == (B, T, encoder_dim), (am.shape, B, T, encoder_dim)
    am_pruned = am.unsqueeze(2).expand((B, T, s_range, encoder_dim))
    lm_pruned = _PruneGather.apply(lm, _dev_i64(ranges, lm))
    return am_pruned, lm_pruned


def _roll_by_shifts(src: Tensor, shifts: Tensor) -> Tensor:
    """k2/python/k2/rnnt_loss.py:957-989: out[b,t,s] = src[b,t,(s - shifts[b,t]) mod S] (the
    fused pruned builder applies this placement itself; kept for callers)."""
    assert src.dim() == 3, src.shape
    (B, T, S) = src.shape
    assert shifts.shape == (B, T), (shifts.shape, B, T)
    index = (torch.arange(S, device=src.device).view(1, 1, S) - shifts.reshape(B, T, 1)) % S
    return torch.gather(src, 2, index)


def get_rnnt_logprobs_pruned(
    logits: Tensor,
    symbols: Tensor,
    ranges: Tensor,
    termination_symbol: int,
    boundary: Tensor,
    rnnt_type: str = "regular",
) -> Tuple[Tensor, Tensor]:
    """k2.get_rnnt_logprobs_pruned (k2/python/k2/rnnt_loss.py:1180-1348): logits
    [B][T][s_range][C], ranges [B][T][s_range]."""
    return _LogprobsPruned.apply(*_pruned_args(logits, symbols, ranges, termination_symbol, boundary,
                                               rnnt_type))


def _pruned_args(logits, symbols, ranges, termination_symbol, boundary, rnnt_type):
    """The reference's checks (k2/python/k2/rnnt_loss.py:1243-1251) and the arguments of
    _LogprobsPruned."""
    assert logits.ndim == 4, logits.shape
    (B, T, s_range, C) = logits.shape
    assert ranges.shape == (B, T, s_range), (ranges.shape, B, T, s_range)
    (B, S) = symbols.shape
    assert rnnt_type in _RNNT_TYPES, rnnt_type
    _validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    return (logits, _dev_i64(symbols, logits), _dev_i64(ranges, logits), int(termination_symbol),
            capi.RNNT_TYPES[rnnt_type], _dev_i64(boundary, logits), False)


def get_hat_logprobs_pruned(
    logits: Tensor,
    symbols: Tensor,
    ranges: Tensor,
    termination_symbol: int,
    boundary: Tensor,
    rnnt_type: str = "regular",
) -> Tuple[Tensor, Tensor]:
    """k2.get_hat_logprobs_pruned (k2/python/k2/rnnt_loss.py:992-1177), the hybrid autoregressive
    transducer: the blank (column 0) has its own sigmoid, py = logsigmoid(logits[..., 0]), and the
    other symbols share a softmax over columns 1..C-1 scaled by 1 - sigmoid(logits[..., 0])."""
    return _LogprobsPruned.apply(*_hat_args(logits, symbols, ranges, termination_symbol, boundary,
                                            rnnt_type))


def _hat_args(logits, symbols, ranges, termination_symbol, boundary, rnnt_type):
    """The reference's checks (k2/python/k2/rnnt_loss.py:1056-1069) and the arguments of
    _LogprobsPruned."""
    assert logits.ndim == 4, logits.shape
    (B, T, s_range, C) = logits.shape
    assert ranges.shape == (B, T, s_range), (ranges.shape, B, T, s_range)
    (B, S) = symbols.shape
    assert S >= 0, S
    assert rnnt_type != "modified" or T >= S, \
        f"Modified transducer requires T >= S, but got T={T} and S={S}"
    assert rnnt_type in _RNNT_TYPES, rnnt_type
    assert termination_symbol == 0, \
        f"Termination symbol must be 0, but got {termination_symbol}"
    return (logits, _dev_i64(symbols, logits), _dev_i64(ranges, logits), 0,
            capi.RNNT_TYPES[rnnt_type], _dev_i64(boundary, logits), True)


def rnnt_loss_pruned(
    logits: Tensor,
    symbols: Tensor,
    ranges: Tensor,
    termination_symbol: int,
    boundary: Tensor = None,
    rnnt_type: str = "regular",
    delay_penalty: float = 0.0,
    reduction: Optional[str] = "mean",
    use_hat_loss: bool = False,
) -> Tensor:
    """k2.rnnt_loss_pruned (k2/python/k2/rnnt_loss.py:1351-1468); ``use_hat_loss`` switches the
    builder to get_hat_logprobs_pruned (:1430-1447)."""
    checked = _hat_args if use_hat_loss else _pruned_args
    args = checked(logits, symbols, ranges, termination_symbol, boundary, rnnt_type)
    return _Scores.apply("pruned", rnnt_type, float(delay_penalty), False, reduction, *args)[0]


def rnnt_loss_pruned_joiner(
    am: Tensor,
    lm: Tensor,
    ranges: Tensor,
    weight: Tensor,
    bias: Optional[Tensor],
    symbols: Tensor,
    termination_symbol: int,
    boundary: Tensor = None,
    rnnt_type: str = "regular",
    delay_penalty: float = 0.0,
    reduction: Optional[str] = "mean",
    precision: str = "fp32",
    use_hat_loss: bool = False,
) -> Tensor:
    """do_rnnt_pruning -> joiner -> rnnt_loss_pruned (k2/python/k2/rnnt_loss.py:913-954, the
    caller's joiner, :1351-1468) as one call for the usual joiner,

        logits = torch.nn.functional.linear(torch.tanh(am_pruned + lm_pruned), weight, bias),

    with am [B][T][D] and lm [B][S+1][D] the projected encoder / decoder outputs, ranges from
    get_rnnt_prune_ranges, weight [C][D] and bias [C] (or None) those of the output layer.  The
    [B][T][s_range][C] logits are never stored; gradients flow to am, lm, weight and bias.
    ``precision``: "fp32" multiplies in fp32; "bf16" rounds the activations, the weight and the logits'
    gradients to bfloat16 for the matrix products (fp32 accumulation), as autocast would.
    ``use_hat_loss``: as in rnnt_loss_pruned (k2/python/k2/rnnt_loss.py:1439-1447), the hybrid
    autoregressive transducer's log-probs, termination_symbol 0.  That variant of the kernels has
    so far run in its host-thread build only (tests/test_cpu_build_host_layer.py), never on a GPU:
    it is refused unless K2AMD_JOINER_HAT=1 is set; the three separate steps serve meanwhile."""
    if use_hat_loss:
        assert termination_symbol == 0, "the hybrid autoregressive transducer's blank is symbol 0"
        if os.environ.get("K2AMD_JOINER_HAT", "0") != "1":
            raise RuntimeError("k2_amd: rnnt_loss_pruned_joiner(use_hat_loss=True) has not run on a GPU yet and is "
                               "off by default: set K2AMD_JOINER_HAT=1 to use it, or call do_rnnt_pruning, the "
                               "joiner and rnnt_loss_pruned(use_hat_loss=True) one after the other")
    assert am.ndim == 3 and lm.ndim == 3, (am.shape, lm.shape)
    (B, T, D) = am.shape
    assert lm.shape[0] == B and lm.shape[2] == D, (am.shape, lm.shape)
    S = lm.shape[1] - 1
    assert ranges.ndim == 3 and ranges.shape[:2] == (B, T), (ranges.shape, B, T)
    assert weight.ndim == 2 and weight.shape[1] == D, (weight.shape, D)
    assert bias is None or bias.shape == (weight.shape[0],), (bias.shape, weight.shape)
    assert symbols.shape == (B, S), (symbols.shape, B, S)
    assert rnnt_type in _RNNT_TYPES, rnnt_type
    assert precision in capi.JOINER_PRECISIONS, precision
    _validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    args = (am, lm, _dev_i64(ranges, am), weight, bias, _dev_i64(symbols, am), int(termination_symbol),
            capi.RNNT_TYPES[rnnt_type], _dev_i64(boundary, am), capi.JOINER_PRECISIONS[precision],
            bool(use_hat_loss))
    return _Scores.apply("joiner", rnnt_type, float(delay_penalty), False, reduction, *args)[0]


def get_rnnt_logprobs_smoothed(
    lm: Tensor,
    am: Tensor,
    symbols: Tensor,
    termination_symbol: int,
    lm_only_scale: float = 0.1,
    am_only_scale: float = 0.1,
    boundary: Optional[Tensor] = None,
    rnnt_type: str = "regular",
) -> Tuple[Tensor, Tensor]:
    """k2.get_rnnt_logprobs_smoothed (k2/python/k2/rnnt_loss.py:1471-1704): interpolates, in the
    log domain, the joint log-probs with "lm only" log-probs and "am only" log-probs (the latter
    against a unigram lm averaged over the batch).

    The joint part (the only one of size [B][S+1][T] x C) is the fused kernel of
    get_rnnt_logprobs.  The two marginal parts, over [B][S+1][C] and [B][T][C], and the mix are a
    dozen torch ops on the device, or with K2AMD_SMOOTHED_KERNELS=1 the library's own kernels (see
    smoothed_kernels_enabled)."""
    assert lm.ndim == 3, lm.shape
    assert am.ndim == 3, am.shape
    assert lm.shape[0] == am.shape[0], (lm.shape, am.shape)
    assert lm.shape[2] == am.shape[2], (lm.shape, am.shape)
    (B, T, C) = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S), (symbols.shape, B, S)
    assert rnnt_type in _RNNT_TYPES, rnnt_type
    _validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    regular = rnnt_type == "regular"
    symbols = _dev_i64(symbols, am)
    blank = int(termination_symbol)
    if smoothed_kernels_enabled() and B > 0 and native.smoothed_supported(lm, am):
        return _LogprobsSmoothed.apply(lm, am, symbols, blank, float(lm_only_scale), float(am_only_scale),
                                       capi.RNNT_TYPES[rnnt_type], _dev_i64(boundary, am))

    # joint part, before the boundary fix / the "constrained" add (both come after interpolation)
    px, py = _LogprobsSimple.apply(lm, am, symbols, blank,
                                   capi.RNNT_TYPES["regular" if regular else "modified"], None)

    # The two marginal parts in probability space, as the reference defines them
    # (k2/python/k2/rnnt_loss.py:1608-1677), written with log_softmax (one kernel forward, one
    # backward) where the reference spells the max, the exponentials, their sum and its log out:
    #   lm only:  log softmax(lm)                                     [B][S+1][C]
    #   am only:  log softmax(am + log unigram), unigram = the batch's mean of softmax(lm) + tiny
    # (its normaliser log sum_c e^am unigram_c is exactly that log-softmax's).
    tiny = torch.finfo(lm.dtype).tiny
    lm_only = torch.log_softmax(lm, dim=2)                                   # [B][S+1][C]
    log_unigram = (lm_only.exp().mean(dim=(0, 1)) + tiny).log()              # [C]
    am_only = torch.log_softmax(am + log_unigram, dim=2)                     # [B][T][C]

    px_am_only = torch.gather(am_only.transpose(1, 2), 1, symbols.unsqueeze(2).expand(B, S, T))  # [B][S][T]
    if regular:  # no symbol can be emitted one past the last frame
        px_am_only = torch.nn.functional.pad(px_am_only, (0, 1), value=float("-inf"))
    px_lm_only = torch.gather(lm_only[:, :S], 2, symbols.unsqueeze(2))       # [B][S][1]
    py_am_only = am_only[:, :, blank].unsqueeze(1)                           # [B][1][T]
    py_lm_only = lm_only[:, :, blank].unsqueeze(2)                           # [B][S+1][1]

    joint_scale = 1.0 - lm_only_scale - am_only_scale
    lm_only_scale = 1.0e-20 if lm_only_scale == 0.0 else lm_only_scale
    am_only_scale = 1.0e-20 if am_only_scale == 0.0 else am_only_scale
    px_mix = torch.add(torch.add(px * joint_scale, px_lm_only, alpha=lm_only_scale), px_am_only,
                       alpha=am_only_scale)
    py_mix = torch.add(torch.add(py * joint_scale, py_lm_only, alpha=lm_only_scale), py_am_only,
                       alpha=am_only_scale)

    if regular:
        px_mix = fix_for_boundary(px_mix, _dev_i64(boundary, px_mix))
    elif rnnt_type == "constrained":
        px_mix = px_mix + py_mix[:, 1:, :]
    return px_mix, py_mix


def rnnt_loss_smoothed(
    lm: Tensor,
    am: Tensor,
    symbols: Tensor,
    termination_symbol: int,
    lm_only_scale: float = 0.1,
    am_only_scale: float = 0.1,
    boundary: Optional[Tensor] = None,
    rnnt_type: str = "regular",
    delay_penalty: float = 0.0,
    reduction: Optional[str] = "mean",
    return_grad: bool = False,
) -> Union[Tuple[Tensor, Tuple[Tensor, Tensor]], Tensor]:
    """k2.rnnt_loss_smoothed (k2/python/k2/rnnt_loss.py:1707-1829)."""
    if smoothed_kernels_enabled() and am.ndim == 3 and am.shape[0] > 0 and native.smoothed_supported(lm, am):
        # builder, recursion and reduction as one graph node, like the other losses
        args = _simple_args(lm, am, symbols, termination_symbol, rnnt_type, boundary)
        loss, px_grad, py_grad = _Scores.apply("smoothed", rnnt_type, float(delay_penalty), bool(return_grad),
                                               reduction, *args, float(lm_only_scale), float(am_only_scale))
        return (loss, (px_grad, py_grad)) if return_grad else loss
    px, py = get_rnnt_logprobs_smoothed(lm=lm, am=am, symbols=symbols,
                                        termination_symbol=termination_symbol,
                                        lm_only_scale=lm_only_scale, am_only_scale=am_only_scale,
                                        boundary=boundary, rnnt_type=rnnt_type)
    if delay_penalty > 0.0:
        px = _delay_penalty(px, boundary, rnnt_type, delay_penalty)
    scores_and_grads = mutual_information_recursion(px=px, py=py, boundary=boundary,
                                                    return_grad=return_grad)
    negated_loss = scores_and_grads[0] if return_grad else scores_and_grads
    loss = _reduce(negated_loss, reduction)
    return (loss, scores_and_grads[1]) if return_grad else loss


def get_rnnt_prune_ranges_deprecated(
    px_grad: Tensor,
    py_grad: Tensor,
    boundary: Tensor,
    s_range: int,
) -> Tensor:
    """k2.get_rnnt_prune_ranges_deprecated (k2/python/k2/rnnt_loss.py:786-910): the older rule,
    which picks for every frame the window of s_range rows with the largest total occupation
    px_grad + py_grad (prefix sums over s), then applies the same padding and monotonicity
    adjustment.  Two launches, like get_rnnt_prune_ranges (csrc/prune.hip)."""
    (B, S, T1) = px_grad.shape
    T = py_grad.shape[-1]
    assert T1 in [T, T + 1], (T1, T)
    assert py_grad.shape == (B, S + 1, T), (py_grad.shape, B, S + 1, T)
    assert boundary.shape == (B, 4), (boundary.shape, B)
    assert S >= 0, S
    if s_range > S:
        s_range = S + 1
    if T1 == T:
        assert s_range >= 1, \
            f"Pruning range for modified RNN-T should be equal to or greater than 1, " \
            f"or no valid paths could survive pruning. Given {s_range}"
    else:
        assert s_range >= 2, \
            f"Pruning range for standard RNN-T should be equal to or greater than 2, " \
            f"or no valid paths could survive pruning. Given {s_range}"
    # (the prefix sums over s are formed as torch.cumsum forms them on the CPU, where the
    # reference's values come from: accumulated in double, every prefix rounded once)
    return native.prune_ranges(px_grad.detach().contiguous(), py_grad.detach().contiguous(),
                               _dev_i64(boundary, px_grad), int(s_range), deprecated=True)
