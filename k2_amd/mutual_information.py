"""Drop-in for k2/python/k2/mutual_information.py on MI355X.

Same function names, argument meaning, return values and exception classes as the reference;
the two native calls ``_k2.mutual_information_forward/backward`` are replaced by the HIP
kernels of libk2amd.so.  Tensors must live on a ROCm device: there is no CPU fallback.
"""
import weakref
from typing import List, Optional, Sequence, Tuple, Union

import torch
from torch import Tensor

from . import native


# host copies of boundary tensors: id(tensor) -> (weak reference, version counter, rows)
_boundary_copies = {}


def boundary_rows(boundary: Tensor) -> Tuple[Tuple[int, int, int, int], ...]:
    """The rows (s_begin, t_begin, s_end, t_end) of a [B][4] boundary tensor as Python integers.
    Reading them from a device tensor is a copy that waits for everything queued on the stream,
    and the reference pays it in each of its checks (k2/python/k2/mutual_information.py:284-289,
    k2/python/k2/rnnt_loss.py:46-62 and 699-705).  Here the copy is kept per tensor object and
    reused by all of them while the tensor has not been written to (its version counter); a new
    tensor is always read."""
    ident = id(boundary)
    hit = _boundary_copies.get(ident)
    if hit is not None and hit[0]() is boundary and hit[1] == boundary._version:
        return hit[2]
    early = _boundary_reads.pop(ident, None)
    if early is not None and early[0]() is boundary and early[1] == boundary._version:
        rows = early[2].rows()  # waits for the copy alone, not for what was queued after it
    elif boundary.is_cuda and boundary.dtype == torch.int64 and boundary.dim() == 2 and boundary.shape[1] == 4:
        # the same read, begun and waited for here: what rides along with it (the error flag of the
        # stream's workspace, native.boundary_read) is looked at in every call that reads a boundary
        rows = native.boundary_read(boundary).rows()
    else:
        rows = tuple(tuple(r) for r in boundary.tolist())
    _boundary_copies[ident] = (weakref.ref(boundary, lambda _, i=ident: _boundary_copies.pop(i, None)),
                               boundary._version, rows)
    return rows


# copies to the host under way: id(tensor) -> (weak reference, version counter, native.boundary_read)
_boundary_reads = {}


def begin_boundary_read(boundary: Optional[Tensor]) -> None:
    """Starts the copy that boundary_rows needs, without waiting for it: a loss function calls this
    before it queues the kernels that do not depend on the boundary's values being valid (a
    non-blocking copy into pinned memory and an event behind it), so that
    the checks after them (k2/python/k2/mutual_information.py:284-289, which the reference reaches
    after get_rnnt_logprobs' kernels too, k2/python/k2/rnnt_loss.py:295-330) find the rows on the
    host instead of waiting for those kernels and leaving the device idle meanwhile.  Nothing to do
    for a tensor whose rows are already here, and for host tensors."""
    if boundary is None or not boundary.is_cuda:
        return
    ident = id(boundary)
    hit = _boundary_copies.get(ident)
    if hit is not None and hit[0]() is boundary and hit[1] == boundary._version:
        return
    _boundary_reads[ident] = (weakref.ref(boundary, lambda _, i=ident: _boundary_reads.pop(i, None)),
                              boundary._version, native.boundary_read(boundary))


def _check_boundary(boundary: Tensor, S: int, T: int) -> None:
    """The range asserts of k2/python/k2/mutual_information.py:284-289."""
    for s_begin, t_begin, s_end, t_end in boundary_rows(boundary):
        assert 0 <= s_begin <= s_end <= S, (s_begin, s_end, S)
        assert 0 <= t_begin <= t_end <= T, (t_begin, t_end, T)


_single_launch_ok = {}


def _single_launch(px: Tensor, py: Tensor) -> bool:
    """Whether both recursions of these inputs run in one launch: where the native layer serves it
    and says it is the faster way on the device (asked once per shape, dtype and device)."""
    key = (px.shape, py.shape[-1], px.dtype, px.device)
    ok = _single_launch_ok.get(key)
    if ok is None:
        ok = _single_launch_ok[key] = bool(native.mutual_information_forward_backward_advised(px, py))
    return ok


def _lattice_buffers(px: Tensor, py: Tensor, want_grad: bool) -> Tuple[Optional[Tensor], Optional[Tensor]]:
    """(p, log_deriv) for a forward call that a backward call may follow: the [B][S+1][T+1]
    buffer the reference allocates as ``p`` (k2/python/k2/mutual_information.py:157) is handed over
    as ``log_deriv`` instead where the kernels pass the px-edge log-derivatives along."""
    (B, S, _), T = px.shape, py.shape[-1]
    buf = torch.empty(B, S + 1, T + 1, device=px.device, dtype=px.dtype)
    if want_grad and native.mutual_information_keeps_log_deriv(px, py):
        return None, buf
    return buf, None


def recursion_values(px: Tensor, py: Tensor, boundary: Optional[Tensor], want_grad: bool):
    """(scores, px_grad, py_grad) of contiguous px, py: the recursion and, when gradients may be
    wanted, the backward recursion with ans_grad = 1 straight away, as the reference's Function does
    (k2/python/k2/mutual_information.py:157-169).  No autograd here: the Function below and the
    loss nodes of rnnt_loss.py, which are autograd nodes themselves, both call it."""
    B = px.shape[0]
    px_grad, py_grad = None, None
    if want_grad and _single_launch(px, py):
        # both recursions in one launch, seeded with 1 per sequence
        (ans, px_grad, py_grad) = native.mutual_information_forward_backward(px, py, boundary, None)
    else:
        # the backward runs right away, so the forward can hand it the px-edge log-derivatives
        # instead of p (which nothing else reads)
        p, log_deriv = _lattice_buffers(px, py, want_grad)
        ans = native.mutual_information_forward(px, py, boundary, p, log_deriv)
        if want_grad:
            ans_grad = torch.ones(B, device=px.device, dtype=px.dtype)
            (px_grad, py_grad) = native.mutual_information_backward(px, py, boundary, p, ans_grad,
                                                                    log_deriv)
    return ans, px_grad, py_grad


def check_recursion_inputs(px: Tensor, py: Tensor, boundary: Optional[Tensor]) -> None:
    """The asserts of k2/python/k2/mutual_information.py:268-289."""
    assert px.ndim == 3, px.shape
    B, S, T1 = px.shape
    T = py.shape[-1]
    assert px.shape[-1] in [T, T + 1], (px.shape, T)
    assert py.shape == (B, S + 1, T), (py.shape, B, S, T)
    assert px.dtype == py.dtype, (px.dtype, py.dtype)
    if boundary is not None:
        assert boundary.dtype == torch.int64, boundary.dtype
        assert boundary.shape == (B, 4), (boundary.shape, B)
        _check_boundary(boundary, S, T)


class MutualInformationRecursionFunction(torch.autograd.Function):
    """Mirrors k2/python/k2/mutual_information.py:24-182: the forward runs the recursion and, when
    gradients may be wanted, the backward recursion with ans_grad = 1 straight away; autograd's
    backward then only scales the saved occupation probabilities."""

    @staticmethod
    def forward(ctx, px: Tensor, py: Tensor, pxy_grads: List[Optional[Tensor]],
                boundary: Optional[Tensor] = None, return_grad: bool = False) -> Tensor:
        (B, S, T1) = px.shape
        T = py.shape[-1]
        assert T1 in [T, T + 1], (T1, T)
        assert py.shape == (B, S + 1, T), (py.shape, S, T)
        if boundary is not None:
            assert boundary.shape == (B, 4), (boundary.shape, B)

        want_grad = return_grad or px.requires_grad or py.requires_grad
        ans, px_grad, py_grad = recursion_values(px, py, boundary, want_grad)
        if want_grad:
            ctx.save_for_backward(px_grad, py_grad)
        assert len(pxy_grads) == 2, len(pxy_grads)
        pxy_grads[0] = px_grad
        pxy_grads[1] = py_grad
        return ans

    @staticmethod
    def backward(ctx, ans_grad: Tensor) -> Tuple[Tensor, Tensor, None, None, None]:
        (px_grad, py_grad) = ctx.saved_tensors
        (B,) = ans_grad.shape
        ans_grad = ans_grad.reshape(B, 1, 1)
        return (px_grad * ans_grad, py_grad * ans_grad, None, None, None)


def mutual_information_recursion(
    px: Tensor,
    py: Tensor,
    boundary: Optional[Tensor] = None,
    return_grad: bool = False,
) -> Union[Tuple[Tensor, Tuple[Tensor, Tensor]], Tensor]:
    """k2.mutual_information_recursion (k2/python/k2/mutual_information.py:185-298).

    px: [B][S][T+1] (regular) or [B][S][T] (modified: inferred from the shape); py: [B][S+1][T];
    boundary: optional int64 [B][4] = (s_begin, t_begin, s_end, t_end).  Returns scores [B], or
    (scores, (px_grad, py_grad)) when return_grad is set, the grads being the occupation
    probabilities d scores.sum() / d px, py.
    """
    check_recursion_inputs(px, py, boundary)
    px, py = px.contiguous(), py.contiguous()
    pxy_grads = [None, None]
    scores = MutualInformationRecursionFunction.apply(px, py, pxy_grads, boundary, return_grad)
    px_grad, py_grad = pxy_grads
    return (scores, (px_grad, py_grad)) if return_grad else scores


class _JointProducts(torch.autograd.Function):
    """prods [N][B] = sum_k px_grad[b][k] * clamp(px[n][b][k]) + the same over py, clamp(v) =
    max(v, most negative finite value): the split of the joint score, one native pass over every
    tensor where the reference stacks, clamps, multiplies and sums with torch ops
    (k2/python/k2/mutual_information.py:404-417).  Differentiable in the inputs like that chain
    (the occupation probabilities are constants there, too)."""

    @staticmethod
    def forward(ctx, px_grad, py_grad, *inputs):
        N = len(inputs) // 2
        px, py = inputs[:N], inputs[N:]
        ctx.save_for_backward(px_grad, py_grad, *inputs)
        return native.mutual_information_joint_products([x.contiguous() for x in px],
                                                        [y.contiguous() for y in py], px_grad, py_grad)

    @staticmethod
    def backward(ctx, g):  # g [N][B]
        px_grad, py_grad = ctx.saved_tensors[:2]
        inputs = ctx.saved_tensors[2:]
        N = len(inputs) // 2
        lowest = torch.finfo(px_grad.dtype).min
        grads = []
        for i, v in enumerate(inputs):
            if not ctx.needs_input_grad[2 + i]:
                grads.append(None)
                continue
            occupation = px_grad if i < N else py_grad
            # d clamp(v) / d v = 1 where v >= lowest (torch.clamp's own rule), else 0
            grads.append(torch.where(v >= lowest, g[i % N].reshape(-1, 1, 1) * occupation,
                                     torch.zeros((), dtype=v.dtype, device=v.device)))
        return (None, None) + tuple(grads)


def _inner_product(a: Tensor, b: Tensor) -> Tensor:
    """Batched dot product over the last axis: [..., N] x [..., N] -> [...]."""
    return (a * b).sum(dim=-1)


def joint_mutual_information_recursion(
    px: Sequence[Tensor],
    py: Sequence[Tensor],
    boundary: Optional[Tensor] = None,
) -> Sequence[Tensor]:
    """k2.joint_mutual_information_recursion (k2/python/k2/mutual_information.py:314-423): runs
    the recursion on the sums of the given px / py and splits the total score over the N inputs
    with the occupation probabilities, so that the result summed over N equals the joint score."""
    N = len(px)
    assert len(py) == N and N > 0
    B, S, T1 = px[0].shape
    T = py[0].shape[-1]
    assert T1 in [T, T + 1]
    for x in px:
        assert x.shape == (B, S, T1) and x.dtype == px[0].dtype
    for y in py:
        assert y.shape == (B, S + 1, T) and y.dtype == px[0].dtype
    if boundary is not None:
        assert boundary.dtype == torch.int64
        assert boundary.shape == (B, 4)
        _check_boundary(boundary, S, T)

    fused = N <= native.JOINT_MAX_INPUTS and B > 0
    if fused:  # the sum of the inputs without a stacked copy of them (nothing differentiates it)
        with torch.no_grad():
            px_tot, py_tot = px[0], py[0]
            for x, y in zip(px[1:], py[1:]):
                px_tot, py_tot = px_tot + x, py_tot + y
            px_tot, py_tot = px_tot.contiguous(), py_tot.contiguous()
    else:
        px_cat = torch.stack(list(px), dim=0)  # [N][B][S][T1]
        py_cat = torch.stack(list(py), dim=0)  # [N][B][S+1][T]
        px_tot = px_cat.sum(dim=0).contiguous()
        py_tot = py_cat.sum(dim=0).contiguous()
    if _single_launch(px_tot, py_tot):
        (tot_probs, px_grad, py_grad) = native.mutual_information_forward_backward(
            px_tot, py_tot, boundary, None)
    else:
        ans_grad = torch.ones(B, device=px_tot.device, dtype=px_tot.dtype)
        p, log_deriv = _lattice_buffers(px_tot, py_tot, True)
        tot_probs = native.mutual_information_forward(px_tot, py_tot, boundary, p, log_deriv)
        (px_grad, py_grad) = native.mutual_information_backward(px_tot, py_tot, boundary, p, ans_grad,
                                                                log_deriv)
    # -inf inputs carry zero occupation: clamp them to the most negative finite value so that
    # 0 * -inf does not produce NaN (k2/python/k2/mutual_information.py:410-411)
    if fused:
        prods = _JointProducts.apply(px_grad, py_grad, *px, *py)  # [N][B]
    else:
        lowest = torch.finfo(px_cat.dtype).min
        x_prods = _inner_product(px_grad.reshape(1, B, -1), px_cat.reshape(N, B, -1).clamp(min=lowest))
        y_prods = _inner_product(py_grad.reshape(1, B, -1), py_cat.reshape(N, B, -1).clamp(min=lowest))
        prods = x_prods + y_prods  # [N][B]
    # the first element absorbs the gap between the sum of logs and the log of the sum
    with torch.no_grad():
        offset = tot_probs - prods.sum(dim=0)
    prods[0] += offset
    return prods
