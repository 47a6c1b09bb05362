"""The native entry points the Python layer calls, named after the reference's ``_k2`` functions.

Backed by the pybind11 host module ``_k2_amd`` (C++ host code over the C-ABI of libk2amd.so)
when it has been built, else by the ctypes binding of the same C-ABI (``capi.py``).  Either way the work runs
in the HIP kernels; a missing libk2amd.so raises, nothing falls back to the CPU.
"""
from typing import List, Optional

import torch

from . import capi

try:  # C++ host layer (k2_amd/csrc/pybind.cpp)
    from . import _k2_amd as _ext  # type: ignore
except ImportError:  # not built: the ctypes host is functionally identical
    _ext = None


def _require_device(t: torch.Tensor):
    if not t.is_cuda:
        raise RuntimeError(
            "k2_amd runs on MI355X only: got a tensor on %s (there is no CPU path)" % t.device)


class _BoundaryRead:
    """The host layer's BoundaryRead with torch's Python API, where the extension is not built:
    the copy of ``boundary`` to the host, and with it the error flag of the stream's workspace
    (a launch that gave up a bounded wait is reported by ``rows()`` as a RuntimeError, once, and
    the workspace initialised again)."""

    def __init__(self, boundary: torch.Tensor):
        self.pinned = torch.empty(boundary.shape, dtype=boundary.dtype, pin_memory=True)
        self.pinned.copy_(boundary, non_blocking=True)
        stream = torch.cuda.current_stream(boundary.device)
        self.key = (boundary.device.index, stream.cuda_stream)
        self.workspace = capi._workspaces.get(self.key)
        self.flag = None
        if self.workspace is not None:
            self.flag = torch.zeros(1, dtype=torch.int32, pin_memory=True)
            with torch.cuda.device(boundary.device):
                capi.check(capi.lib().k2amd_mi_workspace_status_async(
                    self.workspace.data_ptr(), self.flag.data_ptr(), self.key[1]))
        self.event = torch.cuda.Event()
        self.event.record(stream)

    def rows(self):
        self.event.synchronize()  # the copy alone, not what was queued after it
        if self.flag is not None and int(self.flag[0]) != 0:
            self.flag[0] = 0
            with torch.cuda.device(self.key[0]):
                capi.check(capi.lib().k2amd_mi_workspace_init(self.workspace.data_ptr(), self.workspace.numel(),
                                                              self.key[1]))
            raise RuntimeError(
                "k2_amd: in-kernel wait timed out: an earlier launch of the mutual-information kernels on this "
                "stream gave up waiting for a neighbouring workgroup, so its scores and gradients (NaN) are "
                "invalid; the workspace has been initialised again, the next call will work")
        return tuple(tuple(r) for r in self.pinned.tolist())


def boundary_read(boundary: torch.Tensor):
    """Starts the copy of a [B][4] int64 device tensor to the host without waiting for it;
    ``.rows()`` of the returned object waits for that copy alone and gives the rows as tuples of
    Python integers."""
    if _ext is not None and boundary.dtype == torch.int64 and boundary.dim() == 2 and boundary.shape[1] == 4:
        return _ext.BoundaryRead(boundary)
    return _BoundaryRead(boundary)


JOINT_MAX_INPUTS = capi.JOINT_MAX_INPUTS


def mutual_information_joint_products(px, py, px_grad: torch.Tensor, py_grad: torch.Tensor) -> torch.Tensor:
    """prods [N][B] = sum_k px_grad[b][k] * max(px[n][b][k], lowest finite) + the same over py: the
    split of a joint score over the N inputs of joint_mutual_information_recursion
    (k2/python/k2/mutual_information.py:404-417), every tensor read once."""
    _require_device(px_grad)
    if _ext is not None:
        return _ext.mutual_information_joint_products(list(px), list(py), px_grad, py_grad)
    return capi.mi_joint_products(list(px), list(py), px_grad, py_grad)


def mutual_information_recover_workspaces() -> int:
    """Waits for the streams that the pipelined fp32 kernels have run on and reads the error flag
    of each scratch buffer.  Where a kernel gave up a bounded wait (its scores came out as NaN,
    and so would those of every later call), the buffer is initialised again; returns how many
    were.  Call it when a loss turns NaN to tell that cause from the others."""
    if _ext is not None:
        return int(_ext.mutual_information_recover_workspaces())
    n = 0
    for key, ws in list(capi._workspaces.items()):
        with torch.cuda.device(key[0]):
            status = capi.lib().k2amd_mi_workspace_status(ws.data_ptr(), key[1])
            if status == 5:  # K2AMD_ERR_TIMEOUT
                capi.check(capi.lib().k2amd_mi_workspace_init(ws.data_ptr(), ws.numel(), key[1]))
                n += 1
            else:
                capi.check(status)
    return n


def mutual_information_keeps_log_deriv(px: torch.Tensor, py: torch.Tensor) -> bool:
    """True if the forward / backward pair below uses a ``log_deriv`` tensor for these inputs (the
    pipelined fp32 kernels do; the exact kernels leave it untouched, so allocating one is
    wasted)."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_keeps_log_deriv(px, py)
    return capi.mi_keeps_log_deriv(px, py)


def mutual_information_forward(px: torch.Tensor, py: torch.Tensor,
                               boundary: Optional[torch.Tensor], p: torch.Tensor,
                               log_deriv: Optional[torch.Tensor] = None) -> torch.Tensor:
    """_k2.mutual_information_forward (k2/python/csrc/torch/mutual_information.cu:26-44).
    ``log_deriv`` (not in the reference; shaped like ``p``) is filled with what lets the backward
    call on the same inputs read one tensor instead of three."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_forward(px, py, boundary, p, log_deriv)
    return capi.mi_forward(px.contiguous(), py.contiguous(),
                           None if boundary is None else boundary.contiguous(), p,
                           log_deriv=log_deriv)


def mutual_information_backward(px: torch.Tensor, py: torch.Tensor,
                                boundary: Optional[torch.Tensor], p: torch.Tensor,
                                ans_grad: torch.Tensor,
                                log_deriv: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
    """_k2.mutual_information_backward (k2/python/csrc/torch/mutual_information.cu:46-67);
    overwrites ``ans_grad`` like the reference's device path.  ``log_deriv``: the tensor the
    forward call on the same inputs filled, or None."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_backward(px, py, boundary, p, ans_grad, log_deriv)
    gx, gy = capi.mi_backward(px.contiguous(), py.contiguous(),
                              None if boundary is None else boundary.contiguous(), p, ans_grad,
                              overwrite_ans_grad=True, log_deriv=log_deriv)
    return [gx, gy]


def mutual_information_forward_backward_advised(px: torch.Tensor, py: torch.Tensor) -> bool:
    """True if mutual_information_forward_backward serves these inputs and is the faster way on
    their device (a compute unit for every half-sweep of the launch at once)."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_forward_backward_advised(px, py)
    return capi.mi_forward_backward_advised(px, py)


def mutual_information_forward_backward_supported(px: torch.Tensor, py: torch.Tensor) -> bool:
    """True if mutual_information_forward_backward serves these inputs on their device (fp32, the
    pipelined kernels' shapes)."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_forward_backward_supported(px, py)
    return capi.mi_forward_backward_supported(px, py)


def mutual_information_forward_backward(px: torch.Tensor, py: torch.Tensor,
                                        boundary: Optional[torch.Tensor],
                                        ans_grad: Optional[torch.Tensor]) -> List[torch.Tensor]:
    """mutual_information_forward followed by mutual_information_backward in one launch, as the
    reference's autograd function calls them (k2/python/k2/mutual_information.py:157-169):
    returns [ans, px_grad, py_grad] and overwrites ``ans_grad``; ``ans_grad`` None stands for the
    reference's torch.ones(B)."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_forward_backward(px, py, boundary, ans_grad)
    ans, gx, gy = capi.mi_forward_backward(px.contiguous(), py.contiguous(),
                                           None if boundary is None else boundary.contiguous(),
                                           ans_grad, overwrite_ans_grad=True)
    return [ans, gx, gy]


# ---- the fused builders (replacements of the torch-op chains of k2/python/k2/rnnt_loss.py) ----
# Same signatures and return values in both hosts; see capi.py for what each returns.

def logprobs_simple_forward(lm, am, symbols, termination_symbol, rnnt_type, boundary):
    _require_device(am)
    if _ext is not None:
        px, py, lm_probs, am_probs, denom = _ext.logprobs_simple_forward(
            lm, am, symbols, termination_symbol, rnnt_type, boundary)
        return px, py, (lm_probs, am_probs, denom)
    return capi.logprobs_simple_forward(lm, am, symbols, termination_symbol, rnnt_type, boundary)


def logprobs_simple_backward(px_grad, py_grad, symbols, boundary, saved, termination_symbol,
                             rnnt_type, seq_scale=None):
    """``seq_scale`` [B] or None (also in the two *_backward functions below): px_grad[b] and
    py_grad[b] count as multiplied by seq_scale[b]."""
    _require_device(px_grad)
    if _ext is not None:
        lm_probs, am_probs, denom = saved
        return tuple(_ext.logprobs_simple_backward(px_grad, py_grad, symbols, boundary, lm_probs,
                                                   am_probs, denom, termination_symbol, rnnt_type,
                                                   seq_scale))
    return capi.logprobs_simple_backward(px_grad, py_grad, symbols, boundary, saved,
                                         termination_symbol, rnnt_type, seq_scale)


def smoothed_supported(lm, am):
    """Whether the smoothed builder's kernels take these tensors (their row counts have to fit the
    kernels' 32-bit indexing)."""
    if _ext is not None:
        return _ext.smoothed_supported(am.shape[0], lm.shape[1] - 1, am.shape[1], am.shape[2], capi.dtype_code(am))
    return capi.smoothed_supported(lm, am)


def logprobs_smoothed_forward(lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale, rnnt_type,
                              boundary):
    """(px, py, saved) of get_rnnt_logprobs_smoothed; ``saved`` goes to logprobs_smoothed_backward."""
    _require_device(am)
    if _ext is not None:
        out = _ext.logprobs_smoothed_forward(lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale,
                                             rnnt_type, boundary)
        return out[0], out[1], tuple(out[2:])
    return capi.logprobs_smoothed_forward(lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale,
                                          rnnt_type, boundary)


def logprobs_smoothed_backward(px_grad, py_grad, symbols, boundary, saved, termination_symbol, lm_only_scale,
                               am_only_scale, rnnt_type, seq_scale=None):
    _require_device(px_grad)
    if _ext is not None:
        return tuple(_ext.logprobs_smoothed_backward(px_grad, py_grad, symbols, boundary, *saved,
                                                     termination_symbol, lm_only_scale, am_only_scale, rnnt_type,
                                                     seq_scale))
    return capi.logprobs_smoothed_backward(px_grad, py_grad, symbols, boundary, saved, termination_symbol,
                                           lm_only_scale, am_only_scale, rnnt_type, seq_scale)


def logprobs_joint_forward(logits, symbols, termination_symbol, rnnt_type, boundary):
    _require_device(logits)
    if _ext is not None:
        return tuple(_ext.logprobs_joint_forward(logits, symbols, termination_symbol, rnnt_type,
                                                 boundary))
    return capi.logprobs_joint_forward(logits, symbols, termination_symbol, rnnt_type, boundary)


def logprobs_joint_backward(logits, norm, px_grad, py_grad, symbols, boundary, termination_symbol,
                            rnnt_type, seq_scale=None):
    if _ext is not None:
        return _ext.logprobs_joint_backward(logits, norm, px_grad, py_grad, symbols, boundary,
                                            termination_symbol, rnnt_type, seq_scale)
    return capi.logprobs_joint_backward(logits, norm, px_grad, py_grad, symbols, boundary,
                                        termination_symbol, rnnt_type, seq_scale)


def logprobs_pruned_forward(logits, symbols, ranges, termination_symbol, boundary, rnnt_type,
                            hat=False):
    _require_device(logits)
    if _ext is not None:
        return tuple(_ext.logprobs_pruned_forward(logits, symbols, ranges, termination_symbol,
                                                  boundary, rnnt_type, hat))
    return capi.logprobs_pruned_forward(logits, symbols, ranges, termination_symbol, boundary,
                                        rnnt_type, hat)


def logprobs_pruned_backward(logits, norm, px_grad, py_grad, symbols, ranges, boundary,
                             termination_symbol, rnnt_type, hat=False, seq_scale=None):
    if _ext is not None:
        return _ext.logprobs_pruned_backward(logits, norm, px_grad, py_grad, symbols, ranges,
                                             boundary, termination_symbol, rnnt_type, hat, seq_scale)
    return capi.logprobs_pruned_backward(logits, norm, px_grad, py_grad, symbols, ranges, boundary,
                                         termination_symbol, rnnt_type, hat, seq_scale)


def joiner_pruned_forward(am, lm, ranges, weight, bias, symbols, termination_symbol, boundary,
                          rnnt_type, precision, hat=False):
    _require_device(am)
    return capi.joiner_pruned_forward(am, lm, ranges, weight, bias, symbols, termination_symbol,
                                      boundary, rnnt_type, precision, hat)


def joiner_pruned_backward(am, lm, ranges, weight, bias, symbols, termination_symbol, boundary,
                           rnnt_type, norm, px_grad, py_grad, seq_scale, precision, hat=False):
    return capi.joiner_pruned_backward(am, lm, ranges, weight, bias, symbols, termination_symbol,
                                       boundary, rnnt_type, norm, px_grad, py_grad, seq_scale, precision, hat)


def prune_ranges(px_grad, py_grad, boundary, s_range, deprecated=False):
    _require_device(px_grad)
    if _ext is not None:
        return _ext.prune_ranges(px_grad, py_grad, boundary, s_range, deprecated)
    return capi.prune_ranges(px_grad, py_grad, boundary, s_range, deprecated)


def prune_gather(lm, ranges):
    _require_device(lm)
    if _ext is not None:
        return _ext.prune_gather(lm, ranges)
    return capi.prune_gather(lm, ranges)


def prune_gather_backward(grad, ranges, S1):
    if _ext is not None:
        return _ext.prune_gather_backward(grad, ranges, S1)
    return capi.prune_gather_backward(grad, ranges, S1)


def pruned_ranges_to_lattice(ranges, frames, symbols, logits):
    """The parts of the lattice: (state_splits, arc_splits, arcs [N][4] int32, arc_map [N])."""
    _require_device(ranges)
    if _ext is not None:
        return tuple(_ext.pruned_ranges_to_lattice(ranges, frames, symbols, logits))
    if ranges.dtype != torch.int32 or frames.dtype != torch.int32 or symbols.dtype != torch.int64:
        raise RuntimeError("ranges and frames must be int32, symbols int64")
    return capi.pruned_ranges_to_lattice(ranges.contiguous(), frames.contiguous(),
                                         symbols.contiguous(), logits)
