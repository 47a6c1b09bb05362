"""ctypes binding of libk2amd.so's C-ABI (include/k2_amd.h), taking torch tensors.

A thin host: before a pointer goes down it checks that every tensor has the dtype, device and
exact shape the kernels index with (RuntimeError otherwise, nothing launched), then passes
``tensor.data_ptr()`` and torch's current HIP stream, and raises RuntimeError on a non-zero
status.  The parity tests call the kernels through here.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libk2amd.so")
_lib = None

F32, F64 = 0, 1
REGULAR, MODIFIED, CONSTRAINED = 0, 1, 2
RNNT_TYPES = {"regular": REGULAR, "modified": MODIFIED, "constrained": CONSTRAINED}

_vp = ctypes.c_void_p
_ci = ctypes.c_int
_sz = ctypes.c_size_t

_SIGNATURES = {
    "k2amd_version": ([], _ci),
    "k2amd_status_string": ([_ci], ctypes.c_char_p),
    "k2amd_mi_workspace_bytes": ([_ci, _ci, _ci, _ci, _ci], _sz),
    "k2amd_mi_workspace_init": ([_vp, _sz, _vp], _ci),
    "k2amd_mi_workspace_status": ([_vp, _vp], _ci),
    "k2amd_mi_workspace_status_async": ([_vp, _vp, _vp], _ci),
    "k2amd_mi_noalloc_status": ([_vp], _ci),
    "k2amd_mi_forward": ([_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp], _ci),
    "k2amd_mi_forward_noalloc": ([_vp] * 5 + [_ci] * 5 + [_vp], _ci),
    "k2amd_mi_backward": ([_vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci,
                           _vp, _sz, _vp], _ci),
    "k2amd_mi_keeps_log_deriv": ([_ci] * 6, _ci),
    "k2amd_mi_forward_keep": ([_vp] * 6 + [_ci] * 5 + [_vp, _sz, _vp], _ci),
    "k2amd_mi_backward_kept": ([_vp] * 8 + [_ci] * 6 + [_vp, _sz, _vp], _ci),
    "k2amd_mi_forward_backward_supported": ([_ci] * 6, _ci),
    "k2amd_mi_forward_backward_advised": ([_ci] * 6, _ci),
    "k2amd_mi_forward_backward_scratch_bytes": ([_ci] * 5, _sz),
    "k2amd_mi_forward_backward": ([_vp] * 5 + [_sz] + [_vp] * 3 + [_ci] * 6 + [_vp, _sz, _vp], _ci),
    "k2amd_mi_joint_products_scratch_elements": ([_ci] * 2, ctypes.c_size_t),
    "k2amd_mi_joint_products": ([_vp, _vp, _ci, _vp, _vp, _vp, _vp, _ci, ctypes.c_longlong, ctypes.c_longlong,
                                 _ci, _vp], _ci),
    "k2amd_rnnt_logprobs_simple_forward": ([_vp] * 11 + [_ci] * 7 + [_vp], _ci),
    "k2amd_rnnt_logprobs_simple_backward": ([_vp] * 11 + [ctypes.c_size_t] + [_ci] * 7 + [_vp], _ci),
    "k2amd_rnnt_logprobs_simple_backward_scratch_elements": ([_ci] * 3, ctypes.c_size_t),
    "k2amd_rnnt_smoothed_scratch_elements": ([_ci] * 4, ctypes.c_size_t),
    "k2amd_rnnt_smoothed_supported": ([_ci] * 5, _ci),
    "k2amd_rnnt_smoothed_forward": ([_vp] * 16 + [ctypes.c_size_t, ctypes.c_double, ctypes.c_double] + [_ci] * 7
                                    + [_vp], _ci),
    "k2amd_rnnt_smoothed_backward": ([_vp] * 15 + [ctypes.c_size_t, ctypes.c_double, ctypes.c_double] + [_ci] * 7
                                     + [_vp], _ci),
    "k2amd_rnnt_logprobs_joint_forward": ([_vp] * 6 + [_ci] * 7 + [_vp], _ci),
    "k2amd_rnnt_logprobs_joint_backward": ([_vp] * 8 + [_ci] * 7 + [_vp], _ci),
    "k2amd_rnnt_logprobs_pruned_forward": ([_vp] * 7 + [_ci] * 8 + [_vp], _ci),
    "k2amd_rnnt_logprobs_pruned_backward": ([_vp] * 9 + [_ci] * 8 + [_vp], _ci),
    "k2amd_rnnt_hat_logprobs_pruned_forward": ([_vp] * 7 + [_ci] * 7 + [_vp], _ci),
    "k2amd_rnnt_hat_logprobs_pruned_backward": ([_vp] * 9 + [_ci] * 7 + [_vp], _ci),
    "k2amd_rnnt_joiner_pruned_workspace_bytes": ([_ci] * 7, _sz),
    "k2amd_rnnt_joiner_pruned_forward_workspace_bytes": ([_ci] * 7, _sz),
    "k2amd_rnnt_joiner_pruned_forward": ([_vp] * 10 + [_ci] * 9 + [_vp, _sz, _vp], _ci),
    "k2amd_rnnt_joiner_pruned_backward": ([_vp] * 15 + [_ci] * 9 + [_vp, _sz, _vp], _ci),
    "k2amd_rnnt_joiner_hat_pruned_forward": ([_vp] * 10 + [_ci] * 8 + [_vp, _sz, _vp], _ci),
    "k2amd_rnnt_joiner_hat_pruned_backward": ([_vp] * 15 + [_ci] * 8 + [_vp, _sz, _vp], _ci),
    "k2amd_rnnt_prune_ranges": ([_vp] * 4 + [_ci] * 6 + [_vp], _ci),
    "k2amd_rnnt_prune_ranges_deprecated": ([_vp] * 4 + [_ci] * 6 + [_vp], _ci),
    "k2amd_rnnt_prune_gather": ([_vp] * 3 + [_ci] * 6 + [_vp], _ci),
    "k2amd_rnnt_prune_gather_backward": ([_vp] * 3 + [_ci] * 6 + [_vp], _ci),
    "k2amd_lattice_count": ([_vp] * 6 + [_ci] * 3 + [_vp], _ci),
    "k2amd_lattice_fill": ([_vp] * 11 + [_ci] * 6 + [_vp], _ci),
}


def lib():
    """Loads libk2amd.so; fails loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python -m k2_amd.build` "
                "(there is no CPU fallback)")
        _lib = ctypes.CDLL(_LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
    return _lib


def exported_symbols():
    return list(_SIGNATURES)


def check(status):
    if status != 0:
        raise RuntimeError("k2_amd: " + lib().k2amd_status_string(status).decode())


def dtype_code(t):
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.float64:
        return F64
    raise RuntimeError(f"k2_amd: unsupported dtype {t.dtype} (float32 / float64 only)")


def _on_device(t):
    """The one place that decides whether a tensor's memory is the GPU's."""
    return t.is_cuda


def ptr(t):
    if t is None:
        return None
    assert _on_device(t) and t.is_contiguous(), "k2_amd C-ABI takes contiguous device tensors"
    return t.data_ptr()


def expect(t, name, dtype, device, shape):
    """Raises RuntimeError unless ``t`` is a contiguous tensor of exactly this dtype, device and
    shape: the kernels index with the sizes taken from ONE tensor of a call, so a disagreeing
    tensor would be read out of bounds or at the wrong element size."""
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"k2_amd: {name} must be a tensor")
    if not _on_device(t):
        raise RuntimeError(f"k2_amd runs on MI355X only: {name} is on {t.device} (there is no CPU path)")
    if t.dtype != dtype or t.device != device or tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"k2_amd: {name} must be {dtype} {list(shape)} on {device}, "
                           f"got {t.dtype} {list(t.shape)} on {t.device}")
    if not t.is_contiguous():
        raise RuntimeError(f"k2_amd: {name} must be contiguous")


def expect_optional(t, name, dtype, device, shape):
    if t is not None:
        expect(t, name, dtype, device, shape)


def _float_dtype(t, name):
    if not isinstance(t, torch.Tensor) or t.dtype not in (torch.float32, torch.float64):
        raise RuntimeError(f"k2_amd: {name} must be a float32 or float64 tensor")
    if not _on_device(t):
        raise RuntimeError(f"k2_amd runs on MI355X only: {name} is on {t.device} (there is no CPU path)")
    return t.dtype, t.device


def _dims(t, name, n):
    if t.dim() != n:
        raise RuntimeError(f"k2_amd: {name} must have {n} dimensions, got {t.dim()}")
    return tuple(t.shape)


def _mi_shapes(px, py, boundary, lattices=()):
    """(B, S, T, modified) after the checks of k2/python/csrc/torch/mutual_information_cpu.cu:53-77;
    ``lattices``: (tensor or None, name) pairs that must have p's shape."""
    dt, dev = _float_dtype(px, "px")
    B, S, T1 = _dims(px, "px", 3)
    if py.dim() != 3:
        raise RuntimeError("k2_amd: py must have 3 dimensions")
    T = py.shape[2]
    if T1 not in (T, T + 1):
        raise RuntimeError("k2_amd: px.size(2) must be T or T+1")
    expect(px, "px", dt, dev, (B, S, T1))
    expect(py, "py", dt, dev, (B, S + 1, T))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    for t, name in lattices:
        expect_optional(t, name, dt, dev, (B, S + 1, T + 1))
    return B, S, T, int(T1 == T)


def stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


_workspaces = {}


def mi_workspace(B, S, T, modified, dtype, device):
    """The scratch buffer of the pipelined fp32 kernels: one per (device, stream), grown on
    demand and initialised once (the kernels leave it ready for the next call)."""
    n = lib().k2amd_mi_workspace_bytes(B, S, T, int(modified), dtype)
    if not n:
        return None
    stream = torch.cuda.current_stream(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < n:
        ws = torch.empty(max(n, 1 << 20), dtype=torch.uint8, device=device)
        with torch.cuda.device(device):
            check(lib().k2amd_mi_workspace_init(ws.data_ptr(), ws.numel(), stream.cuda_stream))
        _workspaces[key] = ws
    return ws


def mi_workspace_is_clean(device):
    """True when every edge word of the cached workspace holds the sentinel again and the ticket
    counters are back to zero, i.e. the last kernel left the buffer ready for the next call."""
    stream = torch.cuda.current_stream(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is None:
        return True
    torch.cuda.synchronize(device)
    words = ws[: ws.numel() // 4 * 4].view(torch.int32)
    header_ok = bool((words[:3] == 0).all())
    sentinel = 0x7FC5A5A5
    return header_ok and bool((words[64:] == sentinel).all())


def mi_workspace_status(device):
    """Synchronises and raises if a pipelined kernel on this device's current stream timed out."""
    stream = torch.cuda.current_stream(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream.cuda_stream)
    ws = _workspaces.get(key)
    if ws is not None:
        with torch.cuda.device(device):
            check(lib().k2amd_mi_workspace_status(ws.data_ptr(), stream.cuda_stream))


def mi_keeps_log_deriv(px, py):
    """True if mi_forward / mi_backward on these tensors use a ``log_deriv`` tensor when given one
    (the pipelined fp32 kernels do; the exact kernels leave it untouched)."""
    B, S, T1 = px.shape
    T = py.shape[2]
    dt = dtype_code(px)
    has_ws = lib().k2amd_mi_workspace_bytes(B, S, T, int(T1 == T), dt) > 0
    return bool(lib().k2amd_mi_keeps_log_deriv(B, S, T, int(T1 == T), dt, int(has_ws)))


def mi_forward(px, py, boundary, p, log_deriv=None):
    """C-ABI twin of _k2.mutual_information_forward: fills ``p``, returns ans [B].  ``log_deriv``
    (optional, shaped like ``p``) receives what lets mi_backward skip its reads of p and px; where
    mi_keeps_log_deriv(px, py) holds, ``p`` may then be None and is not computed."""
    B, S, T, modified = _mi_shapes(px, py, boundary, ((p, "p"), (log_deriv, "log_deriv")))
    if p is None and log_deriv is None:
        raise RuntimeError("k2_amd: p may only be None where log_deriv is given")
    ans = torch.empty(B, dtype=px.dtype, device=px.device)
    dt = dtype_code(px)
    ws = mi_workspace(B, S, T, modified, dt, px.device)
    with torch.cuda.device(px.device):
        check(lib().k2amd_mi_forward_keep(ptr(px), ptr(py), ptr(boundary), ptr(p), ptr(ans),
                                          ptr(log_deriv), B, S, T, modified, dt, ptr(ws),
                                          0 if ws is None else ws.numel(), stream_ptr(px.device)))
    return ans


def mi_forward_noalloc(px, py, boundary, p, ans):
    """k2amd_mi_forward_noalloc: like mi_forward, but the library brings its own static scratch and
    the caller brings ``ans`` [B] as well, so that nothing is allocated by the call."""
    B, S, T, modified = _mi_shapes(px, py, boundary, ((p, "p"),))
    expect(p, "p", px.dtype, px.device, (B, S + 1, T + 1))
    expect(ans, "ans", px.dtype, px.device, (B,))
    with torch.cuda.device(px.device):
        check(lib().k2amd_mi_forward_noalloc(ptr(px), ptr(py), ptr(boundary), ptr(p), ptr(ans), B, S, T,
                                             modified, dtype_code(px), stream_ptr(px.device)))
    return ans


def mi_backward(px, py, boundary, p, ans_grad, overwrite_ans_grad=True, log_deriv=None):
    """C-ABI twin of _k2.mutual_information_backward: returns (px_grad, py_grad).  ``log_deriv``:
    the tensor the matching mi_forward call filled, or None."""
    B, S, T, modified = _mi_shapes(px, py, boundary, ((p, "p"), (log_deriv, "log_deriv")))
    if p is None and log_deriv is None:
        raise RuntimeError("k2_amd: p may only be None where log_deriv is given")
    expect(ans_grad, "ans_grad", px.dtype, px.device, (B,))
    px_grad = torch.empty_like(px)
    py_grad = torch.empty_like(py)
    dt = dtype_code(px)
    ws = mi_workspace(B, S, T, modified, dt, px.device)
    with torch.cuda.device(px.device):
        check(lib().k2amd_mi_backward_kept(ptr(px), ptr(py), ptr(boundary), ptr(p), ptr(log_deriv),
                                           ptr(ans_grad), ptr(px_grad), ptr(py_grad), B, S, T, modified, dt,
                                      int(overwrite_ans_grad), ptr(ws),
                                      0 if ws is None else ws.numel(), stream_ptr(px.device)))
    return px_grad, py_grad


def mi_forward_backward_supported(px, py):
    """True if mi_forward_backward serves these tensors (fp32, the pipelined kernels' shapes)."""
    B, S, T1 = px.shape
    T = py.shape[2]
    dt = dtype_code(px)
    has_ws = lib().k2amd_mi_workspace_bytes(B, S, T, int(T1 == T), dt) > 0
    with torch.cuda.device(px.device):
        return bool(lib().k2amd_mi_forward_backward_supported(B, S, T, int(T1 == T), dt, int(has_ws)))


def mi_forward_backward_advised(px, py):
    """True if mi_forward_backward serves these tensors and is the faster way on their device (the
    device has a compute unit for every half-sweep of the launch at once)."""
    B, S, T1 = px.shape
    T = py.shape[2]
    dt = dtype_code(px)
    has_ws = lib().k2amd_mi_workspace_bytes(B, S, T, int(T1 == T), dt) > 0
    with torch.cuda.device(px.device):
        return bool(lib().k2amd_mi_forward_backward_advised(B, S, T, int(T1 == T), dt, int(has_ws)))


def mi_forward_backward(px, py, boundary, ans_grad, overwrite_ans_grad=True):
    """Forward and backward recursion in one launch: returns (ans, px_grad, py_grad)."""
    B, S, T, modified = _mi_shapes(px, py, boundary)
    expect_optional(ans_grad, "ans_grad", px.dtype, px.device, (B,))
    ans = torch.empty(B, dtype=px.dtype, device=px.device)
    px_grad = torch.empty_like(px)
    py_grad = torch.empty_like(py)
    dt = dtype_code(px)
    nbytes = lib().k2amd_mi_forward_backward_scratch_bytes(B, S, T, modified, dt)
    scratch = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=px.device)
    ws = mi_workspace(B, S, T, modified, dt, px.device)
    with torch.cuda.device(px.device):
        check(lib().k2amd_mi_forward_backward(ptr(px), ptr(py), ptr(boundary), ptr(ans), ptr(scratch),
                                              scratch.numel(), ptr(ans_grad), ptr(px_grad), ptr(py_grad),
                                              B, S, T, modified, dt, int(overwrite_ans_grad), ptr(ws),
                                              0 if ws is None else ws.numel(), stream_ptr(px.device)))
    return ans, px_grad, py_grad


JOINT_MAX_INPUTS = 8


def mi_joint_products(px, py, px_grad, py_grad):
    """prods [N][B] of joint_mutual_information_recursion: px, py sequences of N tensors shaped
    like px_grad [B][S][T1] and py_grad [B][S+1][T] (same dtype and device, contiguous)."""
    N = len(px)
    if N < 1 or len(py) != N or N > JOINT_MAX_INPUTS:
        raise RuntimeError(f"k2_amd: 1 to {JOINT_MAX_INPUTS} pairs of inputs, got {N} and {len(py)}")
    dt, dev = _float_dtype(px_grad, "px_grad")
    B = px_grad.shape[0]
    expect(px_grad, "px_grad", dt, dev, tuple(px_grad.shape))
    expect(py_grad, "py_grad", dt, dev, (B,) + tuple(py_grad.shape[1:]))
    for n in range(N):
        expect(px[n], f"px[{n}]", dt, dev, tuple(px_grad.shape))
        expect(py[n], f"py[{n}]", dt, dev, tuple(py_grad.shape))
    kx = px_grad.numel() // B if B else 0
    ky = py_grad.numel() // B if B else 0
    prods = torch.empty(N, B, dtype=dt, device=dev)
    partial = torch.empty(lib().k2amd_mi_joint_products_scratch_elements(N, B), dtype=dt, device=dev)
    xs = (ctypes.c_void_p * N)(*[ptr(t) for t in px])
    ys = (ctypes.c_void_p * N)(*[ptr(t) for t in py])
    with torch.cuda.device(dev):
        check(lib().k2amd_mi_joint_products(ctypes.addressof(xs), ctypes.addressof(ys), N, ptr(px_grad),
                                            ptr(py_grad), ptr(prods), ptr(partial), B, kx, ky,
                                            dtype_code(px_grad), stream_ptr(dev)))
    return prods


def _t1(T, rnnt_type):
    return T + 1 if rnnt_type == REGULAR else T


def _rnnt_type(code):
    if code not in (REGULAR, MODIFIED, CONSTRAINED):
        raise RuntimeError(f"k2_amd: unknown rnnt_type code {code}")


def _symbol(termination_symbol, C):
    if not 0 <= int(termination_symbol) < C:
        raise RuntimeError(f"k2_amd: termination_symbol {termination_symbol} outside [0, {C})")


def _expect_lattice_grads(px_grad, py_grad, seq_scale, dt, dev, B, S, T, rnnt_type):
    expect(px_grad, "px_grad", dt, dev, (B, S, _t1(T, rnnt_type)))
    expect(py_grad, "py_grad", dt, dev, (B, S + 1, T))
    expect_optional(seq_scale, "seq_scale", dt, dev, (B,))


def logprobs_simple_forward(lm, am, symbols, termination_symbol, rnnt_type, boundary):
    """C-ABI get_rnnt_logprobs: returns (px, py, saved) with ``saved`` the buffers the backward
    re-uses (lm_probs, am_probs, denom)."""
    dt, dev = _float_dtype(am, "am")
    B, T, C = _dims(am, "am", 3)
    S = _dims(lm, "lm", 3)[1] - 1
    _rnnt_type(rnnt_type)
    expect(am, "am", dt, dev, (B, T, C))
    expect(lm, "lm", dt, dev, (B, S + 1, C))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _symbol(termination_symbol, C)
    px = torch.empty(B, S, _t1(T, rnnt_type), dtype=dt, device=dev)
    py = torch.empty(B, S + 1, T, dtype=dt, device=dev)
    lm_probs = torch.empty_like(lm)
    am_probs = torch.empty_like(am)
    lm_max = torch.empty(B, S + 1, dtype=dt, device=dev)
    am_max = torch.empty(B, T, dtype=dt, device=dev)
    denom = torch.empty(B, S + 1, T, dtype=dt, device=dev)
    with torch.cuda.device(dev):
        check(lib().k2amd_rnnt_logprobs_simple_forward(
            ptr(lm), ptr(am), ptr(symbols), ptr(boundary), ptr(px), ptr(py), ptr(lm_probs),
            ptr(am_probs), ptr(lm_max), ptr(am_max), ptr(denom), B, S, T, C, termination_symbol,
            rnnt_type, dtype_code(am), stream_ptr(dev)))
    return px, py, (lm_probs, am_probs, denom)


def logprobs_simple_backward(px_grad, py_grad, symbols, boundary, saved, termination_symbol,
                             rnnt_type, seq_scale=None):
    """``seq_scale`` [B] or None: px_grad[b], py_grad[b] count as multiplied by seq_scale[b] (the
    same for the two functions below)."""
    lm_probs, am_probs, denom = saved
    dt, dev = _float_dtype(am_probs, "am_probs")
    B, T, C = _dims(am_probs, "am_probs", 3)
    S = _dims(lm_probs, "lm_probs", 3)[1] - 1
    _rnnt_type(rnnt_type)
    expect(am_probs, "am_probs", dt, dev, (B, T, C))
    expect(lm_probs, "lm_probs", dt, dev, (B, S + 1, C))
    expect(denom, "denom", dt, dev, (B, S + 1, T))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _expect_lattice_grads(px_grad, py_grad, seq_scale, dt, dev, B, S, T, rnnt_type)
    _symbol(termination_symbol, C)
    lm_grad = torch.empty_like(lm_probs)
    am_grad = torch.empty_like(am_probs)
    # the products' operand [B][S+1][T], then the gradients' sums along s and along t
    q = torch.empty(lib().k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T), dtype=dt, device=dev)
    dev = am_probs.device
    with torch.cuda.device(dev):
        check(lib().k2amd_rnnt_logprobs_simple_backward(
            ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(symbols), ptr(boundary), ptr(lm_probs),
            ptr(am_probs), ptr(denom), ptr(lm_grad), ptr(am_grad), ptr(q), q.numel(), B, S, T, C, termination_symbol,
            rnnt_type, dtype_code(am_probs), stream_ptr(dev)))
    return lm_grad, am_grad


def smoothed_supported(lm, am):
    """Whether the smoothed builder's kernels take these tensors (their row counts have to fit the
    kernels' 32-bit indexing)."""
    B, T, C = am.shape
    return bool(lib().k2amd_rnnt_smoothed_supported(B, lm.shape[1] - 1, T, C, dtype_code(am)))


def logprobs_smoothed_forward(lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale, rnnt_type,
                              boundary):
    """C-ABI get_rnnt_logprobs_smoothed: the simple builder on the lattice without a boundary, then
    the marginal terms and the mix.  Returns (px, py, saved), ``saved`` = (lm_probs, am_probs, denom,
    lm_max, am_max, lm_norm, am_norm, unigram) for the backward."""
    dt, dev = _float_dtype(am, "am")
    B, T, C = _dims(am, "am", 3)
    S = _dims(lm, "lm", 3)[1] - 1
    _rnnt_type(rnnt_type)
    expect(am, "am", dt, dev, (B, T, C))
    expect(lm, "lm", dt, dev, (B, S + 1, C))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _symbol(termination_symbol, C)
    joint_type = REGULAR if rnnt_type == REGULAR else MODIFIED
    px_joint = torch.empty(B, S, _t1(T, rnnt_type), dtype=dt, device=dev)
    py_joint = torch.empty(B, S + 1, T, dtype=dt, device=dev)
    px, py = torch.empty_like(px_joint), torch.empty_like(py_joint)
    lm_probs, am_probs = torch.empty_like(lm), torch.empty_like(am)
    lm_max, lm_norm = (torch.empty(B, S + 1, dtype=dt, device=dev) for _ in range(2))
    am_max, am_norm = (torch.empty(B, T, dtype=dt, device=dev) for _ in range(2))
    denom = torch.empty(B, S + 1, T, dtype=dt, device=dev)
    unigram = torch.empty(2, C, dtype=dt, device=dev)
    scratch = torch.empty(lib().k2amd_rnnt_smoothed_scratch_elements(B, S, T, C), dtype=dt, device=dev)
    with torch.cuda.device(dev):
        check(lib().k2amd_rnnt_logprobs_simple_forward(
            ptr(lm), ptr(am), ptr(symbols), None, ptr(px_joint), ptr(py_joint), ptr(lm_probs), ptr(am_probs),
            ptr(lm_max), ptr(am_max), ptr(denom), B, S, T, C, termination_symbol, joint_type, dtype_code(am),
            stream_ptr(dev)))
        check(lib().k2amd_rnnt_smoothed_forward(
            ptr(lm), ptr(am), ptr(symbols), ptr(boundary), ptr(lm_probs), ptr(am_probs), ptr(lm_max), ptr(am_max),
            ptr(px_joint), ptr(py_joint), ptr(px), ptr(py), ptr(lm_norm), ptr(am_norm), ptr(unigram), ptr(scratch),
            scratch.numel(), float(lm_only_scale), float(am_only_scale), B, S, T, C, termination_symbol, rnnt_type,
            dtype_code(am), stream_ptr(dev)))
    return px, py, (lm_probs, am_probs, denom, lm_max, am_max, lm_norm, am_norm, unigram)


def logprobs_smoothed_backward(px_grad, py_grad, symbols, boundary, saved, termination_symbol, lm_only_scale,
                               am_only_scale, rnnt_type, seq_scale=None):
    """(lm_grad, am_grad): the simple builder's backward with the gradients scaled by
    1 - lm_only_scale - am_only_scale, then the marginal terms' gradients added."""
    lm_probs, am_probs, denom, lm_max, am_max, lm_norm, am_norm, unigram = saved
    dt, dev = _float_dtype(am_probs, "am_probs")
    B, T, C = _dims(am_probs, "am_probs", 3)
    S = _dims(lm_probs, "lm_probs", 3)[1] - 1
    _rnnt_type(rnnt_type)
    expect(am_probs, "am_probs", dt, dev, (B, T, C))
    expect(lm_probs, "lm_probs", dt, dev, (B, S + 1, C))
    expect(denom, "denom", dt, dev, (B, S + 1, T))
    for t, name, shape in ((lm_max, "lm_max", (B, S + 1)), (lm_norm, "lm_norm", (B, S + 1)), (am_max, "am_max", (B, T)),
                           (am_norm, "am_norm", (B, T)), (unigram, "unigram", (2, C))):
        expect(t, name, dt, dev, shape)
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _expect_lattice_grads(px_grad, py_grad, seq_scale, dt, dev, B, S, T, rnnt_type)
    _symbol(termination_symbol, C)
    joint_scale = 1.0 - float(lm_only_scale) - float(am_only_scale)
    joint_seq_scale = (torch.full((B,), joint_scale, dtype=dt, device=dev) if seq_scale is None
                       else seq_scale * joint_scale)
    lm_grad, am_grad = torch.empty_like(lm_probs), torch.empty_like(am_probs)
    q = torch.empty(lib().k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T), dtype=dt, device=dev)
    scratch = torch.empty(lib().k2amd_rnnt_smoothed_scratch_elements(B, S, T, C), dtype=dt, device=dev)
    with torch.cuda.device(dev):
        check(lib().k2amd_rnnt_logprobs_simple_backward(
            ptr(px_grad), ptr(py_grad), ptr(joint_seq_scale), ptr(symbols), ptr(boundary), ptr(lm_probs),
            ptr(am_probs), ptr(denom), ptr(lm_grad), ptr(am_grad), ptr(q), q.numel(), B, S, T, C, termination_symbol,
            rnnt_type, dtype_code(am_probs), stream_ptr(dev)))
        check(lib().k2amd_rnnt_smoothed_backward(
            ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(symbols), ptr(boundary), ptr(lm_probs), ptr(am_probs),
            ptr(lm_max), ptr(am_max), ptr(lm_norm), ptr(am_norm), ptr(unigram), ptr(lm_grad), ptr(am_grad),
            ptr(scratch), scratch.numel(), float(lm_only_scale), float(am_only_scale), B, S, T, C,
            termination_symbol, rnnt_type, dtype_code(am_probs), stream_ptr(dev)))
    return lm_grad, am_grad


def logprobs_joint_forward(logits, symbols, termination_symbol, rnnt_type, boundary):
    dt, dev = _float_dtype(logits, "logits")
    B, T, S1, C = _dims(logits, "logits", 4)
    S = S1 - 1
    _rnnt_type(rnnt_type)
    expect(logits, "logits", dt, dev, (B, T, S1, C))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _symbol(termination_symbol, C)
    px = torch.empty(B, S, _t1(T, rnnt_type), dtype=dt, device=dev)
    py = torch.empty(B, S + 1, T, dtype=dt, device=dev)
    norm = torch.empty(B, T, S1, dtype=dt, device=dev)
    with torch.cuda.device(dev):
        check(lib().k2amd_rnnt_logprobs_joint_forward(
            ptr(logits), ptr(symbols), ptr(boundary), ptr(px), ptr(py), ptr(norm), B, S, T, C,
            termination_symbol, rnnt_type, dtype_code(logits), stream_ptr(dev)))
    return px, py, norm


def logprobs_joint_backward(logits, norm, px_grad, py_grad, symbols, boundary,
                            termination_symbol, rnnt_type, seq_scale=None):
    dt, dev = _float_dtype(logits, "logits")
    B, T, S1, C = _dims(logits, "logits", 4)
    _rnnt_type(rnnt_type)
    expect(logits, "logits", dt, dev, (B, T, S1, C))
    expect(norm, "normalizers", dt, dev, (B, T, S1))
    expect(symbols, "symbols", torch.int64, dev, (B, S1 - 1))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _expect_lattice_grads(px_grad, py_grad, seq_scale, dt, dev, B, S1 - 1, T, rnnt_type)
    _symbol(termination_symbol, C)
    grad = torch.empty_like(logits)
    with torch.cuda.device(dev):
        check(lib().k2amd_rnnt_logprobs_joint_backward(
            ptr(logits), ptr(norm), ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(symbols),
            ptr(boundary), ptr(grad), B, S1 - 1, T, C, termination_symbol, rnnt_type, dtype_code(logits),
            stream_ptr(dev)))
    return grad


def logprobs_pruned_forward(logits, symbols, ranges, termination_symbol, boundary, rnnt_type,
                            hat=False):
    """``hat`` selects get_hat_logprobs_pruned (blank = column 0, termination_symbol unused)."""
    dt, dev = _float_dtype(logits, "logits")
    B, T, R, C = _dims(logits, "logits", 4)
    S = _dims(symbols, "symbols", 2)[1]
    _rnnt_type(rnnt_type)
    expect(logits, "logits", dt, dev, (B, T, R, C))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect(ranges, "ranges", torch.int64, dev, (B, T, R))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _symbol(0 if hat else termination_symbol, C)
    px = torch.empty(B, S, _t1(T, rnnt_type), dtype=dt, device=dev)
    py = torch.empty(B, S + 1, T, dtype=dt, device=dev)
    norm = torch.empty(B, T, R, dtype=dt, device=dev)
    with torch.cuda.device(dev):
        if hat:
            check(lib().k2amd_rnnt_hat_logprobs_pruned_forward(
                ptr(logits), ptr(symbols), ptr(ranges), ptr(boundary), ptr(px), ptr(py), ptr(norm),
                B, S, T, R, C, rnnt_type, dtype_code(logits), stream_ptr(dev)))
            return px, py, norm
        check(lib().k2amd_rnnt_logprobs_pruned_forward(
            ptr(logits), ptr(symbols), ptr(ranges), ptr(boundary), ptr(px), ptr(py), ptr(norm),
            B, S, T, R, C, termination_symbol, rnnt_type, dtype_code(logits), stream_ptr(dev)))
    return px, py, norm


def logprobs_pruned_backward(logits, norm, px_grad, py_grad, symbols, ranges, boundary,
                             termination_symbol, rnnt_type, hat=False, seq_scale=None):
    dt, dev = _float_dtype(logits, "logits")
    B, T, R, C = _dims(logits, "logits", 4)
    S = _dims(symbols, "symbols", 2)[1]
    _rnnt_type(rnnt_type)
    expect(logits, "logits", dt, dev, (B, T, R, C))
    expect(norm, "normalizers", dt, dev, (B, T, R))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect(ranges, "ranges", torch.int64, dev, (B, T, R))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _expect_lattice_grads(px_grad, py_grad, seq_scale, dt, dev, B, S, T, rnnt_type)
    _symbol(0 if hat else termination_symbol, C)
    grad = torch.empty_like(logits)
    with torch.cuda.device(dev):
        if hat:
            check(lib().k2amd_rnnt_hat_logprobs_pruned_backward(
                ptr(logits), ptr(norm), ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(symbols),
                ptr(ranges), ptr(boundary), ptr(grad), B, S, T, R, C, rnnt_type, dtype_code(logits),
                stream_ptr(dev)))
            return grad
        check(lib().k2amd_rnnt_logprobs_pruned_backward(
            ptr(logits), ptr(norm), ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(symbols),
            ptr(ranges), ptr(boundary), ptr(grad), B, S, T, R, C, termination_symbol, rnnt_type,
            dtype_code(logits), stream_ptr(dev)))
    return grad


JOINER_PRECISIONS = {"fp32": 0, "bf16": 1}


def _joiner_shapes(am, lm, ranges, weight, bias, symbols, boundary, termination_symbol, rnnt_type,
                   precision, forward):
    """Checks every tensor of the fused joiner calls; returns (B, S, T, R, C, D, workspace), the
    workspace of the size the forward (or the backward) call asks for."""
    dev = am.device
    if am.dtype != torch.float32:
        raise RuntimeError(f"k2_amd: the fused joiner takes float32 tensors, am is {am.dtype}")
    if precision not in (0, 1):
        raise RuntimeError(f"k2_amd: unknown joiner precision code {precision}")
    B, T, D = _dims(am, "am", 3)
    S1 = _dims(lm, "lm", 3)[1]
    R = _dims(ranges, "ranges", 3)[2]
    C = _dims(weight, "weight", 2)[0]
    S = S1 - 1
    _rnnt_type(rnnt_type)
    expect(am, "am", torch.float32, dev, (B, T, D))
    expect(lm, "lm", torch.float32, dev, (B, S1, D))
    expect(ranges, "ranges", torch.int64, dev, (B, T, R))
    expect(weight, "weight", torch.float32, dev, (C, D))
    expect_optional(bias, "bias", torch.float32, dev, (C,))
    expect(symbols, "symbols", torch.int64, dev, (B, S))
    expect_optional(boundary, "boundary", torch.int64, dev, (B, 4))
    _symbol(termination_symbol, C)
    size_of = (lib().k2amd_rnnt_joiner_pruned_forward_workspace_bytes if forward
               else lib().k2amd_rnnt_joiner_pruned_workspace_bytes)
    nbytes = size_of(B, S, T, R, C, D, precision)
    if nbytes == 0:
        raise RuntimeError(f"k2_amd: the fused joiner does not serve B={B} S={S} T={T} R={R} C={C} D={D} "
                           "(D must be a multiple of 64 up to 512, R at most 32 and S + 1)")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    return B, S, T, R, C, D, ws


def joiner_pruned_forward(am, lm, ranges, weight, bias, symbols, termination_symbol, boundary,
                          rnnt_type, precision=0, hat=False):
    """tanh(am[b,t] + lm[b,ranges[b,t,k]]) . weight^T + bias and get_rnnt_logprobs_pruned on it in one
    pass: returns (px, py, normalizers [B][T][R]); the logits never exist in memory.  ``hat``:
    get_hat_logprobs_pruned instead (column 0 is the blank; termination_symbol must be 0)."""
    if hat and int(termination_symbol) != 0:
        raise RuntimeError("k2_amd: the hybrid autoregressive transducer's blank is symbol 0")
    B, S, T, R, C, D, ws = _joiner_shapes(am, lm, ranges, weight, bias, symbols, boundary,
                                          termination_symbol, rnnt_type, precision, True)
    dev = am.device
    px = torch.empty(B, S, _t1(T, rnnt_type), dtype=torch.float32, device=dev)
    py = torch.empty(B, S + 1, T, dtype=torch.float32, device=dev)
    norm = torch.empty(B, T, R, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        if hat:
            check(lib().k2amd_rnnt_joiner_hat_pruned_forward(
                ptr(am), ptr(lm), ptr(ranges), ptr(weight), ptr(bias), ptr(symbols), ptr(boundary),
                ptr(px), ptr(py), ptr(norm), B, S, T, R, C, D, rnnt_type, precision,
                ptr(ws), ws.numel(), stream_ptr(dev)))
        else:
            check(lib().k2amd_rnnt_joiner_pruned_forward(
                ptr(am), ptr(lm), ptr(ranges), ptr(weight), ptr(bias), ptr(symbols), ptr(boundary),
                ptr(px), ptr(py), ptr(norm), B, S, T, R, C, D, termination_symbol, rnnt_type, precision,
                ptr(ws), ws.numel(), stream_ptr(dev)))
    return px, py, norm


def joiner_pruned_backward(am, lm, ranges, weight, bias, symbols, termination_symbol, boundary,
                           rnnt_type, norm, px_grad, py_grad, seq_scale=None, precision=0, hat=False):
    """Gradients of sum_b seq_scale[b] * score_b through the fused joiner: returns (am_grad, lm_grad,
    weight_grad, bias_grad or None)."""
    B, S, T, R, C, D, ws = _joiner_shapes(am, lm, ranges, weight, bias, symbols, boundary,
                                          termination_symbol, rnnt_type, precision, False)
    dev = am.device
    expect(norm, "normalizers", torch.float32, dev, (B, T, R))
    _expect_lattice_grads(px_grad, py_grad, seq_scale, torch.float32, dev, B, S, T, rnnt_type)
    am_grad = torch.empty_like(am)
    lm_grad = torch.empty_like(lm)
    weight_grad = torch.empty_like(weight)
    bias_grad = torch.empty_like(bias) if bias is not None else None
    with torch.cuda.device(dev):
        if hat:
            check(lib().k2amd_rnnt_joiner_hat_pruned_backward(
                ptr(am), ptr(lm), ptr(ranges), ptr(weight), ptr(bias), ptr(symbols), ptr(boundary),
                ptr(norm), ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(am_grad), ptr(lm_grad),
                ptr(weight_grad), ptr(bias_grad), B, S, T, R, C, D, rnnt_type,
                precision, ptr(ws), ws.numel(), stream_ptr(dev)))
        else:
            check(lib().k2amd_rnnt_joiner_pruned_backward(
                ptr(am), ptr(lm), ptr(ranges), ptr(weight), ptr(bias), ptr(symbols), ptr(boundary),
                ptr(norm), ptr(px_grad), ptr(py_grad), ptr(seq_scale), ptr(am_grad), ptr(lm_grad),
                ptr(weight_grad), ptr(bias_grad), B, S, T, R, C, D, termination_symbol, rnnt_type,
                precision, ptr(ws), ws.numel(), stream_ptr(dev)))
    return am_grad, lm_grad, weight_grad, bias_grad


def prune_ranges(px_grad, py_grad, boundary, s_range, deprecated=False):
    """``s_range`` is the final value (after the adjustments the Python layer applies);
    ``deprecated``: the rule of get_rnnt_prune_ranges_deprecated instead."""
    dt, dev = _float_dtype(px_grad, "px_grad")
    B, S, T1 = _dims(px_grad, "px_grad", 3)
    T = _dims(py_grad, "py_grad", 3)[2]
    if T1 not in (T, T + 1):
        raise RuntimeError("k2_amd: px_grad.size(2) must be T or T+1")
    expect(px_grad, "px_grad", dt, dev, (B, S, T1))
    expect(py_grad, "py_grad", dt, dev, (B, S + 1, T))
    expect(boundary, "boundary", torch.int64, dev, (B, 4))
    if not 1 <= int(s_range) <= S + 1:
        raise RuntimeError(f"k2_amd: s_range {s_range} outside [1, S + 1 = {S + 1}]")
    ranges = torch.empty(B, T, s_range, dtype=torch.int64, device=px_grad.device)
    with torch.cuda.device(dev):
        entry = lib().k2amd_rnnt_prune_ranges_deprecated if deprecated else lib().k2amd_rnnt_prune_ranges
        check(entry(ptr(px_grad), ptr(py_grad), ptr(boundary), ptr(ranges), B, S, T, int(T1 == T),
                    s_range, dtype_code(px_grad), stream_ptr(dev)))
    return ranges


def prune_gather(lm, ranges):
    dt, dev = _float_dtype(lm, "lm")
    B, S1, D = _dims(lm, "lm", 3)
    _, T, R = _dims(ranges, "ranges", 3)
    expect(lm, "lm", dt, dev, (B, S1, D))
    expect(ranges, "ranges", torch.int64, dev, (B, T, R))
    out = torch.empty(B, T, R, D, dtype=lm.dtype, device=lm.device)
    with torch.cuda.device(lm.device):
        check(lib().k2amd_rnnt_prune_gather(ptr(lm), ptr(ranges), ptr(out), B, S1, T, R, D,
                                            dtype_code(lm), stream_ptr(lm.device)))
    return out


def prune_gather_backward(grad, ranges, S1):
    dt, dev = _float_dtype(grad, "grad")
    B, T, R, D = _dims(grad, "grad", 4)
    expect(grad, "grad", dt, dev, (B, T, R, D))
    expect(ranges, "ranges", torch.int64, dev, (B, T, R))
    if int(S1) < 1:
        raise RuntimeError("k2_amd: S1 must be positive")
    lm_grad = torch.empty(B, S1, D, dtype=grad.dtype, device=grad.device)
    with torch.cuda.device(grad.device):
        check(lib().k2amd_rnnt_prune_gather_backward(ptr(grad), ptr(ranges), ptr(lm_grad), B, S1,
                                                     T, R, D, dtype_code(grad),
                                                     stream_ptr(grad.device)))
    return lm_grad


F16 = 2


def pruned_ranges_to_lattice(ranges, frames, symbols, logits):
    """C-ABI pruned_ranges_to_lattice: returns (state_splits [B+1], arc_splits [states+1],
    arcs int32 [arcs][4] (score bits in column 3), arc_map int32 [arcs])."""
    B, T, R = ranges.shape
    S = symbols.shape[1]
    C = logits.shape[3]
    dev = ranges.device
    i32 = dict(dtype=torch.int32, device=dev)
    arc_local = torch.empty(B, T * R + 1, **i32)
    seq_arcs = torch.empty(max(B, 1), **i32)
    splits = torch.empty(2, B + 1, **i32)  # one buffer: the two totals come to the host in one copy
    state_splits, arc_base = splits[0], splits[1]
    code = {torch.float32: F32, torch.float64: F64, torch.float16: F16}.get(logits.dtype)
    if code is None:
        raise RuntimeError(f"k2_amd: unsupported logits dtype {logits.dtype}")
    with torch.cuda.device(dev):
        check(lib().k2amd_lattice_count(ptr(ranges), ptr(frames), ptr(arc_local), ptr(seq_arcs),
                                        ptr(state_splits), ptr(arc_base), B, T, R, stream_ptr(dev)))
        n_states, n_arcs = splits[:, B].tolist()  # the one host read, as in k2
        arc_splits = torch.empty(n_states + 1, **i32)
        arcs = torch.empty(n_arcs, 4, **i32)
        arc_map = torch.empty(n_arcs, **i32)
        if B == 0:
            arc_splits.zero_()
        strides = (ctypes.c_int64 * 4)(*logits.stride())
        assert _on_device(logits)
        check(lib().k2amd_lattice_fill(ptr(ranges), ptr(frames), ptr(symbols), logits.data_ptr(),
                                       ctypes.addressof(strides), ptr(state_splits), ptr(arc_base),
                                       ptr(arc_local), ptr(arc_splits), ptr(arcs), ptr(arc_map), B, T,
                                       R, S, C, code, stream_ptr(dev)))
    return state_splits, arc_splits, arcs, arc_map
