"""ctypes binding of libk2amd.so's C-ABI (include/k2_amd.h), taking torch tensors.

This is the thinnest possible host: it checks nothing beyond device/dtype/contiguity, passes
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
    "k2amd_mi_forward": ([_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp, _sz, _vp], _ci),
    "k2amd_mi_backward": ([_vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci,
                           _vp, _sz, _vp], _ci),
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


def ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "k2_amd C-ABI takes contiguous device tensors"
    return t.data_ptr()


def stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


def mi_workspace(B, S, T, modified, dtype, device):
    n = lib().k2amd_mi_workspace_bytes(B, S, T, int(modified), dtype)
    return torch.empty(n, dtype=torch.uint8, device=device) if n else None


def mi_forward(px, py, boundary, p):
    """C-ABI twin of _k2.mutual_information_forward: fills ``p``, returns ans [B]."""
    B, S, T1 = px.shape
    T = py.shape[2]
    modified = int(T1 == T)
    ans = torch.empty(B, dtype=px.dtype, device=px.device)
    dt = dtype_code(px)
    ws = mi_workspace(B, S, T, modified, dt, px.device)
    with torch.cuda.device(px.device):
        check(lib().k2amd_mi_forward(ptr(px), ptr(py), ptr(boundary), ptr(p), ptr(ans), B, S, T,
                                     modified, dt, ptr(ws), 0 if ws is None else ws.numel(),
                                     stream_ptr(px.device)))
    return ans


def mi_backward(px, py, boundary, p, ans_grad, overwrite_ans_grad=True):
    """C-ABI twin of _k2.mutual_information_backward: returns (px_grad, py_grad)."""
    B, S, T1 = px.shape
    T = py.shape[2]
    modified = int(T1 == T)
    px_grad = torch.empty_like(px)
    py_grad = torch.empty_like(py)
    dt = dtype_code(px)
    ws = mi_workspace(B, S, T, modified, dt, px.device)
    with torch.cuda.device(px.device):
        check(lib().k2amd_mi_backward(ptr(px), ptr(py), ptr(boundary), ptr(p), ptr(ans_grad),
                                      ptr(px_grad), ptr(py_grad), B, S, T, modified, dt,
                                      int(overwrite_ans_grad), ptr(ws),
                                      0 if ws is None else ws.numel(), stream_ptr(px.device)))
    return px_grad, py_grad
