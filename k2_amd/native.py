"""The native entry points the Python layer calls, named after the reference's ``_k2`` functions.

Backed by the pybind11 host module ``_k2_amd`` (C++ host code over the C-ABI of libk2amd.so)
when it has been built, else by the ctypes binding of the same C-ABI.  Either way the work runs
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


def mutual_information_forward(px: torch.Tensor, py: torch.Tensor,
                               boundary: Optional[torch.Tensor], p: torch.Tensor) -> torch.Tensor:
    """_k2.mutual_information_forward (k2/python/csrc/torch/mutual_information.cu:26-44)."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_forward(px, py, boundary, p)
    return capi.mi_forward(px.contiguous(), py.contiguous(),
                           None if boundary is None else boundary.contiguous(), p)


def mutual_information_backward(px: torch.Tensor, py: torch.Tensor,
                                boundary: Optional[torch.Tensor], p: torch.Tensor,
                                ans_grad: torch.Tensor) -> List[torch.Tensor]:
    """_k2.mutual_information_backward (k2/python/csrc/torch/mutual_information.cu:46-67);
    overwrites ``ans_grad`` like the reference's device path."""
    _require_device(px)
    if _ext is not None:
        return _ext.mutual_information_backward(px, py, boundary, p, ans_grad)
    gx, gy = capi.mi_backward(px.contiguous(), py.contiguous(),
                              None if boundary is None else boundary.contiguous(), p, ans_grad,
                              overwrite_ans_grad=True)
    return [gx, gy]
