"""Host-side checks of the Python layer that need no GPU: the shared host copy of a boundary
tensor and the integer arithmetic of the s_range adjustment."""
import gc
import importlib

import pytest
import torch

kmi = importlib.import_module("k2_amd.mutual_information")
krl = importlib.import_module("k2_amd.rnnt_loss")  # the package attribute of that name is the function


def test_boundary_rows_are_read_once_per_tensor_version():
    bd = torch.tensor([[0, 0, 3, 7], [1, 2, 4, 9]], dtype=torch.int64)
    rows = kmi.boundary_rows(bd)
    assert rows == ((0, 0, 3, 7), (1, 2, 4, 9))
    assert kmi.boundary_rows(bd) is rows                    # reused, not read again
    bd[0, 2] = 5                                            # an in-place write bumps the version
    assert kmi.boundary_rows(bd) == ((0, 0, 5, 7), (1, 2, 4, 9))
    other = bd.clone()                                      # another tensor is always read
    assert kmi.boundary_rows(other) == kmi.boundary_rows(bd)
    assert kmi.boundary_rows(other) is not kmi.boundary_rows(bd)
    key = id(other)
    assert key in kmi._boundary_copies
    del other
    gc.collect()
    assert key not in kmi._boundary_copies                  # the copy goes with its tensor


def test_range_asserts_follow_the_reference():
    """k2/python/k2/mutual_information.py:284-289 and k2/python/k2/rnnt_loss.py:46-62."""
    bd = torch.tensor([[0, 0, 3, 7]], dtype=torch.int64)
    kmi._check_boundary(bd, 3, 7)
    with pytest.raises(AssertionError):
        kmi._check_boundary(bd, 2, 7)
    with pytest.raises(AssertionError):
        kmi._check_boundary(bd, 3, 6)
    with pytest.raises(AssertionError):
        kmi._check_boundary(torch.tensor([[2, 0, 1, 7]]), 3, 7)
    krl._validate_st_lengths(3, 7, False, bd)
    short = torch.tensor([[0, 0, 3, 7], [0, 0, 5, 4]], dtype=torch.int64)
    krl._validate_st_lengths(5, 7, True, short)             # a regular lattice may have T < S
    with pytest.raises(AssertionError, match="Modified transducer requires T >= S"):
        krl._validate_st_lengths(5, 7, False, short)
    with pytest.raises(AssertionError, match="Modified transducer requires T >= S"):
        krl._validate_st_lengths(5, 4, False, None)


def test_trunc_div_is_torch_trunc_division():
    a = torch.arange(-7, 30).repeat_interleave(9)
    b = torch.arange(1, 10).repeat(37)
    want = torch.div(a, b, rounding_mode="trunc").tolist()
    got = [krl._trunc_div(x, y) for x, y in zip(a.tolist(), b.tolist())]
    assert got == want
