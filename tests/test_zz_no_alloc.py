"""k2amd_mi_forward_noalloc (the entry point that allocates nothing: its scratch is a static device
array inside the library) against k2amd_mi_forward with a caller's workspace, through the C-ABI:
identical bits for ans and for p, on two calls in a row, the second with a smaller input, so that
what the first call left in the shared array would show."""
import numpy as np
import pytest
import torch

import cases

pytestmark = pytest.mark.gpu


def _both(c, device, check_memory=True):
    from k2_amd import capi
    px, py = (torch.from_numpy(c[k]).to(device) for k in ("px", "py"))
    bd = None if c["boundary"] is None else torch.from_numpy(c["boundary"]).to(device)
    B, S, T = c["B"], c["S"], c["T"]
    p_ref = torch.full((B, S + 1, T + 1), float("nan"), dtype=px.dtype, device=device)
    ans_ref = capi.mi_forward(px, py, bd, p_ref)
    p = torch.full_like(p_ref, float("nan"))
    ans = torch.full((B,), float("nan"), dtype=px.dtype, device=device)
    free_before = torch.cuda.mem_get_info(device)[0]
    capi.mi_forward_noalloc(px, py, bd, p, ans)
    torch.cuda.synchronize(device)
    if check_memory:
        assert torch.cuda.mem_get_info(device)[0] >= free_before    # no device memory was taken
    view = torch.int32 if px.dtype == torch.float32 else torch.int64
    assert torch.equal(ans.view(view), ans_ref.view(view))
    assert torch.equal(p.view(view), p_ref.view(view))              # cells outside the boxes stay NaN in both
    assert torch.isfinite(ans_ref).any()


def test_noalloc_forward_equals_the_workspace_entry_point(device):
    from k2_amd import capi
    # set-up ahead of the calls that are measured: the address look-up, and the kernels' code
    assert capi.lib().k2amd_mi_forward_noalloc(None, None, None, None, None, 0, 3, 3, 0, 0, None) == 0
    tiny = cases.mi_case(3, dtype=np.float32, max_B=2, max_S=5, max_T=9)
    _both(tiny, device, check_memory=False)
    big = cases.c4_case()                                           # B=32, S=200, T=1000: four chunks a sequence
    _both(big, device)
    small = cases.mi_case(5003, dtype=np.float32, max_B=5, max_S=130, max_T=150,
                          force=dict(modified=False, rand_bd=True))
    _both(small, device)
    _both(cases.mi_case(77, dtype=np.float64, max_B=3, max_S=20, max_T=40), device)   # the fp64 kernels, same array
    _both(big, device)
    # A shape that the pipelined kernels take and whose scratch is beyond the static array: refused
    # with its own status, nothing launched.  (Null pointers: were the refusal ever to fail, the
    # call would be turned down for them instead of reaching a kernel.)
    lib = capi.lib()
    assert lib.k2amd_mi_keeps_log_deriv(2048, 100, 500, 1, 0, 1) == 1
    assert lib.k2amd_mi_workspace_bytes(2048, 100, 500, 1, 0) > (8 << 20)
    assert lib.k2amd_mi_forward_noalloc(None, None, None, None, None, 2048, 100, 500, 1, 0, None) == 6
    # what the exact kernels serve without scratch is not refused for the array's size: a lattice
    # of 2 GiB and more gets as far as the check of its pointers
    assert lib.k2amd_mi_keeps_log_deriv(4096, 200, 1000, 1, 0, 1) == 0
    assert lib.k2amd_mi_forward_noalloc(None, None, None, None, None, 4096, 200, 1000, 1, 0, None) == 1
    with pytest.raises(RuntimeError, match="static array"):
        capi.check(6)
    assert lib.k2amd_mi_forward_noalloc(None, None, None, None, None, 0, 3, 3, 0, 0, None) == 0
    # no wait gave up in any of the calls above (the flag sits in the static array)
    assert lib.k2amd_mi_noalloc_status(torch.cuda.current_stream(device).cuda_stream) == 0
