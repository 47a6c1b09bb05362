"""Host-side checks of the Python layer: the shared host copy of a boundary tensor (its early,
non-blocking read needs a device) and the integer arithmetic of the s_range adjustment."""
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


def test_an_early_read_is_for_host_tensors_a_no_op():
    bd = torch.tensor([[0, 0, 3, 7]], dtype=torch.int64)
    kmi.begin_boundary_read(bd)
    kmi.begin_boundary_read(None)
    assert id(bd) not in kmi._boundary_reads
    assert kmi.boundary_rows(bd) == ((0, 0, 3, 7),)


@pytest.mark.gpu
def test_an_early_read_of_a_device_boundary_gives_the_same_rows(device):
    """begin_boundary_read starts the copy, boundary_rows waits for it alone; a tensor written in
    between is read again, and rows already on the host are not asked for twice."""
    want = ((0, 0, 3, 7), (1, 2, 4, 9))
    bd = torch.tensor(want, dtype=torch.int64, device=device)
    kmi.begin_boundary_read(bd)
    assert id(bd) in kmi._boundary_reads
    big = torch.randn(4096, 4096, device=device)
    for _ in range(4):                                      # work queued behind the copy
        big = big @ big * 1e-3
    assert kmi.boundary_rows(bd) == want
    assert id(bd) not in kmi._boundary_reads
    kmi.begin_boundary_read(bd)                             # the rows are here already
    assert id(bd) not in kmi._boundary_reads
    other = bd.clone()
    kmi.begin_boundary_read(other)
    other[0, 2] = 2                                         # written after the copy was queued
    assert kmi.boundary_rows(other) == ((0, 0, 2, 7), (1, 2, 4, 9))
    third = bd.clone()
    kmi.begin_boundary_read(third)
    key = id(third)
    del third
    gc.collect()
    assert key not in kmi._boundary_reads                   # a read nobody asked the rows of


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


# ---- both hosts refuse tensors that disagree in dtype, device or shape ---------------------------
# (GPU tests although nothing is launched: the checks come after "is it a device tensor")

def _hosts():
    from k2_amd import capi
    hosts = [("ctypes", capi)]
    try:
        from k2_amd import _k2_amd
        hosts.append(("pybind", _k2_amd))
    except ImportError:
        pass
    return hosts


def _builder_cases(device):
    """(function name, good positional arguments, {argument index: bad replacement, ...})."""
    f32 = dict(dtype=torch.float32, device=device)
    f64 = dict(dtype=torch.float64, device=device)
    i64 = dict(dtype=torch.int64, device=device)
    B, T, S, C, R = 2, 6, 3, 5, 2
    lm, am = torch.zeros(B, S + 1, C, **f32), torch.zeros(B, T, C, **f32)
    sym, bd = torch.ones(B, S, **i64), torch.tensor([[0, 0, S, T]] * B, **i64)
    px_g, py_g = torch.zeros(B, S, T + 1, **f32), torch.zeros(B, S + 1, T, **f32)
    denom = torch.ones(B, S + 1, T, **f32)
    logits4 = torch.zeros(B, T, S + 1, C, **f32)
    norm4 = torch.zeros(B, T, S + 1, **f32)
    pl = torch.zeros(B, T, R, C, **f32)
    pn = torch.zeros(B, T, R, **f32)
    ranges = torch.zeros(B, T, R, **i64)
    scale = torch.ones(B, **f32)
    bad_sym = [torch.ones(B, S + 1, **i64), torch.ones(B, S, dtype=torch.int32, device=device), sym.cpu()]
    bad_bd = [torch.zeros(B, 3, **i64), torch.zeros(B + 1, 4, **i64), torch.zeros(B, 4, dtype=torch.int32, device=device)]
    bad_gx = [torch.zeros(B, S, T + 1, **f64), torch.zeros(B, S + 1, T + 1, **f32), torch.zeros(B, S, T, **f32)]
    bad_gy = [torch.zeros(B, S + 1, T, **f64), torch.zeros(B, S, T, **f32)]
    return [
        ("logprobs_simple_forward", [lm, am, sym, 0, 0, bd],
         {0: [torch.zeros(B, S + 1, C, **f64), torch.zeros(B, S + 1, C + 1, **f32), torch.zeros(B + 1, S + 1, C, **f32)],
          2: bad_sym, 5: bad_bd, 3: [C, -1], 4: [7]}),
        ("logprobs_joint_forward", [logits4, sym, 0, 0, bd], {1: bad_sym, 4: bad_bd, 2: [C]}),
        ("logprobs_joint_backward", [logits4, norm4, px_g, py_g, sym, bd, 0, 0, scale],
         {1: [torch.zeros(B, T, S, **f32), torch.zeros(B, T, S + 1, **f64)], 2: bad_gx, 3: bad_gy, 4: bad_sym,
          5: bad_bd, 8: [torch.ones(B + 1, **f32), torch.ones(B, **f64)]}),
        ("logprobs_pruned_forward", [pl, sym, ranges, 0, bd, 0, False],
         {1: bad_sym[1:], 2: [torch.zeros(B, T, R + 1, **i64), torch.zeros(B, T, R, dtype=torch.int32, device=device)],
          4: bad_bd}),
        ("logprobs_pruned_backward", [pl, pn, px_g, py_g, sym, ranges, bd, 0, 0, False, scale],
         {1: [torch.zeros(B, T, R + 1, **f32)], 2: bad_gx, 3: bad_gy, 5: [torch.zeros(B, T + 1, R, **i64)], 6: bad_bd}),
        ("prune_ranges", [px_g, py_g, bd, 2],
         {1: bad_gy, 2: bad_bd, 3: [0, S + 2]}),
        ("prune_gather", [lm, ranges], {1: [torch.zeros(B + 1, T, R, **i64), ranges.to(torch.int32)]}),
        ("prune_gather_backward", [torch.zeros(B, T, R, C, **f32), ranges, S + 1],
         {1: [torch.zeros(B, T, R + 1, **i64)], 2: [0]}),
    ]


@pytest.mark.gpu
def test_builders_refuse_disagreeing_tensors(device):
    """A tensor whose dtype, device or shape differs from what the sizes of the call imply would
    be read out of bounds by the kernels (a float32 lm next to a float64 am is read at twice its
    element size): both hosts raise RuntimeError first.  The good arguments are accepted."""
    for host_name, host in _hosts():
        for fn_name, good, bad in _builder_cases(device):
            fn = getattr(host, fn_name)
            fn(*good)
            for index, replacements in bad.items():
                for r in replacements:
                    args = list(good)
                    args[index] = r
                    with pytest.raises(RuntimeError):
                        fn(*args)
                        pytest.fail(f"{host_name}.{fn_name} accepted a bad argument {index}")
        # the simple builder's backward takes the forward's saved tensors
        f32 = dict(dtype=torch.float32, device=device)
        B, T, S, C = 2, 6, 3, 5
        lm_p, am_p, den = torch.ones(B, S + 1, C, **f32), torch.ones(B, T, C, **f32), torch.ones(B, S + 1, T, **f32)
        gx, gy = torch.zeros(B, S, T + 1, **f32), torch.zeros(B, S + 1, T, **f32)
        sym = torch.ones(B, S, dtype=torch.int64, device=device)
        if host_name == "ctypes":
            call = lambda gx=gx, gy=gy, lm_p=lm_p, den=den: host.logprobs_simple_backward(
                gx, gy, sym, None, (lm_p, am_p, den), 0, 0)
        else:
            call = lambda gx=gx, gy=gy, lm_p=lm_p, den=den: host.logprobs_simple_backward(
                gx, gy, sym, None, lm_p, am_p, den, 0, 0, None)
        call()
        for kw in (dict(gx=gx.double()), dict(gy=torch.zeros(B, S, T, **f32)), dict(lm_p=lm_p.double()),
                   dict(den=torch.ones(B, S + 1, T + 1, **f32))):
            with pytest.raises(RuntimeError):
                call(**kw)
    torch.cuda.synchronize(device)


@pytest.mark.gpu
def test_recursion_refuses_disagreeing_tensors(device):
    from k2_amd import capi
    f32 = dict(dtype=torch.float32, device=device)
    B, S, T = 2, 3, 5
    px, py = torch.zeros(B, S, T + 1, **f32), torch.zeros(B, S + 1, T, **f32)
    p = torch.empty(B, S + 1, T + 1, **f32)
    capi.mi_forward(px, py, None, p)
    for bad in (dict(py=py.double()), dict(py=torch.zeros(B, S, T, **f32)), dict(p=torch.empty(B, S + 1, T, **f32)),
                dict(p=p.double()), dict(boundary=torch.zeros(B, 4, dtype=torch.int32, device=device)),
                dict(boundary=torch.zeros(B + 1, 4, dtype=torch.int64, device=device)), dict(px=px.cpu())):
        args = dict(px=px, py=py, boundary=None, p=p)
        args.update(bad)
        with pytest.raises(RuntimeError):
            capi.mi_forward(args["px"], args["py"], args["boundary"], args["p"])
    g = torch.ones(B, **f32)
    with pytest.raises(RuntimeError):
        capi.mi_backward(px, py, None, p, g.double())
    with pytest.raises(RuntimeError):
        capi.mi_backward(px, py, None, p, torch.ones(B + 1, **f32))
    torch.cuda.synchronize(device)
