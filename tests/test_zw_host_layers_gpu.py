"""The two host layers over the C-ABI, the C++ extension (k2_amd/csrc/pybind.cpp) and the ctypes
binding (k2_amd/capi.py), against each other for every family of the RNN-T builders: the same
inputs have to give the same bits, since both make the same C-ABI calls.  (The MI recursion's
pair of host layers is compared in tests/test_mi_gpu.py.)

Written while no GPU was at hand and not run on one yet; the ctypes side has run against the host
build of the kernels (tests/test_cpu_build_host_layer.py), the extension's side in all other GPU
tests.  Also here: the fused joiner's case without frames, written at the same time.  The file's
name puts it behind the tests that have run on a GPU."""
import os

import numpy as np
import pytest
import torch

import cases

pytestmark = pytest.mark.gpu

CODES = {"regular": 0, "modified": 1, "constrained": 2}


def dev(x, device):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(device)


def _same(a, b, what):
    a = a if isinstance(a, (tuple, list)) else (a,)
    b = b if isinstance(b, (tuple, list)) else (b,)
    flat_a = [t for x in a for t in (x if isinstance(x, (tuple, list)) else (x,))]
    flat_b = [t for x in b for t in (x if isinstance(x, (tuple, list)) else (x,))]
    assert len(flat_a) == len(flat_b), what
    for i, (x, y) in enumerate(zip(flat_a, flat_b)):
        if x is None or y is None:
            assert x is None and y is None, (what, i)
            continue
        assert x.dtype == y.dtype and x.shape == y.shape, (what, i)
        assert torch.equal(x, y) or bool(((x == y) | (x.isnan() & y.isnan())).all()), (what, i)


@pytest.fixture
def hosts():
    from k2_amd import capi, native
    if native._ext is None:
        pytest.skip("the C++ host module is not built")
    return native, capi


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_builders(device, hosts, rnnt_type, dtype):
    native, capi = hosts
    code = CODES[rnnt_type]
    B, T, S, C, R = 3, 37, 9, 70, 4
    c = cases.rnnt_case(91, B, T, S, C, dtype=dtype, t_lo=20, s_lo=4, modified=rnnt_type != "regular")
    lm, am, sym, bd = (dev(c[k], device) for k in ("lm", "am", "symbols", "boundary"))
    rng = np.random.default_rng(92)
    scale = dev(np.linspace(0.5, 1.5, B).astype(dtype), device)
    T1 = T + 1 if rnnt_type == "regular" else T
    gx, gy = dev(rng.uniform(0, 1, (B, S, T1)).astype(dtype), device), dev(rng.uniform(0, 1, (B, S + 1, T)).astype(dtype), device)

    a, b = native.logprobs_simple_forward(lm, am, sym, 0, code, bd), capi.logprobs_simple_forward(lm, am, sym, 0, code, bd)
    _same(a, b, "simple forward")
    for seq in (None, scale):
        _same(native.logprobs_simple_backward(gx, gy, sym, bd, a[2], 0, code, seq),
              capi.logprobs_simple_backward(gx, gy, sym, bd, b[2], 0, code, seq), "simple backward")

    logits = dev(rng.standard_normal((B, T, S + 1, C)).astype(dtype), device)
    a, b = native.logprobs_joint_forward(logits, sym, 0, code, bd), capi.logprobs_joint_forward(logits, sym, 0, code, bd)
    _same(a, b, "joint forward")
    for seq in (None, scale):
        _same(native.logprobs_joint_backward(logits, a[2], gx, gy, sym, bd, 0, code, seq),
              capi.logprobs_joint_backward(logits, b[2], gx, gy, sym, bd, 0, code, seq), "joint backward")

    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    start[:, 0], start[:, -2:] = 0, S - R + 1
    ranges = dev((np.maximum.accumulate(start, axis=1)[:, :, None] + np.arange(R)).astype(np.int64), device)
    logits = dev(rng.standard_normal((B, T, R, C)).astype(dtype), device)
    for hat in (False, True):
        a = native.logprobs_pruned_forward(logits, sym, ranges, 0, bd, code, hat)
        b = capi.logprobs_pruned_forward(logits, sym, ranges, 0, bd, code, hat)
        _same(a, b, f"pruned forward hat={hat}")
        for seq in (None, scale):
            _same(native.logprobs_pruned_backward(logits, a[2], gx, gy, sym, ranges, bd, 0, code, hat, seq),
                  capi.logprobs_pruned_backward(logits, b[2], gx, gy, sym, ranges, bd, 0, code, hat, seq),
                  f"pruned backward hat={hat}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pruning_and_lattice(device, hosts, dtype):
    native, capi = hosts
    B, T, S, R, D, C = 3, 41, 11, 4, 48, 9
    rng = np.random.default_rng(93)
    gx, gy = dev(rng.uniform(0, 1, (B, S, T + 1)).astype(dtype), device), dev(rng.uniform(0, 1, (B, S + 1, T)).astype(dtype), device)
    bd = dev(np.array([[0, 0, S, T], [0, 0, S - 2, T - 5], [0, 0, S - 1, T]], np.int64), device)
    ranges = native.prune_ranges(gx, gy, bd, R)
    _same(ranges, capi.prune_ranges(gx, gy, bd, R), "prune ranges")
    lm = dev(rng.standard_normal((B, S + 1, D)).astype(dtype), device)
    _same(native.prune_gather(lm, ranges), capi.prune_gather(lm, ranges), "gather")
    g = dev(rng.standard_normal((B, T, R, D)).astype(dtype), device)
    _same(native.prune_gather_backward(g, ranges, S + 1), capi.prune_gather_backward(g, ranges, S + 1), "gather backward")
    logits = dev(rng.standard_normal((B, T, R, C)).astype(dtype), device)
    sym = dev(rng.integers(1, C, (B, S)).astype(np.int64), device)
    frames = bd[:, 3].to(torch.int32).contiguous()
    _same(native.pruned_ranges_to_lattice(ranges.to(torch.int32), frames, sym, logits),
          capi.pruned_ranges_to_lattice(ranges.to(torch.int32), frames, sym, logits), "lattice")


@pytest.mark.parametrize("modified", [False, True])
def test_deprecated_ranges(device, hosts, modified):
    native, capi = hosts
    B, T, S, R = 3, 41, 11, 4
    rng = np.random.default_rng(94)
    T1 = T if modified else T + 1
    gx, gy = dev(rng.uniform(0, 1, (B, S, T1)).astype(np.float32), device), dev(rng.uniform(0, 1, (B, S + 1, T)).astype(np.float32), device)
    bd = dev(np.array([[0, 0, S, T], [0, 0, S - 2, T - 5], [0, 0, S - 1, T]], np.int64), device)
    a, b = native.prune_ranges(gx, gy, bd, R, deprecated=True), capi.prune_ranges(gx, gy, bd, R, deprecated=True)
    _same(a, b, "deprecated ranges")
    assert not torch.equal(a, native.prune_ranges(gx, gy, bd, R))  # (the two rules differ on random occupation)
    from oracle import rnnt as orn
    assert np.array_equal(a.cpu().numpy(), orn.prune_ranges_deprecated(gx.cpu().numpy(), gy.cpu().numpy(), bd.cpu().numpy(), R))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", ["regular", "modified"])
def test_smoothed_builder(device, hosts, rnnt_type, dtype):
    """The smoothed builder's own kernels through both hosts (they are called directly here,
    whatever K2AMD_SMOOTHED_KERNELS says about the Python layer's choice)."""
    native, capi = hosts
    if torch.device(device).type != "cpu" and os.environ.get("K2AMD_SMOOTHED_KERNELS", "0") != "1":
        pytest.skip("the smoothed builder's kernels have not run on a GPU yet: set K2AMD_SMOOTHED_KERNELS=1")
    code = CODES[rnnt_type]
    B, T, S, C = 3, 13, 5, 33
    c = cases.rnnt_case(95, B, T, S, C, dtype=dtype, t_lo=max(S, T - 3), s_lo=max(1, S - 2), modified=rnnt_type != "regular")
    lm, am, sym, bd = (dev(c[k], device) for k in ("lm", "am", "symbols", "boundary"))
    assert native.smoothed_supported(lm, am) and capi.smoothed_supported(lm, am)
    a = native.logprobs_smoothed_forward(lm, am, sym, 0, 0.25, 0.1, code, bd)
    b = capi.logprobs_smoothed_forward(lm, am, sym, 0, 0.25, 0.1, code, bd)
    _same(a, b, "smoothed forward")
    rng = np.random.default_rng(96)
    T1 = T + 1 if rnnt_type == "regular" else T
    gx, gy = dev(rng.uniform(0, 1, (B, S, T1)).astype(dtype), device), dev(rng.uniform(0, 1, (B, S + 1, T)).astype(dtype), device)
    for seq in (None, dev(np.linspace(0.5, 1.5, B).astype(dtype), device)):
        _same(native.logprobs_smoothed_backward(gx, gy, sym, bd, a[2], 0, 0.25, 0.1, code, seq),
              capi.logprobs_smoothed_backward(gx, gy, sym, bd, b[2], 0, 0.25, 0.1, code, seq), "smoothed backward")


def test_fused_joiner_without_frames(device):
    """T = 0: py is empty, and a regular lattice still has its px column T, which the reference
    pads with -inf (k2/python/k2/rnnt_loss.py:1310-1319); nothing may be left as allocated."""
    from k2_amd import capi
    B, S, R, C, D = 2, 5, 3, 11, 64
    rng = np.random.default_rng(3)
    am = torch.zeros(B, 0, D, device=device)
    lm = dev(rng.standard_normal((B, S + 1, D)).astype(np.float32), device)
    ranges = torch.zeros(B, 0, R, dtype=torch.int64, device=device)
    weight = dev(rng.standard_normal((C, D)).astype(np.float32), device)
    symbols = dev(rng.integers(1, C, (B, S)).astype(np.int64), device)
    px, py, _ = capi.joiner_pruned_forward(am, lm, ranges, weight, None, symbols, 0, None, 0)
    torch.cuda.synchronize(device)
    assert tuple(px.shape) == (B, S, 1) and tuple(py.shape) == (B, S + 1, 0)
    assert torch.isneginf(px).all()
