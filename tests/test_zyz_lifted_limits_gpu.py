"""Shapes beyond what the kernels' LDS rows and two-dimensional grids used to hold: the exact
mutual-information kernels on sequences with more rows than two LDS rows of 64 KiB take
(mi_generic.hip: the previous step read back from p and from px_grad / py_grad),
get_rnnt_prune_ranges with more frames than its finishing kernel's LDS scans take (prune.hip: the
scans run inside `ranges`), and batches of more than 65535 sequences in the joint recursion's
split (mi_joint.hip).  The switches K2AMD_MI_GENERIC_ROWS=global and K2AMD_PRUNE_SCAN_ROWS=global
select the row-less forms at any size, which must give the bits of the LDS forms.

Written while no GPU was at hand and not run on one yet; the same kernels have run in the host
build (tests/test_cpu_build_kernels.py).  The file's name puts it behind the tests that have run
on a GPU."""
import numpy as np
import pytest
import torch

import cases
import tolerance
from oracle import mi as omi
from oracle import rnnt as orn

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): dict(rtol=1e-4, atol=1e-5), np.dtype(np.float64): dict(rtol=1e-10, atol=1e-10)}


def dev(x, device):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(device)


def _against_the_oracle(name, c, got):
    """ans, px_grad, py_grad of the kernels against the CPU oracle: fp64 within 1e-10; fp32 within
    1e-5 + 1e-4 |x| of the fp32 oracle, the elements that miss it arbitrated by the fp64 oracle
    (tests/tolerance.py), 3 % of them at most."""
    ans, _, gx, gy, _ = got
    px, py, bd = c["px"], c["py"], c["boundary"]
    want_ans, want_p = omi.mi_forward(px, py, bd)
    want_gx, want_gy = omi.mi_backward(px, py, bd, want_p)
    if px.dtype == np.float64:
        for a, b in ((ans, want_ans), (gx, want_gx), (gy, want_gy)):
            np.testing.assert_allclose(a, b, **TOL[np.dtype(np.float64)])
        return
    a64, p64 = omi.mi_forward(px.astype(np.float64), py.astype(np.float64), bd)
    gx64, gy64 = omi.mi_backward(px.astype(np.float64), py.astype(np.float64), bd, p64)
    tolerance.close_f32(name + " ans", ans, want_ans, a64, mode="absolute", max_arbitrated=0.03)
    tolerance.close_f32(name + " px_grad", gx, want_gx, gx64, max_arbitrated=0.03)
    tolerance.close_f32(name + " py_grad", gy, want_gy, gy64, max_arbitrated=0.03)


def _exact_pair(c, device):
    """ans, p, px_grad, py_grad, ans_grad of the exact kernels (the caller has set K2AMD_MI_PATH)."""
    from k2_amd import capi
    px, py, bd = dev(c["px"], device), dev(c["py"], device), dev(c["boundary"], device)
    B, S, T = c["B"], c["S"], c["T"]
    p = torch.full((B, S + 1, T + 1), float("nan"), dtype=px.dtype, device=device)
    ans = capi.mi_forward(px, py, bd, p)
    g = torch.ones(B, dtype=px.dtype, device=device)
    gx, gy = capi.mi_backward(px, py, bd, p, g, overwrite_ans_grad=True)
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (ans, p, gx, gy, g)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_exact_mi_kernels_without_lds_rows_give_the_same_bits(device, dtype, modified, monkeypatch):
    monkeypatch.setenv("K2AMD_MI_PATH", "generic")
    for seed in range(6):
        c = cases.mi_case(900 + seed, dtype=dtype, max_B=3, max_S=40, max_T=70,
                          force={"modified": modified, "rand_bd": seed % 3 != 0})
        if seed % 2:
            rng = np.random.default_rng(seed)
            for name in ("px", "py"):
                c[name][rng.random(c[name].shape) < 0.15] = -np.inf
        print("case", seed, c["B"], c["S"], c["T"], dtype.__name__, modified, flush=True)
        monkeypatch.delenv("K2AMD_MI_GENERIC_ROWS", raising=False)
        lds = _exact_pair(c, device)
        monkeypatch.setenv("K2AMD_MI_GENERIC_ROWS", "global")
        glob = _exact_pair(c, device)
        for name, a, b in zip(("ans", "p", "px_grad", "py_grad", "ans_grad"), lds, glob):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (seed, name)
        _against_the_oracle(f"case {seed}", c, glob)


@pytest.mark.parametrize("full", [False, True])
@pytest.mark.parametrize("dtype,S", [(np.float32, 8200), (np.float64, 4100)])
def test_exact_mi_kernels_beyond_the_lds_rows(device, dtype, S, full, monkeypatch):
    """Tensors with more rows than two LDS rows of 64 KiB hold (S > 8190 in fp32, 4094 in fp64), no
    workspace in play (K2AMD_MI_PATH=generic): served, within the tolerance of the oracle.  Boxes
    of a hundred rows at either end of such a tensor, or all of its rows; log-probabilities close
    to zero, so that p stays small over thousands of rows and the comparison says something about
    the kernels rather than about the conditioning of fp32 sums of that length."""
    monkeypatch.setenv("K2AMD_MI_PATH", "generic")
    monkeypatch.delenv("K2AMD_MI_GENERIC_ROWS", raising=False)
    rng = np.random.default_rng(S)
    B, T = 2, 3
    bd = np.array([[0, 0, S, T], [5, 1, S - 7, T]] if full else [[S - 100, 0, S, T], [3, 1, 90, T]], dtype=np.int64)
    spread = 0.002 if full else 0.3
    c = {"B": B, "S": S, "T": T, "boundary": bd,
         "px": -rng.uniform(0, spread, (B, S, T + 1)).astype(dtype),
         "py": -rng.uniform(0, spread, (B, S + 1, T)).astype(dtype)}
    _against_the_oracle(f"S={S} full={full}", c, _exact_pair(c, device))


@pytest.mark.parametrize("modified", [False, True])
def test_prune_ranges_scans_inside_ranges_give_the_same_integers(device, modified, monkeypatch):
    from k2_amd import capi
    rt = "modified" if modified else "regular"
    for k, (B, T, S, R) in enumerate(((2, 9, 5, 3), (1, 70, 20, 5), (3, 300, 33, 7), (2, 130, 4, 1), (1, 5, 1, 2), (2, 1, 1, 2))):
        c = cases.rnnt_case(660 + k, B, T, S, 6, dtype=np.float32, t_lo=max(S, T - 3), s_lo=max(1, S - 2), modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        want = orn.prune_ranges(gx, gy, c["boundary"], R)
        tgx, tgy, tbd = dev(gx, device), dev(gy, device), dev(c["boundary"], device)
        monkeypatch.delenv("K2AMD_PRUNE_SCAN_ROWS", raising=False)
        lds = capi.prune_ranges(tgx, tgy, tbd, want.shape[2]).cpu().numpy()
        monkeypatch.setenv("K2AMD_PRUNE_SCAN_ROWS", "global")
        glob = capi.prune_ranges(tgx, tgy, tbd, want.shape[2]).cpu().numpy()
        np.testing.assert_array_equal(lds, want)
        np.testing.assert_array_equal(glob, want)


def test_prune_ranges_with_more_frames_than_lds_rows_hold(device, monkeypatch):
    """T = 8300 frames; occupation counts drawn at random stand in for a recursion's gradients
    (the ranges are a function of these two tensors and the boundary alone)."""
    from k2_amd import capi
    monkeypatch.delenv("K2AMD_PRUNE_SCAN_ROWS", raising=False)
    rng = np.random.default_rng(83)
    B, T, S, R = 2, 8300, 6, 3
    gx = rng.random((B, S, T + 1)).astype(np.float32)
    gy = rng.random((B, S + 1, T)).astype(np.float32)
    bd = np.array([[0, 0, S, T], [0, 0, S - 2, T - 11]], dtype=np.int64)
    want = orn.prune_ranges(gx, gy, bd, R)
    got = capi.prune_ranges(dev(gx, device), dev(gy, device), dev(bd, device), R).cpu().numpy()
    np.testing.assert_array_equal(got, want)


BIG_BATCH = 66000


def test_joint_products_of_more_than_65535_sequences(device):
    from k2_amd import capi
    rng = np.random.default_rng(66)
    N, B, S, T = 2, BIG_BATCH, 1, 2
    pxs = [np.minimum(rng.standard_normal((B, S, T + 1)) - 2, 0).astype(np.float32) for _ in range(N)]
    pys = [np.minimum(rng.standard_normal((B, S + 1, T)) - 2, 0).astype(np.float32) for _ in range(N)]
    gx, gy = rng.uniform(0, 1, (B, S, T + 1)).astype(np.float32), rng.uniform(0, 1, (B, S + 1, T)).astype(np.float32)
    got = capi.mi_joint_products([dev(a, device) for a in pxs], [dev(a, device) for a in pys],
                                 dev(gx, device), dev(gy, device)).cpu().numpy()
    want = np.array([(pxs[n].astype(np.float64) * gx).sum(axis=(1, 2)) + (pys[n].astype(np.float64) * gy).sum(axis=(1, 2))
                     for n in range(N)])
    np.testing.assert_allclose(got, want, rtol=2e-5)
