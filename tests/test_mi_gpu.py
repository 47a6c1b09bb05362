"""Parity of the HIP MI kernels, called through the C-ABI, against the CPU oracle and the
golden fixtures recorded from the reference's own CPU code.

Tolerances (stated by the task): fp32 |a-b| <= 1e-5 + 1e-4*|b|, fp64 within 1e-10."""
import os

import numpy as np
import pytest
import torch

import cases
import tolerance
from oracle import mi as omi

pytestmark = pytest.mark.gpu

FIX = os.path.join(os.path.dirname(__file__), "golden", "mi_ref_fixtures.npz")
TOL = {np.dtype(np.float32): dict(rtol=1e-4, atol=1e-5), np.dtype(np.float64): dict(rtol=1e-10, atol=1e-10)}


def run_gpu(px, py, bd, device, ans_grad=None):
    from k2_amd import capi
    tpx = torch.from_numpy(px).to(device)
    tpy = torch.from_numpy(py).to(device)
    tbd = None if bd is None else torch.from_numpy(bd).to(device)
    B, S, T1 = px.shape
    T = py.shape[2]
    p = torch.full((B, S + 1, T + 1), float("nan"), dtype=tpx.dtype, device=device)
    ans = capi.mi_forward(tpx, tpy, tbd, p)
    g = torch.ones(B, dtype=tpx.dtype, device=device) if ans_grad is None else torch.from_numpy(ans_grad).to(device)
    g_in = g.clone()
    gx, gy = capi.mi_backward(tpx, tpy, tbd, p, g, overwrite_ans_grad=True)
    torch.cuda.synchronize()
    # the pipelined kernels hand data between workgroups through a scratch buffer that every
    # call must leave exactly as it found it, and no in-kernel wait may have timed out
    assert capi.mi_workspace_is_clean(device), "workspace left dirty"
    capi.mi_workspace_status(device)
    if capi.mi_keeps_log_deriv(tpx, tpy):
        # the same pair with the log-derivative tensor between them: identical bits
        p2 = torch.full_like(p, float("nan"))
        log_deriv = torch.full_like(p, float("nan"))
        ans2 = capi.mi_forward(tpx, tpy, tbd, p2, log_deriv=log_deriv)
        g2 = g_in.clone()
        gx2, gy2 = capi.mi_backward(tpx, tpy, tbd, p2, g2, overwrite_ans_grad=True, log_deriv=log_deriv)
        torch.cuda.synchronize()
        assert capi.mi_workspace_is_clean(device), "workspace left dirty (kept pair)"
        capi.mi_workspace_status(device)
        for name, x, y in (("ans", ans2, ans), ("p", p2, p), ("px_grad", gx2, gx), ("py_grad", gy2, gy),
                           ("ans_grad", g2, g)):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), "kept pair differs in " + name
        # and without p at all, as mutual_information_recursion calls it
        log_deriv.fill_(float("nan"))
        ans3 = capi.mi_forward(tpx, tpy, tbd, None, log_deriv=log_deriv)
        g3 = g_in.clone()
        gx3, gy3 = capi.mi_backward(tpx, tpy, tbd, None, g3, overwrite_ans_grad=True, log_deriv=log_deriv)
        torch.cuda.synchronize()
        assert capi.mi_workspace_is_clean(device), "workspace left dirty (kept pair without p)"
        for name, x, y in (("ans", ans3, ans), ("px_grad", gx3, gx), ("py_grad", gy3, gy), ("ans_grad", g3, g)):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), "kept pair without p differs in " + name
    single = None
    if capi.mi_forward_backward_supported(tpx, tpy):
        # Both recursions in one launch.  That launch sweeps every lattice from both ends and joins
        # the halves in the middle, so its results are not the pair's bits: they are returned for
        # the caller to compare with the oracle like the pair's.  What must be identical is the
        # launch with itself: a second run, and a run without a seed tensor (which stands for ones).
        g4 = g_in.clone()
        ans4, gx4, gy4 = capi.mi_forward_backward(tpx, tpy, tbd, g4, overwrite_ans_grad=True)
        torch.cuda.synchronize()
        assert capi.mi_workspace_is_clean(device), "workspace left dirty (single launch)"
        capi.mi_workspace_status(device)
        g6 = g_in.clone()
        ans6, gx6, gy6 = capi.mi_forward_backward(tpx, tpy, tbd, g6, overwrite_ans_grad=True)
        torch.cuda.synchronize()
        assert capi.mi_workspace_is_clean(device), "workspace left dirty (single launch, again)"
        for name, x, y in (("ans", ans6, ans4), ("px_grad", gx6, gx4), ("py_grad", gy6, gy4), ("ans_grad", g6, g4)):
            assert torch.equal(x.view(torch.int32), y.view(torch.int32)), "single launch not reproducible in " + name
        if ans_grad is None:  # no seed tensor at all stands for ones
            ans5, gx5, gy5 = capi.mi_forward_backward(tpx, tpy, tbd, None)
            torch.cuda.synchronize()
            for name, x, y in (("ans", ans5, ans4), ("px_grad", gx5, gx4), ("py_grad", gy5, gy4)):
                assert torch.equal(x.view(torch.int32), y.view(torch.int32)), "seedless single launch differs in " + name
        single = (ans4.cpu().numpy(), gx4.cpu().numpy(), gy4.cpu().numpy(), g4.cpu().numpy())
    run_gpu.single = single
    return ans.cpu().numpy(), p.cpu().numpy(), gx.cpu().numpy(), gy.cpu().numpy(), g.cpu().numpy(), g_in.cpu().numpy()


# The share of a case's elements that may need the fp64 oracle's arbitration at all (tolerance.py):
# the rule is for a thin tail of elements, not a second tolerance.
MAX_ARBITRATED = 0.03


def _close(name, got, want, want64, tol, mode="relative", max_arbitrated=MAX_ARBITRATED):
    """fp64: the stated tolerance.  fp32: the stated tolerance against the fp32 CPU oracle; the
    elements that miss it are arbitrated by the fp64 oracle element by element (tolerance.py),
    and may be max_arbitrated of the case's elements at most."""
    if tol["rtol"] < 1e-6 or want64 is None:
        with np.errstate(invalid="ignore"):
            ok = np.isclose(got, want, equal_nan=True, **tol)
        assert ok.all(), (name, int((~ok).sum()), got[~ok][:5], want[~ok][:5])
        return None
    st = tolerance.close_f32(name, got, want, want64, mode=mode, max_arbitrated=max_arbitrated)
    if st["arbitrated"]:
        print(f"{name}: {st['beyond_fp32_bar']} of {st['n']} elements beyond the bar against the fp32 result, "
              f"{st['arbitrated']} of them ({100 * st['arbitrated_frac']:.3f} %) beyond it against the fp64 "
              f"result too: arbitrated")
    return st


def check(name, px, py, bd, want, device):
    ans_w, p_w, gx_w, gy_w = want
    ans, p, gx, gy, g_out, g_in = run_gpu(px, py, bd, device)
    tol = TOL[px.dtype]
    w64 = (None, None, None, None)
    if px.dtype == np.float32:
        a64, p64 = omi.mi_forward(px.astype(np.float64), py.astype(np.float64), bd)
        w64 = (a64, p64) + tuple(omi.mi_backward(px.astype(np.float64), py.astype(np.float64), bd, p64))
    _close(name + " ans", ans, ans_w, w64[0], tol, mode="absolute")
    inside = ~np.isnan(p_w)
    assert not np.isnan(p[inside]).any(), name
    if w64[1] is not None:
        with np.errstate(invalid="ignore"):
            p_g, p_32, p_64 = (np.where(inside, a, 0.0) for a in (p, p_w, w64[1]))
        _close(name + " p", p_g, p_32, p_64, tol, mode="absolute")
    else:
        _close(name + " p", p[inside], p_w[inside], None, tol)
    _close(name + " px_grad", gx, gx_w, w64[2], tol)
    _close(name + " py_grad", gy, gy_w, w64[3], tol)
    # the gradient that reaches the start cell equals the one injected at the end cell
    # whenever the end cell is reachable
    ok = np.isfinite(ans_w)
    np.testing.assert_allclose(g_out[ok], g_in[ok], rtol=1e-3)
    if run_gpu.single is not None:  # the single launch, against the same oracles
        ans1, gx1, gy1, g1 = run_gpu.single
        _close(name + " ans (single launch)", ans1, ans_w, w64[0], tol, mode="absolute")
        _close(name + " px_grad (single launch)", gx1, gx_w, w64[2], tol)
        _close(name + " py_grad (single launch)", gy1, gy_w, w64[3], tol)
        np.testing.assert_allclose(g1[ok], g_in[ok], rtol=1e-3)


def test_reference_fixtures(device):
    z = np.load(FIX)
    for name in z["names"]:
        name = str(name)
        bd = z[name + "/boundary"] if bool(z[name + "/has_boundary"]) else None
        check(name, z[name + "/px"], z[name + "/py"], bd,
              (z[name + "/ans"], z[name + "/p"], z[name + "/px_grad"], z[name + "/py_grad"]), device)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_random_cases_vs_oracle(device, dtype):
    for seed in range(300, 360):
        c = cases.mi_case(seed, dtype=dtype)
        ans, p = omi.mi_forward(c["px"], c["py"], c["boundary"])
        gx, gy = omi.mi_backward(c["px"], c["py"], c["boundary"], p)
        check(f"seed{seed}", c["px"], c["py"], c["boundary"], (ans, p, gx, gy), device)


def test_random_multi_chunk_cases_vs_oracle(device):
    """Random shapes of up to five 64-row chunks and many 32-column blocks, random boundaries,
    both lattice types, fp32 (the pipelined kernels in all their launch variants) and fp64."""
    for seed in range(5000, 5040):
        shape = (dict(max_B=12, max_S=300, max_T=400), dict(max_B=40, max_S=130, max_T=150),
                 dict(max_B=3, max_S=70, max_T=1500))[seed % 3]
        c = cases.mi_case(seed, dtype=np.float64 if seed % 5 == 0 else np.float32, **shape)
        ans, p = omi.mi_forward(c["px"], c["py"], c["boundary"])
        gx, gy = omi.mi_backward(c["px"], c["py"], c["boundary"], p)
        check(f"seed{seed}", c["px"], c["py"], c["boundary"], (ans, p, gx, gy), device)


@pytest.mark.parametrize("modified", [False, True])
def test_sequences_shorter_than_a_quad(device, modified):
    """Lattices of one to three cells a side, several to a batch: the 16-byte loads of every
    sequence then start in front of the sequence's own first element (for the mirrored half of the
    single launch up to three floats back), for the first sequences in front of the tensor."""
    rng = np.random.default_rng(77)
    for S, T in ((1, 1), (1, 2), (2, 2), (1, 3), (2, 3), (3, 3)):
        if modified and T < S:
            continue
        B = 7
        T1 = T if modified else T + 1
        px = rng.standard_normal((B, S, T1)).astype(np.float32)
        py = rng.standard_normal((B, S + 1, T)).astype(np.float32)
        full = np.tile(np.array([[0, 0, S, T]], np.int64), (B, 1))
        for bd in (None, full):
            if bd is None and not modified:
                px[:, :, -1] = -np.inf
            ans, p = omi.mi_forward(px, py, bd)
            gx, gy = omi.mi_backward(px, py, bd, p)
            check(f"S{S}T{T}", px, py, bd, (ans, p, gx, gy), device)


@pytest.mark.parametrize("modified", [False, True])
def test_wide_lattice_more_rows_than_a_wavefront(device, modified):
    # S+1 > 256 exercises the row loop of a workgroup; long T exercises many steps.
    rng = np.random.default_rng(5)
    B, S, T = 3, 300, 700
    px = rng.normal(-2, 1, (B, S, T if modified else T + 1)).astype(np.float64)
    py = rng.normal(-2, 1, (B, S + 1, T)).astype(np.float64)
    bd = np.array([[0, 0, 300, 700], [10, 5, 290, 650], [0, 100, 257, 600]], dtype=np.int64)
    ans, p = omi.mi_forward(px, py, bd)
    gx, gy = omi.mi_backward(px, py, bd, p)
    check("wide", px, py, bd, (ans, p, gx, gy), device)


@pytest.mark.parametrize("modified", [False, True])
def test_single_launch_at_its_row_limit(device, modified):
    """S + 2 = 2056 rows, the most the single launch's join keeps in LDS: 33 chunks a half, the
    join's words fetched in nine batches a pass.  fp32 (the pipelined kernels in all their
    variants, the single launch among them)."""
    rng = np.random.default_rng(11)
    B, S, T = 2, 2054, (2070 if modified else 37)
    px = rng.normal(-1.5, 1, (B, S, T if modified else T + 1)).astype(np.float32)
    py = rng.normal(-1.5, 1, (B, S + 1, T)).astype(np.float32)
    bd = np.array([[0, 0, S, T], [3, 1, S - 40, T - 2]], dtype=np.int64)
    ans, p = omi.mi_forward(px, py, bd)
    gx, gy = omi.mi_backward(px, py, bd, p)
    check("tall", px, py, bd, (ans, p, gx, gy), device)


@pytest.mark.parametrize("B", [80, 150])
@pytest.mark.parametrize("modified", [False, True])
def test_more_workgroups_than_compute_units(device, modified, B):
    """Three chunks per sequence on 256 compute units.  B=80: 240 sweeping + 240 clearing
    workgroups, still one launch, two workgroups to a unit.  B=150: 450 chunks, the pair of
    launches, two sweeping workgroups to a unit."""
    rng = np.random.default_rng(77)
    S, T = 140, 170
    px = rng.normal(-2, 1, (B, S, T if modified else T + 1)).astype(np.float32)
    py = rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32)
    bd = cases.random_boundary(rng, B, S, T, modified)
    ans, p = omi.mi_forward(px, py, bd)
    gx, gy = omi.mi_backward(px, py, bd, p)
    check("oversubscribed", px, py, bd, (ans, p, gx, gy), device)


@pytest.mark.parametrize("modified", [False, True])
def test_fp32_multi_chunk_and_block_edges(device, modified):
    """fp32 lattices taller than one 64-row chunk, with T chosen around multiples of the 32-step
    block so that chunk hand-over and the first/last block paths are all exercised."""
    rng = np.random.default_rng(17)
    for (B, S, T) in ((2, 70, 95), (3, 130, 160), (2, 200, 127), (1, 64, 128), (2, 63, 129), (1, 129, 191)):
        px = rng.normal(-2, 1, (B, S, T if modified else T + 1)).astype(np.float32)
        py = rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32)
        for with_bd in (False, True):
            bd = None
            if with_bd:
                rows = []
                for _ in range(B):
                    s_len = int(rng.integers(S // 2, S + 1)); t_len = int(rng.integers(max(s_len, T // 2), T + 1)) if T >= s_len else T
                    s_len = min(s_len, t_len) if modified else s_len
                    s0 = int(rng.integers(0, S - s_len + 1)); t0 = int(rng.integers(0, T - t_len + 1))
                    rows.append([s0, t0, s0 + s_len, t0 + t_len])
                bd = np.array(rows, dtype=np.int64)
            ans, p = omi.mi_forward(px, py, bd)
            gx, gy = omi.mi_backward(px, py, bd, p)
            check(f"S{S}T{T}bd{with_bd}", px, py, bd, (ans, p, gx, gy), device)
    # every T_b around a block boundary, boundaries given
    B, S, T = 8, 70, 200
    px = rng.normal(-2, 1, (B, S, T if modified else T + 1)).astype(np.float32)
    py = rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32)
    bd = np.array([[0, 0, 66 + b % 4, 92 + b] for b in range(B)], dtype=np.int64)
    ans, p = omi.mi_forward(px, py, bd)
    gx, gy = omi.mi_backward(px, py, bd, p)
    check("block-edge sweep", px, py, bd, (ans, p, gx, gy), device)


HIGH_MAGNITUDE_SEEDS = tuple(range(9000, 9024))
MAX_NORM_K = 2.0


def high_magnitude_case(seed):
    """px or py (or both) offset by +15 as in k2/python/tests/mutual_information_test.py:117-130, on
    lattices of several chunks and many blocks: scores of 1e3 .. 2e4, where one fp32 ulp of p is
    1e-4 .. 2e-3 and the reference's own fp32 gradients are percents off the fp64 ones at some
    elements."""
    shape = (dict(max_B=6, max_S=300, max_T=400), dict(max_B=12, max_S=130, max_T=150),
             dict(max_B=3, max_S=70, max_T=1500))[seed % 3]
    which = seed % 4
    return cases.mi_case(seed, dtype=np.float32,
                         force=dict(big_px=which in (0, 2, 3), big_py=which in (1, 2), random_px=True,
                                    random_py=seed % 5 != 0), **shape)


def max_norm_check(name, got, want32, want64, k=MAX_NORM_K):
    """The criterion for inputs on which two correct fp32 recursions cannot agree element by
    element: per sequence, in the max norm, the GPU is no further from the fp64 result than the
    stated tolerance plus k times what the reference's own fp32 code is,
        max |gpu - f64| <= 1e-5 + 1e-4 max |f64| + k max |cpu32 - f64|.
    Returns the largest ratio max|gpu - f64| / max|cpu32 - f64| over the sequences."""
    worst = 0.0
    for b in range(got.shape[0]):
        g, w32, w64 = (np.asarray(a[b], dtype=np.float64).ravel() for a in (got, want32, want64))
        fin = np.isfinite(w64)
        assert (np.isfinite(g) == fin).all() and (np.isfinite(w32) == fin).all(), (name, b)
        if not fin.any():
            continue
        e_gpu, e_ref = np.abs(g[fin] - w64[fin]).max(), np.abs(w32[fin] - w64[fin]).max()
        bound = 1e-5 + 1e-4 * np.abs(w64[fin]).max() + k * e_ref
        assert e_gpu <= bound, (name, b, e_gpu, e_ref, bound)
        worst = max(worst, e_gpu / max(e_ref, 1e-30))
    return worst


def test_high_magnitude_scores_in_the_max_norm(device):
    """Both launch variants on the inputs of high_magnitude_case, each against the fp64 oracle with
    the reference's fp32 code as the yardstick (max_norm_check, k = 2); prints the worst ratio."""
    from k2_amd import capi
    worst = {}
    n_single = 0
    for seed in HIGH_MAGNITUDE_SEEDS:
        c = high_magnitude_case(seed)
        px, py, bd = c["px"], c["py"], c["boundary"]
        a32, p32 = omi.mi_forward(px, py, bd)
        gx32, gy32 = omi.mi_backward(px, py, bd, p32)
        a64, p64 = omi.mi_forward(px.astype(np.float64), py.astype(np.float64), bd)
        gx64, gy64 = omi.mi_backward(px.astype(np.float64), py.astype(np.float64), bd, p64)
        ans, p, gx, gy, g_out, g_in = run_gpu(px, py, bd, device)
        routes = [("two launches", ans, gx, gy)]
        if run_gpu.single is not None:
            n_single += 1
            routes.append(("single launch", run_gpu.single[0], run_gpu.single[1], run_gpu.single[2]))
        for route, a, x, y in routes:
            fin = np.isfinite(a64)
            assert (np.isfinite(a) == fin).all(), (seed, route)
            np.testing.assert_allclose(a[fin], a64[fin], rtol=1e-4, atol=1e-5, err_msg=f"seed {seed} {route} ans")
            for what, got, w32, w64 in (("px_grad", x, gx32, gx64), ("py_grad", y, gy32, gy64)):
                r = max_norm_check(f"seed {seed} {route} {what}", got, w32, w64)
                worst[route, what] = max(worst.get((route, what), 0.0), r)
    assert n_single >= 20
    for (route, what), r in sorted(worst.items()):
        print(f"high-magnitude cases, {route}, {what}: worst max|gpu-fp64| / max|cpu32-fp64| over the sequences = {r:.3f}")


def test_scaled_ans_grad(device):
    c = cases.mi_case(42, dtype=np.float64)
    B = c["B"]
    g = np.linspace(0.5, 3.0, B)
    ans, p = omi.mi_forward(c["px"], c["py"], c["boundary"])
    gx, gy = omi.mi_backward(c["px"], c["py"], c["boundary"], p, ans_grad=g)
    a, pp, x, y, g_out, g_in = run_gpu(c["px"], c["py"], c["boundary"], device, ans_grad=g)
    np.testing.assert_allclose(x, gx, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(y, gy, rtol=1e-10, atol=1e-10)


def test_headline_shape_three_way(device):
    """B=32, S=200, T=1000, modified, random boundary.  |p| reaches a few thousand here, where
    one fp32 ulp is 2.4e-4, so two correct fp32 implementations need not agree to 1e-4 on every
    gradient element; the elements that do not are arbitrated by the fp64 oracle one by one
    (tolerance.py), and their share is bounded and printed."""
    c = cases.c4_case()
    px, py, bd = c["px"], c["py"], c["boundary"]
    ans32, p32 = omi.mi_forward(px, py, bd)
    gx32, gy32 = omi.mi_backward(px, py, bd, p32)
    ans64, p64 = omi.mi_forward(px.astype(np.float64), py.astype(np.float64), bd)
    gx64, gy64 = omi.mi_backward(px.astype(np.float64), py.astype(np.float64), bd, p64)
    ans, p, gx, gy, g_out, g_in = run_gpu(px, py, bd, device)
    # loss: the stated tolerance holds directly
    np.testing.assert_allclose(ans, ans32, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ans, ans64, rtol=1e-4, atol=1e-5)
    for name, g, g32, g64 in (("px_grad", gx, gx32, gx64), ("py_grad", gy, gy32, gy64)):
        st = tolerance.close_f32("c4 " + name, g, g32, g64, max_arbitrated=0.05)
        print(f"c4 {name}: max|gpu-fp64|={st['max_gpu_vs_fp64']:.3e}  max|cpu32-fp64|={st['max_cpu32_vs_fp64']:.3e}  "
              f"max|gpu-cpu32|={st['max_gpu_vs_cpu32']:.3e}  arbitrated {st['arbitrated']} of {st['n']} "
              f"({100 * st['arbitrated_frac']:.4f} %), reference's own 99.9th-percentile relative error "
              f"{st.get('reference_error_quantile_max', 0):.3e}")
    ans1, gx1, gy1, g1 = run_gpu.single
    np.testing.assert_allclose(ans1, ans32, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(ans1, ans64, rtol=1e-4, atol=1e-5)
    for name, g, g32, g64 in (("px_grad", gx1, gx32, gx64), ("py_grad", gy1, gy32, gy64)):
        st = tolerance.close_f32("c4 single launch " + name, g, g32, g64, max_arbitrated=0.05)
        print(f"c4 single launch {name}: max|gpu-fp64|={st['max_gpu_vs_fp64']:.3e}  max|cpu32-fp64|={st['max_cpu32_vs_fp64']:.3e}  "
              f"max|gpu-cpu32|={st['max_gpu_vs_cpu32']:.3e}  arbitrated {st['arbitrated']} of {st['n']} "
              f"({100 * st['arbitrated_frac']:.4f} %)")
    # flow conservation at full size: each symbol row is emitted exactly once
    for grads in (gx, gx1):
        for b in range(c["B"]):
            s1 = int(bd[b, 2])
            np.testing.assert_allclose(grads[b, :s1].sum(axis=1), 1.0, rtol=2e-3)
    np.testing.assert_allclose(g_out, g_in, rtol=2e-3)
    np.testing.assert_allclose(g1, g_in, rtol=2e-3)


@pytest.mark.gpu
def test_pybind_host_matches_ctypes_host(device):
    """The C++ host module and the ctypes binding drive the same kernels: identical bits, on the
    current stream, with a strided px view made contiguous by the host layer, and ans_grad
    overwritten by the gradient that reached the origin."""
    from k2_amd import _k2_amd, capi
    rng = np.random.default_rng(77)
    B, S, T = 3, 70, 90
    px = torch.from_numpy(rng.standard_normal((B, S, T + 1)).astype(np.float32)).to(device)
    py = torch.from_numpy(rng.standard_normal((B, S + 1, T)).astype(np.float32)).to(device)
    bd = torch.tensor([[0, 0, S, T], [3, 5, 66, 80], [0, 10, 70, 90]], dtype=torch.int64, device=device)
    p1 = torch.empty(B, S + 1, T + 1, device=device)
    p2 = torch.empty_like(p1)
    ans1 = capi.mi_forward(px, py, bd, p1)
    px_strided = torch.empty(B, S, 2 * px.shape[2], device=device)[:, :, ::2]
    px_strided.copy_(px)
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        ans2 = _k2_amd.mutual_information_forward(px=px_strided, py=py, boundary=bd, p=p2)
        g2 = torch.full((B,), 2.0, device=device)
        gx2, gy2 = _k2_amd.mutual_information_backward(px=px, py=py, boundary=bd, p=p2, ans_grad=g2)
        # the same through the pair that passes the log-derivatives along
        assert _k2_amd.mutual_information_keeps_log_deriv(px=px, py=py)
        p3 = torch.empty_like(p1)
        kept = torch.full_like(p1, float("nan"))
        ans3 = _k2_amd.mutual_information_forward(px=px_strided, py=py, boundary=bd, p=p3, log_deriv=kept)
        g3 = torch.full((B,), 2.0, device=device)
        gx3, gy3 = _k2_amd.mutual_information_backward(px=px, py=py, boundary=bd, p=p3, ans_grad=g3,
                                                       log_deriv=kept)
    side.synchronize()
    assert torch.equal(ans3, ans2) and torch.equal(gx3, gx2) and torch.equal(gy3, gy2) and torch.equal(g3, g2)
    assert _k2_amd.mutual_information_forward_backward_supported(px=px, py=py)
    # the single launch sweeps the lattices from both ends: the hosts agree with each other bit
    # for bit, and with the pair to the fp32 tolerance
    g5 = torch.full((B,), 2.0, device=device)
    ans5, gx5, gy5 = _k2_amd.mutual_information_forward_backward(px=px_strided, py=py, boundary=bd, ans_grad=g5)
    g6 = torch.full((B,), 2.0, device=device)
    ans6, gx6, gy6 = capi.mi_forward_backward(px, py, bd, g6, overwrite_ans_grad=True)
    torch.cuda.synchronize()
    assert torch.equal(ans5, ans6) and torch.equal(gx5, gx6) and torch.equal(gy5, gy6) and torch.equal(g5, g6)
    for a, b in ((ans5, ans2), (gx5, gx2), (gy5, gy2), (g5, g2)):
        np.testing.assert_allclose(a.cpu().numpy(), b.cpu().numpy(), rtol=1e-4, atol=1e-5)
    with pytest.raises(RuntimeError):  # wrong shape
        _k2_amd.mutual_information_forward(px=px, py=py, boundary=bd, p=p3, log_deriv=kept[:, :-1])
    g1 = torch.full((B,), 2.0, device=device)
    gx1, gy1 = capi.mi_backward(px, py, bd, p1, g1, overwrite_ans_grad=True)
    torch.cuda.synchronize()
    assert torch.equal(ans1, ans2)
    assert torch.equal(gx1, gx2) and torch.equal(gy1, gy2)
    assert torch.equal(g1, g2)
    np.testing.assert_allclose(g2.cpu().numpy(), 2.0, rtol=1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_joint_recursion_identities(device, dtype):
    """The checks of k2/python/tests/mutual_information_test.py:137-166: the joint recursion on
    one input equals the plain one, on two halves it equals it after summing over the inputs,
    and backprop through either gives the same derivative."""
    import k2_amd as k2
    rng = np.random.default_rng(5)
    for modified in (False, True):
        B, S, T = 4, 9, 40
        T1 = T if modified else T + 1
        npx = rng.standard_normal((B, S, T1))
        npy = rng.standard_normal((B, S + 1, T))
        bd = torch.tensor([[0, 0, S, T], [1, 2, 8, 37], [0, 5, 9, 40], [2, 0, 2, 30]],
                          dtype=torch.int64, device=device)
        grads = []
        for which in range(3):
            px = torch.tensor(npx, dtype=dtype, device=device, requires_grad=True)
            py = torch.tensor(npy, dtype=dtype, device=device, requires_grad=True)
            m = k2.mutual_information_recursion(px, py, bd)
            m2 = k2.joint_mutual_information_recursion((px,), (py,), bd)
            m3 = k2.joint_mutual_information_recursion((px * 0.5, px * 0.5), (py * 0.5, py * 0.5), bd)
            assert m2.shape == (1, B) and m3.shape == (2, B)
            tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-10, atol=1e-10)
            assert torch.allclose(m, m2[0], **tol)
            assert torch.allclose(m, m3.sum(dim=0), **tol)
            ((m, m2, m3)[which].sum() * 3).backward()
            grads.append((px.grad.clone(), py.grad.clone()))
        for gx, gy in grads[1:]:
            assert torch.allclose(gx, grads[0][0], rtol=1e-4, atol=1e-5)
            assert torch.allclose(gy, grads[0][1], rtol=1e-4, atol=1e-5)
        # and the plain recursion's derivative is the oracle's occupation probabilities x 3
        a, p = omi.mi_forward(npx, npy, bd.cpu().numpy())
        wx, wy = omi.mi_backward(npx, npy, bd.cpu().numpy(), p)
        np.testing.assert_allclose(grads[0][0].cpu().numpy(), 3 * wx, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(grads[0][1].cpu().numpy(), 3 * wy, rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_log_deriv_is_left_alone_by_the_exact_kernels(device):
    """The fp64 kernels (and the exact kernels that run without a workspace) neither write nor read
    the log-derivative tensor: the hosts say so and results are unchanged."""
    from k2_amd import capi
    rng = np.random.default_rng(3)
    B, S, T = 2, 12, 30
    px = torch.from_numpy(rng.standard_normal((B, S, T + 1))).to(device)
    py = torch.from_numpy(rng.standard_normal((B, S + 1, T))).to(device)
    assert not capi.mi_keeps_log_deriv(px, py)
    p1 = torch.empty(B, S + 1, T + 1, dtype=torch.float64, device=device)
    p2 = torch.empty_like(p1)
    kept = torch.full_like(p1, 7.0)
    a1 = capi.mi_forward(px, py, None, p1)
    a2 = capi.mi_forward(px, py, None, p2, log_deriv=kept)
    g1 = torch.ones(B, dtype=torch.float64, device=device)
    g2 = torch.ones(B, dtype=torch.float64, device=device)
    x1, y1 = capi.mi_backward(px, py, None, p1, g1)
    x2, y2 = capi.mi_backward(px, py, None, p2, g2, log_deriv=kept)
    torch.cuda.synchronize()
    assert torch.equal(a1, a2) and torch.equal(x1, x2) and torch.equal(y1, y2)
    assert bool((kept == 7.0).all())


@pytest.mark.gpu
def test_single_launch_serves_any_batch_and_says_what_it_does_not(device):
    """The single launch hands its work to a fixed set of workgroups in an order in which every
    wait is for work handed out earlier, so it needs no particular number of resident workgroups:
    a batch with several times more chunks than the device has compute units is one launch like
    any other.  fp64 and lattices of more rows than its join keeps are refused (the Python layer
    then makes the two calls)."""
    from k2_amd import capi
    big = torch.zeros(300, 70, 11, device=device)   # 2 * 300 * 2 sweeps each way on 256 compute units
    assert capi.mi_forward_backward_supported(big, torch.zeros(300, 71, 10, device=device))
    px = torch.zeros(2, 5, 8, dtype=torch.float64, device=device)
    py = torch.zeros(2, 6, 7, dtype=torch.float64, device=device)
    assert not capi.mi_forward_backward_supported(px, py)
    with pytest.raises(RuntimeError):
        capi.mi_forward_backward(px, py, None, torch.ones(2, dtype=torch.float64, device=device))
    tall = torch.zeros(1, 2100, 2101, device=device)
    assert not capi.mi_forward_backward_supported(tall, torch.zeros(1, 2101, 2100, device=device))
    import k2_amd as k2
    bx = torch.randn(300, 70, 11, device=device)
    by = torch.randn(300, 71, 10, device=device)
    # (each call overwrites its ans_grad with the gradient that reached the origin)
    scores, gx, gy = capi.mi_forward_backward(bx, by, None, torch.ones(300, device=device))
    small, sx, sy = capi.mi_forward_backward(bx[:4].contiguous(), by[:4].contiguous(), None,
                                             torch.ones(4, device=device))
    torch.cuda.synchronize()
    assert torch.equal(scores[:4], small) and torch.equal(gx[:4], sx) and torch.equal(gy[:4], sy)
    a, p = omi.mi_forward(bx.cpu().numpy(), by.cpu().numpy(), None)
    wx, wy = omi.mi_backward(bx.cpu().numpy(), by.cpu().numpy(), None, p)
    np.testing.assert_allclose(scores.cpu().numpy(), a, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gx.cpu().numpy(), wx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gy.cpu().numpy(), wy, rtol=1e-4, atol=1e-5)
    # With many more (short) half-sweeps than compute units the two launches are the faster way, the
    # library says so, and the Python layer follows: its results are then the pair's bits.
    assert capi.mi_forward_backward_advised(bx[:4].contiguous(), by[:4].contiguous())
    assert not capi.mi_forward_backward_advised(bx, by)
    assert not capi.mi_forward_backward_advised(px, py)
    api_scores, (ax, ay) = k2.mutual_information_recursion(bx, by, None, return_grad=True)
    kept = torch.empty(300, 71, 11, device=device)
    pair_scores = capi.mi_forward(bx, by, None, None, log_deriv=kept)
    qx, qy = capi.mi_backward(bx, by, None, None, torch.ones(300, device=device), log_deriv=kept)
    torch.cuda.synchronize()
    assert torch.equal(api_scores, pair_scores) and torch.equal(ax, qx) and torch.equal(ay, qy)


@pytest.mark.gpu
def test_path_switches(device, monkeypatch):
    """K2AMD_MI_PATH selects the kernels at every call: `generic` runs the exact kernels on fp32
    input that would otherwise take the pipelined ones (same results within the fp32 tolerance),
    `two-launches` withdraws the single launch."""
    from k2_amd import capi
    c = cases.mi_case(11, dtype=np.float32, max_B=3, max_S=90, max_T=120)
    want = run_gpu(c["px"], c["py"], c["boundary"], device)
    tpx = torch.from_numpy(c["px"]).to(device)
    tpy = torch.from_numpy(c["py"]).to(device)
    assert capi.mi_keeps_log_deriv(tpx, tpy) and capi.mi_forward_backward_supported(tpx, tpy)
    monkeypatch.setenv("K2AMD_MI_PATH", "two-launches")
    assert capi.mi_keeps_log_deriv(tpx, tpy) and not capi.mi_forward_backward_supported(tpx, tpy)
    monkeypatch.setenv("K2AMD_MI_PATH", "generic")
    assert not capi.mi_keeps_log_deriv(tpx, tpy) and not capi.mi_forward_backward_supported(tpx, tpy)
    got = run_gpu(c["px"], c["py"], c["boundary"], device)
    for name, a, b in zip(("ans", "p", "px_grad", "py_grad"), got, want):
        _close(name, a, b, None, TOL[np.dtype(np.float32)])


@pytest.mark.gpu
@pytest.mark.parametrize("modified", [False, True])
def test_blocked_and_improbable_edges(device, modified):
    """Edges of log-probability -inf (a few per cent of them, so that whole regions of the lattice
    and some end cells become unreachable) and of -3000 (far below fp32's exp range): all kernels
    must agree with the CPU code's guards (k2/python/csrc/torch/mutual_information_cpu.cu:195-211)
    and the pairs of launches with each other bit for bit.  Sequences whose end cell no path reaches
    take the exact recursion inside the single launch."""
    rng = np.random.default_rng(90 + int(modified))
    B, S, T = 4, 150, 210
    T1 = T if modified else T + 1
    for frac_inf in (0.002, 0.05):
        px = rng.normal(-2.0, 1.0, (B, S, T1)).astype(np.float32)
        py = rng.normal(-2.0, 1.0, (B, S + 1, T)).astype(np.float32)
        for a in (px, py):
            a[rng.random(a.shape) < frac_inf] = -np.inf
            a[rng.random(a.shape) < 0.02] = -3000.0
        bd = np.array([[0, 0, S, T], [2, 3, 140, 200], [0, 10, 64, 74 if modified else 30], [5, 0, 5, 100]],
                      dtype=np.int64)
        ans, p = omi.mi_forward(px, py, bd)
        gx, gy = omi.mi_backward(px, py, bd, p)
        check("blocked %g modified=%s" % (frac_inf, modified), px, py, bd, (ans, p, gx, gy), device)


def test_a_wait_that_gave_up_is_loud(device):
    """The workspace's error flag, raised by a kernel whose bounded wait expired, is forced from
    the host here (every wait then returns after a few polls, so all kernels end normally): ans
    comes out as NaN from both the forward and the single launch, the status call reports it, and
    a freshly initialised workspace serves the same call correctly again."""
    from k2_amd import capi
    rng = np.random.default_rng(9)
    B, S, T = 2, 100, 70
    px = torch.from_numpy(rng.normal(-2, 1, (B, S, T + 1)).astype(np.float32)).to(device)
    py = torch.from_numpy(rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32)).to(device)
    p = torch.empty(B, S + 1, T + 1, device=device)
    good = capi.mi_forward(px, py, None, p).clone()
    assert torch.isfinite(good).all()
    capi.mi_workspace_status(device)
    key = (px.device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = capi._workspaces[key]
    try:
        ws[:16].view(torch.int32)[2] = 1                     # FastHeader::error
        assert torch.isnan(capi.mi_forward(px, py, None, p)).all()
        g = torch.ones(B, device=device)
        capi.mi_backward(px, py, None, p, g, overwrite_ans_grad=True)
        assert torch.isnan(g).all()
        ans, _, _ = capi.mi_forward_backward(px, py, None, torch.ones(B, device=device))
        assert torch.isnan(ans).all()
        with pytest.raises(RuntimeError, match="timed out"):
            capi.mi_workspace_status(device)
    finally:
        torch.cuda.synchronize(device)
        del capi._workspaces[key]                            # the next call initialises a new one
    assert torch.equal(capi.mi_forward(px, py, None, p), good)
    assert capi.mi_workspace_is_clean(device)
    # the host module's own buffers: nothing to recover after ordinary calls
    from k2_amd import native
    import k2_amd as k2
    k2.mutual_information_recursion(px, py, None, return_grad=True)
    assert native.mutual_information_recover_workspaces() == 0


@pytest.mark.parametrize("host", ["extension", "ctypes"])
def test_a_wait_that_gave_up_raises_at_the_next_call(device, host, monkeypatch):
    """Through the API: after a launch whose bounded wait expired (the flag is forced from the
    host, so every kernel ends normally), the NEXT call that reads its boundary raises a
    RuntimeError that names the timeout, without a status call by the user, and the call after
    that one works again: no NaN is handed on silently.  Both host layers."""
    import k2_amd as k2
    from k2_amd import capi, native
    if host == "ctypes":
        monkeypatch.setattr(native, "_ext", None)
    elif native._ext is None:
        pytest.skip("the C++ host module is not built")
    rng = np.random.default_rng(19)
    B, S, T = 3, 90, 120
    px = torch.from_numpy(rng.normal(-2, 1, (B, S, T + 1)).astype(np.float32)).to(device)
    py = torch.from_numpy(rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32)).to(device)
    bd = torch.tensor([[0, 0, S, T], [1, 2, 80, 100], [0, 0, 64, 64]], dtype=torch.int64, device=device)
    good, (gx, gy) = k2.mutual_information_recursion(px, py, bd.clone(), return_grad=True)
    assert torch.isfinite(good).all()
    if host == "ctypes":
        ws = capi._workspaces[(px.device.index, torch.cuda.current_stream(device).cuda_stream)]
    else:
        ws = native._ext.mutual_information_workspace(px)
    assert ws is not None
    torch.cuda.synchronize(device)
    ws[:16].view(torch.int32)[2] = 1                         # FastHeader::error
    with pytest.raises(RuntimeError, match="timed out"):
        k2.mutual_information_recursion(px, py, bd.clone(), return_grad=True)
    again, (gx2, gy2) = k2.mutual_information_recursion(px, py, bd.clone(), return_grad=True)
    assert torch.equal(again, good) and torch.equal(gx2, gx) and torch.equal(gy2, gy)
    assert native.mutual_information_recover_workspaces() == 0


def test_single_launches_on_two_streams(device):
    """Two streams issue the single launch at the same time, each with its own workspace.  The
    clearing workgroups of a launch never wait and leave, so what must be resident together is
    the sweeping workgroups of the launches in flight: 2 x 128 here, on 256 compute units."""
    from k2_amd import capi
    c = cases.c4_case()
    px, py, bd = (torch.from_numpy(c[k]).to(device) for k in ("px", "py", "boundary"))
    ones = torch.ones(px.shape[0], device=device)
    ref = capi.mi_forward_backward(px, py, bd, ones, overwrite_ans_grad=False)
    torch.cuda.synchronize(device)
    streams = [torch.cuda.Stream(device=device) for _ in range(2)]
    outs = [[], []]
    for _ in range(20):
        for i, s in enumerate(streams):
            with torch.cuda.stream(s):
                outs[i].append(capi.mi_forward_backward(px, py, bd, ones, overwrite_ans_grad=False))
    torch.cuda.synchronize(device)
    for i, s in enumerate(streams):
        with torch.cuda.stream(s):
            capi.mi_workspace_status(device)
            assert capi.mi_workspace_is_clean(device)
        for o in outs[i]:
            for a, b in zip(o, ref):
                assert torch.equal(a, b)


@pytest.mark.gpu
def test_fp64_headline_shape_on_the_wave_kernels(device, monkeypatch):
    """fp64 with a workspace takes the kernels of mi_wave.hip (one wavefront per 64-row chunk,
    pipelined): at BASELINE config 4's shape within 1e-10 of the fp64 oracle, like the exact
    one-workgroup-per-sequence kernels, which K2AMD_MI_PATH=generic still selects; and on shapes
    that put chunk borders, the 32-word hand-over blocks and the column clamps at their edges."""
    from k2_amd import capi
    c = cases.c4_case(dtype=np.float64)
    assert capi.lib().k2amd_mi_workspace_bytes(32, 200, 1000, 1, capi.F64) > 0

    def against_oracle(name, px, py, bd):
        ans, p = omi.mi_forward(px, py, bd)
        gx, gy = omi.mi_backward(px, py, bd, p)
        check(name, px, py, bd, (ans, p, gx, gy), device)

    against_oracle("c4 fp64", c["px"], c["py"], c["boundary"])
    monkeypatch.setenv("K2AMD_MI_PATH", "generic")
    against_oracle("c4 fp64, exact kernels", c["px"], c["py"], c["boundary"])
    monkeypatch.delenv("K2AMD_MI_PATH")
    rng = np.random.default_rng(64)
    for modified in (False, True):
        for B, S, T in ((3, 63, 40), (2, 64, 33), (2, 130, 70), (1, 0, 5), (2, 5, 5), (2, 200, 31),
                        (1, 65, 32), (2, 127, 129), (1, 1, 1)):
            if modified and T < S:
                continue
            T1 = T if modified else T + 1
            px = rng.standard_normal((B, S, T1))
            py = rng.standard_normal((B, S + 1, T))
            bd = cases.random_boundary(rng, B, S, T, modified)
            for boundary in (None, bd):
                against_oracle(f"modified={modified} B={B} S={S} T={T} bd={boundary is not None}", px, py, boundary)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_joint_recursion_split_matches_the_torch_chain(device, dtype):
    """The fused split of joint_mutual_information_recursion against the reference's chain of torch
    ops (stack, clamp, product, sum; k2/python/k2/mutual_information.py:404-417) on the same
    occupation probabilities: values and the gradients to every input, with -inf entries in the
    inputs, sizes that are no multiple of anything, one to three pairs."""
    import importlib
    kmi = importlib.import_module("k2_amd.mutual_information")
    g = torch.Generator().manual_seed(5)
    B, S, T = 3, 7, 41
    lowest = torch.finfo(dtype).min
    rtol = 2e-5 if dtype == torch.float32 else 1e-12
    for N in (1, 2, 3):
        def leaf(*shape):
            return (torch.randn(*shape, generator=g, dtype=torch.float64) - 2).to(dtype).to(device).requires_grad_(True)
        px = [leaf(B, S, T + 1) for _ in range(N)]
        py = [leaf(B, S + 1, T) for _ in range(N)]
        px_grad = torch.rand(B, S, T + 1, generator=g, dtype=torch.float64).to(dtype).to(device)
        py_grad = torch.rand(B, S + 1, T, generator=g, dtype=torch.float64).to(dtype).to(device)
        with torch.no_grad():
            px[0][0, 1, 5] = float("-inf")
            px_grad[0, 1, 5] = 0.0
            py[N - 1][2, 0, 0] = float("-inf")
            py_grad[2, 0, 0] = 0.0
        w = torch.randn(N, B, generator=g, dtype=torch.float64).to(dtype).to(device)
        got = kmi._JointProducts.apply(px_grad, py_grad, *px, *py)
        (got * w).sum().backward()
        got_grads = [t.grad.clone() for t in px + py]
        for t in px + py:
            t.grad = None
        px_cat, py_cat = torch.stack(px), torch.stack(py)
        want = ((px_grad.reshape(1, B, -1) * px_cat.reshape(N, B, -1).clamp(min=lowest)).sum(-1)
                + (py_grad.reshape(1, B, -1) * py_cat.reshape(N, B, -1).clamp(min=lowest)).sum(-1))
        (want * w).sum().backward()
        assert got.shape == (N, B) and torch.isfinite(got).all()
        torch.testing.assert_close(got, want.detach(), rtol=rtol, atol=0)
        for a, t in zip(got_grads, px + py):
            torch.testing.assert_close(a, t.grad, rtol=rtol, atol=0)
