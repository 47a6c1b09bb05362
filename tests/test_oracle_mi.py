"""Pins the CPU oracle of the MI recursion (oracle/mi_oracle.c) before anything trusts it:
against the reference's own compiled CPU code (fixtures + live, bit-exact), closed forms,
brute-force path enumeration, flow-conservation invariants and finite differences."""
import itertools
import math
import os

import numpy as np
import pytest

import cases
from oracle import mi

FIX = os.path.join(os.path.dirname(__file__), "golden", "mi_ref_fixtures.npz")


def _load_fixtures():
    z = np.load(FIX)
    for name in z["names"]:
        name = str(name)
        bd = z[name + "/boundary"] if bool(z[name + "/has_boundary"]) else None
        yield name, z[name + "/px"], z[name + "/py"], bd, z[name + "/p"], z[name + "/ans"], \
            z[name + "/px_grad"], z[name + "/py_grad"]


def test_port_matches_reference_fixtures_bit_exact():
    n = 0
    for name, px, py, bd, p, ans, gx, gy in _load_fixtures():
        a, pp = mi.mi_forward(px, py, bd)
        assert np.array_equal(a, ans, equal_nan=True), name
        assert np.array_equal(pp, p, equal_nan=True), name
        x, y = mi.mi_backward(px, py, bd, pp)
        assert np.array_equal(x, gx, equal_nan=True), name
        assert np.array_equal(y, gy, equal_nan=True), name
        n += 1
    assert n >= 50


@pytest.mark.skipif(not mi.have_ref(), reason="oracle/_ref not built (needs the reference tree)")
def test_port_matches_compiled_reference_live():
    for seed in range(100, 140):
        for dtype in (np.float32, np.float64):
            c = cases.mi_case(seed, dtype=dtype, max_B=4, max_S=16, max_T=120)
            a1, p1 = mi.mi_forward(c["px"], c["py"], c["boundary"], backend="port")
            a2, p2 = mi.mi_forward(c["px"], c["py"], c["boundary"], backend="ref")
            assert np.array_equal(a1, a2, equal_nan=True)
            assert np.array_equal(p1, p2, equal_nan=True)
            g1 = mi.mi_backward(c["px"], c["py"], c["boundary"], p1, backend="port")
            g2 = mi.mi_backward(c["px"], c["py"], c["boundary"], p2, backend="ref")
            assert np.array_equal(g1[0], g2[0], equal_nan=True)
            assert np.array_equal(g1[1], g2[1], equal_nan=True)


def test_log_add_special_cases():
    inf = float("inf")
    for dt in (np.float32, np.float64):
        assert mi.log_add(-inf, -inf, dt) == -inf          # NaN difference falls through to x
        assert mi.log_add(-inf, 1.5, dt) == dt(1.5)
        assert mi.log_add(2.5, -inf, dt) == dt(2.5)
        assert mi.log_add(0.0, 0.0, dt) == pytest.approx(math.log(2.0), rel=1e-6)
        # below log(eps) the smaller operand is dropped exactly
        cut = 16.0 if dt == np.float32 else 36.1
        assert mi.log_add(0.0, -cut, dt) == 0.0
        assert mi.log_add(0.0, -cut + 0.2, dt) > 0.0
        # symmetric
        assert mi.log_add(1.0, 3.0, dt) == mi.log_add(3.0, 1.0, dt)


@pytest.mark.parametrize("S,T", [(1, 1), (3, 5), (7, 7), (10, 20), (16, 40)])
def test_closed_form_zero_weights(S, T):
    # px = py = 0: exp(ans) counts lattice paths: C(S+T, S) regular, C(T, S) modified.
    for dt, tol in ((np.float32, 2e-5), (np.float64, 1e-12)):
        px = np.zeros((1, S, T + 1), dt)
        py = np.zeros((1, S + 1, T), dt)
        ans, _, _ = mi.mi(px, py)
        assert ans[0] == pytest.approx(math.log(math.comb(S + T, S)), rel=tol)
        if T >= S:
            ans, gx, gy = mi.mi(np.zeros((1, S, T), dt), py)
            assert ans[0] == pytest.approx(math.log(math.comb(T, S)), rel=tol)
            # occupation of the arc (s,t)->(s+1,t+1): paths through it / all paths
            s, t = S // 2, T // 2
            if t >= s and T - t - 1 >= S - s - 1:
                want = math.comb(t, s) * math.comb(T - t - 1, S - s - 1) / math.comb(T, S)
                assert gx[0, s, t] == pytest.approx(want, rel=50 * tol, abs=1e-7)


def _brute_force(px, py, s0, t0, s1, t1, modified):
    """Enumerates every monotone path from (s0,t0) to (s1,t1); returns (log total, px occupancy,
    py occupancy) in float64."""
    ns, nt = s1 - s0, t1 - t0
    gx = np.zeros_like(px, dtype=np.float64)
    gy = np.zeros_like(py, dtype=np.float64)
    total = 0.0
    paths = []
    if modified:
        # nt steps; ns of them are diagonal (emit + advance), the rest horizontal
        for diag in itertools.combinations(range(nt), ns):
            paths.append(["d" if k in diag else "h" for k in range(nt)])
    else:
        for ups in itertools.combinations(range(ns + nt), ns):
            paths.append(["v" if k in ups else "h" for k in range(ns + nt)])
    for path in paths:
        s, t, w, arcs = s0, t0, 0.0, []
        for step in path:
            if step == "h":
                w += py[s, t]; arcs.append(("y", s, t)); t += 1
            elif step == "v":
                w += px[s, t]; arcs.append(("x", s, t)); s += 1
            else:
                w += px[s, t]; arcs.append(("x", s, t)); s += 1; t += 1
        e = math.exp(w)
        total += e
        for kind, s, t in arcs:
            (gx if kind == "x" else gy)[s, t] += e
    return math.log(total), gx / total, gy / total


@pytest.mark.parametrize("modified", [False, True])
def test_brute_force_enumeration(modified):
    rng = np.random.default_rng(7)
    for trial in range(12):
        S, T = int(rng.integers(1, 5)), int(rng.integers(1, 6))
        if modified and T < S:
            T = S
        T1 = T if modified else T + 1
        px = rng.standard_normal((1, S, T1))
        py = rng.standard_normal((1, S + 1, T))
        this_S = int(rng.integers(0, S + 1))
        this_T = int(rng.integers(max(this_S, 1) if modified else 1, T + 1))
        s0 = int(rng.integers(0, S - this_S + 1)); t0 = int(rng.integers(0, T - this_T + 1))
        bd = np.array([[s0, t0, s0 + this_S, t0 + this_T]], dtype=np.int64)
        want, wx, wy = _brute_force(px[0], py[0], s0, t0, s0 + this_S, t0 + this_T, modified)
        for dt, tol in ((np.float64, 1e-12), (np.float32, 2e-5)):
            ans, gx, gy = mi.mi(px.astype(dt), py.astype(dt), bd)
            assert ans[0] == pytest.approx(want, rel=tol, abs=tol)
            np.testing.assert_allclose(gx[0], wx, rtol=10 * tol, atol=tol)
            np.testing.assert_allclose(gy[0], wy, rtol=10 * tol, atol=tol)


def test_flow_conservation():
    # Every path crosses each frame exactly once and emits each symbol exactly once.
    for seed in range(200, 230):
        c = cases.mi_case(seed, dtype=np.float64, max_B=3, max_S=12, max_T=60)
        bd = c["boundary"]
        ans, gx, gy = mi.mi(c["px"], c["py"], bd)
        for b in range(c["B"]):
            s0, t0, s1, t1 = (0, 0, c["S"], c["T"]) if bd is None else [int(v) for v in bd[b]]
            if not np.isfinite(ans[b]):
                continue
            for s in range(s0, s1):
                assert gx[b, s].sum() == pytest.approx(1.0, abs=1e-9)
            for t in range(t0, t1):
                if c["modified"]:
                    tot = gy[b, :, t].sum() + gx[b, :, t].sum()
                else:
                    tot = gy[b, :, t].sum()
                assert tot == pytest.approx(1.0, abs=1e-9)


def test_finite_difference_fp64():
    # The recipe of k2/python/tests/mutual_information_test.py:276-306 with a tighter delta.
    rng = np.random.default_rng(11)
    for modified in (False, True):
        S, T = 5, 9
        T1 = T if modified else T + 1
        px = rng.standard_normal((2, S, T1)); py = rng.standard_normal((2, S + 1, T))
        ans, gx, gy = mi.mi(px, py)
        dpx = rng.standard_normal(px.shape) * 1e-6; dpy = rng.standard_normal(py.shape) * 1e-6
        ans2, _, _ = mi.mi(px + dpx, py + dpy)
        pred = (gx * dpx).sum(axis=(1, 2)) + (gy * dpy).sum(axis=(1, 2))
        np.testing.assert_allclose(ans2 - ans, pred, rtol=1e-4, atol=1e-10)


def test_empty_sequences_and_degenerate_boxes():
    px = np.arange(2 * 3 * 5, dtype=np.float64).reshape(2, 3, 5) * 0.1
    py = np.arange(2 * 4 * 4, dtype=np.float64).reshape(2, 4, 4) * -0.1
    # s_begin == s_end: only the first-row recursion runs, ans = sum of py along that row
    bd = np.array([[1, 1, 1, 4], [2, 0, 2, 3]], dtype=np.int64)
    ans, gx, gy = mi.mi(px, py, bd)
    assert ans[0] == pytest.approx(py[0, 1, 1:4].sum())
    assert ans[1] == pytest.approx(py[1, 2, 0:3].sum())
    assert np.all(gx == 0)
    assert np.all(gy[0, 1, 1:4] == 1) and gy[0].sum() == 3
    # t_begin == t_end on a regular lattice: ans = sum of px down that column
    bd = np.array([[0, 2, 3, 2], [1, 4, 2, 4]], dtype=np.int64)
    ans, gx, gy = mi.mi(px, py, bd)
    assert ans[0] == pytest.approx(px[0, 0:3, 2].sum())
    assert ans[1] == pytest.approx(px[1, 1:2, 4].sum())
    assert np.all(gy == 0)
