"""Pins oracle/rnnt.py against what the reference's own Python chain computes
(tests/golden/rnnt_ref_fixtures.npz, recorded by tests/golden/make_rnnt_fixtures.py from
k2/python/k2/rnnt_loss.py running on the reference's compiled CPU recursion), and pins the delay
penalty independently by brute force over every alignment of small lattices.

Integer outputs (prune ranges, both rules) must be identical; floats within fp32 tolerance."""
import itertools
import math
import os

import numpy as np
import pytest

from oracle import rnnt as orn

FIXTURES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rnnt_ref_fixtures.npz")
F32 = dict(rtol=1e-4, atol=1e-5)


class Fixtures:
    def __init__(self):
        self.f = np.load(FIXTURES)
        self.names = [str(n) for n in self.f["names"]]

    def get(self, name, key):
        k = f"{name}/{key}"
        return self.f[k] if k in self.f.files else None

    def of_kind(self, kind):
        return [n for n in self.names if n.startswith(kind)]


@pytest.fixture(scope="module")
def fx():
    return Fixtures()


def _chain_names():
    return [f"chain{i}" for i in range(8)]


@pytest.mark.parametrize("name", _chain_names())
def test_losses_match_the_reference_chain(fx, name):
    am, lm, sym, bd = (fx.get(name, k) for k in ("am", "lm", "symbols", "boundary"))
    rt, dp = str(fx.get(name, "rnnt_type")), float(fx.get(name, "delay_penalty"))
    loss, (gx, gy) = orn.rnnt_loss_simple(lm, am, sym, 0, bd, rt, dp, "none", True)
    np.testing.assert_allclose(loss, fx.get(name, "simple_loss"), **F32)
    np.testing.assert_allclose(gx, fx.get(name, "px_grad"), **F32)
    np.testing.assert_allclose(gy, fx.get(name, "py_grad"), **F32)
    ranges = fx.get(name, "ranges")
    am_p, lm_p = orn.do_pruning(am, lm, ranges)
    logits = am_p + lm_p
    np.testing.assert_allclose(orn.rnnt_loss_pruned(logits, sym, ranges, 0, bd, rt, dp, "none"),
                               fx.get(name, "pruned_loss"), **F32)
    np.testing.assert_allclose(orn.rnnt_loss_pruned(logits, sym, ranges, 0, bd, rt, dp, "none", True),
                               fx.get(name, "hat_loss"), **F32)
    np.testing.assert_allclose(orn.rnnt_loss(am[:, :, None, :] + lm[:, None, :, :], sym, 0, bd, rt, dp, "none"),
                               fx.get(name, "full_loss"), **F32)
    np.testing.assert_allclose(orn.rnnt_loss_smoothed(lm, am, sym, 0, 0.2, 0.1, bd, rt, dp, "none"),
                               fx.get(name, "smoothed_loss"), **F32)


def _boundary_for_ranges(fx, name):
    bd = fx.get(name, "boundary")
    if bd is None:
        B, S, _ = fx.get(name, "px_grad").shape
        T = fx.get(name, "py_grad").shape[2]
        bd = np.tile(np.array([[0, 0, S, T]], np.int64), (B, 1))
    return bd


@pytest.mark.parametrize("name", _chain_names() + [f"ties{i}" for i in range(10)])
def test_prune_ranges_identical_to_the_reference(fx, name):
    """Same gradients in, same integers out: the reference's occupation gradients on real chains
    (window lengths 2..9 and S+1, the widened range of k2/python/k2/rnnt_loss.py:694-717, both
    lattice types), gradients whose window sums tie exactly, and gradients whose sums differ in
    the last bits, where the order of the additions decides the arg-max."""
    gx, gy = fx.get(name, "px_grad"), fx.get(name, "py_grad")
    bd = _boundary_for_ranges(fx, name)
    R = int(fx.get(name, "s_range"))
    want = fx.get(name, "ranges")
    got = orn.prune_ranges(gx, gy, bd, R)
    assert got.shape == want.shape and got.dtype == np.int64
    assert np.array_equal(got, want)
    want_old = fx.get(name, "ranges_deprecated")
    got_old = orn.prune_ranges_deprecated(gx, gy, bd, R)
    assert got_old.shape == want_old.shape
    assert np.array_equal(got_old, want_old)


@pytest.mark.parametrize("name", ["floor0", "floor1", "floor2"])
def test_logprobs_where_the_shifted_exponentials_underflow(fx, name):
    """am, lm scaled until sum_c exp(lm - max) exp(am - max) underflows for some cells: the
    reference's `+ tiny` keeps the logarithm finite there (k2/python/k2/rnnt_loss.py:172-184)."""
    am, lm = fx.get(name, "am"), fx.get(name, "lm")
    px, py = orn.logprobs_simple(lm, am, fx.get(name, "symbols"), 0, str(fx.get(name, "rnnt_type")),
                                 fx.get(name, "boundary"))
    want_px, want_py = fx.get(name, "px"), fx.get(name, "py")
    if name != "floor2":
        prod = np.matmul(np.exp(lm - lm.max(2, keepdims=True)),
                         np.exp(am - am.max(2, keepdims=True)).transpose(0, 2, 1))
        assert (prod == 0).any()  # the floor is what decides these cells
    assert np.array_equal(np.isfinite(px), np.isfinite(want_px))
    fin = np.isfinite(want_px)
    np.testing.assert_allclose(px[fin], want_px[fin], **F32)
    np.testing.assert_allclose(py, want_py, **F32)


# ---- the delay penalty, by brute force -----------------------------------------------------------

def _enumerate_alignments(lp, symbols, blank, S_b, T_b, rnnt_type, delay_penalty):
    """-log of the sum over every path through the lattice of one sequence, each emitted symbol
    at frame t weighted by an extra ((T_b - 1) / 2 - t) * delay_penalty
    (k2/python/k2/rnnt_loss.py:307-322).  lp [T][S+1][C] = log-softmax of the joiner output.
    regular: a symbol keeps the frame, a blank advances it, and the last step is a blank;
    modified: a symbol advances the frame too; constrained: as modified, and the symbol's
    probability is multiplied by that of a blank in the state it leads to (rnnt_loss.py:220-223)."""
    total = 0.0

    def walk(s, t, w):
        nonlocal total
        if s == S_b and t == T_b:
            total += math.exp(w)
            return
        if t < T_b:  # blank
            walk(s, t + 1, w + lp[t, s, blank])
        if s < S_b and t < T_b:  # symbol s emitted at frame t
            pen = ((T_b - 1) / 2 - t) * delay_penalty
            if rnnt_type == "regular":
                walk(s + 1, t, w + lp[t, s, symbols[s]] + pen)
            elif rnnt_type == "modified":
                walk(s + 1, t + 1, w + lp[t, s, symbols[s]] + pen)
            else:
                walk(s + 1, t + 1, w + lp[t, s, symbols[s]] + lp[t, s + 1, blank] + pen)

    walk(0, 0, 0.0)
    return -math.log(total)


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
@pytest.mark.parametrize("with_boundary", [False, True])
def test_delay_penalty_by_brute_force(rnnt_type, with_boundary):
    rng = np.random.default_rng(7)
    B, T, S, C = 3, 6, 3, 5
    am = rng.standard_normal((B, T, C))
    lm = rng.standard_normal((B, S + 1, C))
    symbols = rng.integers(1, C, (B, S)).astype(np.int64)
    boundary = None
    if with_boundary:
        boundary = np.array([[0, 0, 3, 6], [0, 0, 2, 4], [0, 0, 3, 5]], np.int64)
    logits = am[:, :, None, :] + lm[:, None, :, :]
    lp = logits - np.log(np.exp(logits).sum(-1, keepdims=True))
    for delay in (0.0, 0.25, 1.5):
        want = []
        for b in range(B):
            S_b, T_b = (S, T) if boundary is None else (int(boundary[b, 2]), int(boundary[b, 3]))
            want.append(_enumerate_alignments(lp[b], symbols[b], 0, S_b, T_b, rnnt_type, delay))
        want = np.array(want)
        got = orn.rnnt_loss_simple(lm, am, symbols, 0, boundary, rnnt_type, delay, "none")
        np.testing.assert_allclose(got, want, rtol=1e-10)
        got = orn.rnnt_loss(logits, symbols, 0, boundary, rnnt_type, delay, "none")
        np.testing.assert_allclose(got, want, rtol=1e-10)
        # no pruning (every window starts at 0 and holds all S + 1 rows): the pruned loss is the same
        ranges = np.tile(np.arange(S + 1, dtype=np.int64), (B, T, 1))
        got = orn.rnnt_loss_pruned(logits, symbols, ranges, 0, boundary, rnnt_type, delay, "none")
        np.testing.assert_allclose(got, want, rtol=1e-10)
    # the penalty moves the loss by the expected emission delay: d loss / d lambda at 0 equals
    # sum over symbols of E[t - (T_b - 1) / 2], a number the enumeration gives as well
    eps = 1e-6
    a = orn.rnnt_loss_simple(lm, am, symbols, 0, boundary, rnnt_type, eps, "none")
    b0 = orn.rnnt_loss_simple(lm, am, symbols, 0, boundary, rnnt_type, 0.0, "none")
    _, (gx, _) = orn.rnnt_loss_simple(lm, am, symbols, 0, boundary, rnnt_type, 0.0, "none", True)
    for b in range(B):
        T_b = T if boundary is None else int(boundary[b, 3])
        t = np.arange(gx.shape[2])
        expected = -(gx[b] * ((T_b - 1) / 2 - t)[None, :]).sum()
        assert (a[b] - b0[b]) / eps == pytest.approx(expected, rel=1e-4, abs=1e-6)


@pytest.mark.parametrize("name", [f"joint{i}" for i in range(6)])
def test_joint_recursion_matches_the_reference(fx, name):
    """oracle.mi.joint_mi against k2.joint_mutual_information_recursion's recorded split and the
    gradients torch's autograd gave for it (k2/python/k2/mutual_information.py:314-423)."""
    from oracle import mi as omi
    N = int(fx.get(name, "n"))
    pxs = [fx.get(name, f"px{i}") for i in range(N)]
    pys = [fx.get(name, f"py{i}") for i in range(N)]
    prods, gx, gy = omi.joint_mi(pxs, pys, fx.get(name, "boundary"))
    # the elements are differences of sums of hundreds of terms: absolute tolerance scaled by the
    # size of the terms' sum
    np.testing.assert_allclose(prods, fx.get(name, "prods"), rtol=1e-4, atol=1e-4)
    w = fx.get(name, "weights")
    lo = np.finfo(np.float32).min
    for i in range(N):
        np.testing.assert_allclose(np.where(pxs[i] > lo, w[i][:, None, None] * gx, 0.0), fx.get(name, f"px{i}_grad"), **F32)
        np.testing.assert_allclose(np.where(pys[i] > lo, w[i][:, None, None] * gy, 0.0), fx.get(name, f"py{i}_grad"), **F32)


@pytest.mark.parametrize("name", [f"grad{i}" for i in range(4)])
def test_smoothed_and_hat_losses_of_the_gradient_cases(fx, name):
    am, lm, sym, bd = (fx.get(name, k) for k in ("am", "lm", "symbols", "boundary"))
    rt = str(fx.get(name, "rnnt_type"))
    np.testing.assert_allclose(
        orn.rnnt_loss_smoothed(lm, am, sym, 0, float(fx.get(name, "lm_only_scale")),
                               float(fx.get(name, "am_only_scale")), bd, rt, 0.0, "none"),
        fx.get(name, "smoothed_loss"), **F32)
    np.testing.assert_allclose(
        orn.rnnt_loss_pruned(fx.get(name, "hat_logits"), sym, fx.get(name, "ranges"), 0, bd, rt, 0.0, "none", True),
        fx.get(name, "hat_loss"), **F32)
