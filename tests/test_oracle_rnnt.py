"""Pins the numpy restatement of the rnnt_loss.py op chains (oracle/rnnt.py): the reference's hand
fixture solved by brute force, the identities its tests assert, its doc-test vectors, the
invariants its comments state, and an independent log-softmax formulation."""
import itertools
import math

import numpy as np
import pytest
import torch

import cases
import torch_ref
from oracle import rnnt as orn


def _fixture():
    # k2/python/tests/rnnt_loss_test.py:127-139
    lm = np.array([[[0, 0, 1], [0, 1, 1], [1, 0, 1], [2, 2, 0]]], dtype=np.float32)
    am = np.array([[[0, 1, 2], [0, 0, 0], [0, 2, 4], [0, 3, 3]]], dtype=np.float32)
    symbols = np.array([[0, 1, 0]], dtype=np.int64)
    return lm, am, symbols, 2


def _brute_force_rnnt(lm, am, symbols, blank):
    """Sum over every alignment of the standard transducer: T blanks (one per frame, the last
    one terminating) interleaved with the S symbols; log-probs from log_softmax(am[t] + lm[s])."""
    T, S = am.shape[0], lm.shape[0] - 1
    logits = am[:, None, :].astype(np.float64) + lm[None, :, :].astype(np.float64)
    lp = logits - np.log(np.exp(logits).sum(-1, keepdims=True))
    total = 0.0
    # positions of the S symbol emissions among S+T-1 free slots before the final blank
    for emit in itertools.combinations(range(S + T - 1), S):
        s = t = 0
        w = 0.0
        for slot in range(S + T - 1):
            if slot in emit:
                w += lp[t, s, symbols[s]]; s += 1
            else:
                w += lp[t, s, blank]; t += 1
        assert s == S and t == T - 1
        w += lp[T - 1, S, blank]
        total += math.exp(w)
    return -math.log(total)


def test_hand_fixture_matches_brute_force():
    lm, am, symbols, blank = _fixture()
    want = _brute_force_rnnt(lm[0], am[0], symbols[0], blank)
    got = orn.rnnt_loss_simple(lm, am, symbols, blank, reduction="none")
    assert got[0] == pytest.approx(want, rel=1e-5)
    logits = am[:, :, None, :] + lm[:, None, :, :]
    got2 = orn.rnnt_loss(logits, symbols, blank, reduction="none")
    assert got2[0] == pytest.approx(want, rel=1e-5)
    # invariance to a per-frame constant (k2/python/tests/rnnt_loss_test.py:210-244)
    rng = np.random.default_rng(0)
    lm2 = lm + rng.standard_normal((1, 4, 1)).astype(np.float32)
    am2 = am + rng.standard_normal((1, 4, 1)).astype(np.float32)
    got3 = orn.rnnt_loss_simple(lm2, am2, symbols, blank, reduction="none")
    assert got3[0] == pytest.approx(want, rel=1e-5)


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_simple_equals_joint_and_log_softmax_definition(rnnt_type):
    c = cases.rnnt_case(3, B=3, T=12, S=5, C=9, dtype=np.float64, t_lo=8, s_lo=2,
                        modified=rnnt_type != "regular")
    px1, py1 = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rnnt_type, c["boundary"])
    logits = c["am"][:, :, None, :] + c["lm"][:, None, :, :]
    px2, py2 = orn.logprobs_joint(logits, c["symbols"], 0, rnnt_type, c["boundary"])
    np.testing.assert_allclose(px1, px2, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(py1, py2, rtol=1e-12, atol=1e-12)
    bd = None if c["boundary"] is None else torch.from_numpy(c["boundary"])
    px3, py3 = torch_ref.logprobs_from_logits(torch.from_numpy(logits), torch.from_numpy(c["symbols"]),
                                              0, rnnt_type, bd)
    np.testing.assert_allclose(px1, px3.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(py1, py3.numpy(), rtol=1e-12, atol=1e-12)
    l1 = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], rnnt_type, reduction="none")
    l3 = -torch_ref.mi_scores(px3, py3, bd).numpy()
    np.testing.assert_allclose(l1, l3, rtol=1e-10)


def test_doc_vectors():
    # k2/python/k2/rnnt_loss.py:551-565
    x = np.array([0, 2, 1, 3, 6, 5, 8])
    assert orn.monotonic_lower_bound(x).tolist() == [0, 1, 1, 3, 5, 5, 8]
    x = np.array([[12, 18, 5, 4, 18, 17], [11, 14, 14, 3, 10, 4], [19, 3, 8, 13, 7, 19]])
    assert orn.monotonic_lower_bound(x).tolist() == [[4, 4, 4, 4, 17, 17], [3, 3, 3, 3, 4, 4],
                                                     [3, 3, 7, 7, 7, 19]]
    # k2/python/k2/rnnt_loss.py:965-976
    src = np.arange(15).reshape(1, 3, 5)
    out = orn.roll_by_shifts(src, np.array([[1, 2, 3]]))
    assert out.tolist() == [[[4, 0, 1, 2, 3], [8, 9, 5, 6, 7], [12, 13, 14, 10, 11]]]


def _torch_prune_ranges(px_grad, py_grad, boundary, s_range):
    """The same computation expressed with torch's own CPU reductions (sum over a strided window
    view, argmax, cummin); torch is a dependency of both sides, not the reference."""
    px_grad, py_grad, boundary = map(torch.from_numpy, (px_grad, py_grad, boundary))
    B, S, T1 = px_grad.shape
    T = py_grad.shape[-1]
    S1 = S + 1
    n = S1 - s_range + 1
    win = py_grad.unfold(1, s_range, 1)  # [B, n, T, s_range]
    blk = win.sum(dim=3)
    pad = torch.cat([torch.zeros(B, 1, T1, dtype=px_grad.dtype), px_grad], dim=1)[:, :n, :T]
    s_begin = torch.argmax(blk - pad, dim=1)
    t_idx = torch.arange(T).reshape(1, T)
    fill = torch.clamp(boundary[:, 2].reshape(B, 1) - s_range + 1, min=0)
    s_begin = torch.where(t_idx < boundary[:, 3].reshape(B, 1) - 1, s_begin, fill)
    ramp = ((2 if T1 == T else s_range) - 1) * torch.arange(T)
    rev = lambda v: torch.flip(torch.cummin(torch.flip(v, (-1,)), -1)[0], (-1,))
    s_begin = rev(s_begin)
    s_begin = rev(-(s_begin - ramp)).clamp(min=0)
    s_begin = -(s_begin - ramp)
    return (s_begin.reshape(B, T, 1) + torch.arange(s_range)).numpy()


@pytest.mark.parametrize("modified", [False, True])
def test_prune_ranges_invariants_and_torch_agreement(modified):
    from oracle import mi as omi
    for seed in range(6):
        c = cases.rnnt_case(seed, B=4, T=40, S=12, C=11, t_lo=25, s_lo=5, modified=modified)
        rt = "modified" if modified else "regular"
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        for R in (2, 3, 5):
            ranges = orn.prune_ranges(gx, gy, c["boundary"], R)
            R_eff = ranges.shape[2]
            assert ranges.dtype == np.int64 and ranges.shape[:2] == (4, 40)
            s_begin = ranges[:, :, 0]
            assert (np.diff(ranges, axis=2) == 1).all()
            assert (s_begin[:, 0] == 0).all()                      # starts at symbol 0
            d = np.diff(s_begin, axis=1)
            assert (d >= 0).all()                                  # monotone
            assert (d < (2 if modified else R_eff)).all()          # skips no symbol
            for b in range(4):
                S_b, T_b = int(c["boundary"][b, 2]), int(c["boundary"][b, 3])
                assert (s_begin[b, T_b - 1:] == max(S_b - R_eff + 1, 0)).all()
            want = _torch_prune_ranges(gx, gy, c["boundary"], R_eff)
            assert np.array_equal(ranges, want)


def test_prune_ranges_s_range_adjustments():
    # regular lattice with more symbols than frames needs s_range >= (S_b-1)//T_b + 2
    gx = np.zeros((1, 9, 4), np.float32); gy = np.zeros((1, 10, 3), np.float32)
    bd = np.array([[0, 0, 9, 3]], dtype=np.int64)
    assert orn.prune_ranges(gx, gy, bd, 2).shape[2] == (9 - 1) // 3 + 2
    # s_range > S collapses to S + 1 (no pruning)
    assert orn.prune_ranges(gx, gy, bd, 50).shape[2] == 10


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_no_pruning_equals_joint(rnnt_type):
    # s_range = S+1 with every window starting at 0 keeps the whole lattice
    c = cases.rnnt_case(9, B=2, T=9, S=4, C=7, dtype=np.float64, t_lo=7, s_lo=3,
                        modified=rnnt_type != "regular")
    B, T, S = 2, 9, 4
    logits = np.random.default_rng(1).standard_normal((B, T, S + 1, 7))
    ranges = np.tile(np.arange(S + 1, dtype=np.int64), (B, T, 1))
    a = orn.logprobs_pruned(logits, c["symbols"], ranges, 0, c["boundary"], rnnt_type)
    b = orn.logprobs_joint(logits, c["symbols"], 0, rnnt_type, c["boundary"])
    np.testing.assert_array_equal(a[0], b[0])
    np.testing.assert_array_equal(a[1], b[1])


def test_pruned_matches_band_definition():
    rng = np.random.default_rng(4)
    B, T, S, R, C = 2, 10, 6, 3, 8
    logits = rng.standard_normal((B, T, R, C))
    symbols = rng.integers(1, C, (B, S)).astype(np.int64)
    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    ranges = (start[:, :, None] + np.arange(R)).astype(np.int64)
    bd = np.array([[0, 0, S, T], [0, 0, S - 1, T - 2]], dtype=np.int64)
    px, py = orn.logprobs_pruned(logits, symbols, ranges, 0, bd, "regular")
    px2, py2 = torch_ref.logprobs_pruned(torch.from_numpy(logits), torch.from_numpy(symbols),
                                         torch.from_numpy(ranges), 0, torch.from_numpy(bd), "regular")
    np.testing.assert_allclose(px, px2.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(py, py2.numpy(), rtol=1e-12, atol=1e-12)


def test_do_pruning_is_a_gather():
    rng = np.random.default_rng(5)
    am = rng.standard_normal((2, 5, 3)); lm = rng.standard_normal((2, 7, 4))
    ranges = rng.integers(0, 7, (2, 5, 3)).astype(np.int64)
    a, l = orn.do_pruning(am, lm, ranges)
    assert a.shape == (2, 5, 3, 3) and l.shape == (2, 5, 3, 4)
    for b in range(2):
        for t in range(5):
            for k in range(3):
                assert np.array_equal(l[b, t, k], lm[b, ranges[b, t, k]])
                assert np.array_equal(a[b, t, k], am[b, t])


def test_delay_penalty_and_reduction():
    c = cases.rnnt_case(2, B=3, T=8, S=3, C=6, dtype=np.float64, t_lo=5, s_lo=2)
    base = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="none")
    pen = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], delay_penalty=0.1,
                               reduction="none")
    assert not np.allclose(base, pen)
    assert orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="sum") == \
        pytest.approx(base.sum())
    assert orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="mean") == \
        pytest.approx(base.mean())
    with pytest.raises(ValueError):
        orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="bogus")


# ---- the variants next to the path: HAT, smoothed, the older range rule ------------------------

def _random_band(rng, B, T, S, R):
    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    return (start[:, :, None] + np.arange(R)).astype(np.int64)


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_hat_matches_probability_space_definition(rnnt_type):
    """P(blank) = sigmoid(l0), P(c) = (1 - sigmoid(l0)) softmax(l[1:])[c]: evaluated directly with
    probabilities in fp64 (no logsigmoid, no logsumexp), placed by an explicit loop."""
    rng = np.random.default_rng(31)
    B, T, S, R, C = 2, 9, 5, 3, 6
    logits = rng.standard_normal((B, T, R, C))
    symbols = rng.integers(1, C, (B, S)).astype(np.int64)
    ranges = _random_band(rng, B, T, S, R)
    bd = np.array([[0, 0, S, T], [0, 0, S - 1, T - 2]], dtype=np.int64)
    px, py = orn.hat_logprobs_pruned(logits, symbols, ranges, 0, bd, rnnt_type)
    T1 = T + 1 if rnnt_type == "regular" else T
    want_px = np.full((B, S, T1), -np.inf)
    want_py = np.full((B, S + 1, T), -np.inf)
    for b in range(B):
        for t in range(T):
            for k in range(R):
                s = ranges[b, t, k]
                row = logits[b, t, k]
                pb = 1.0 / (1.0 + math.exp(-row[0]))
                nb = np.exp(row[1:]) / np.exp(row[1:]).sum()
                want_py[b, s, t] = math.log(pb)
                if s < S:
                    want_px[b, s, t] = math.log((1.0 - pb) * nb[symbols[b, s] - 1])
                # the row is a distribution: blank + non-blank mass = 1
                assert pb + (1.0 - pb) * nb.sum() == pytest.approx(1.0, abs=1e-12)
    if rnnt_type == "regular":
        for b in range(B):
            want_px[b, :, bd[b, 3]] = -np.inf
    elif rnnt_type == "constrained":
        want_px = want_px + want_py[:, 1:, :]
    np.testing.assert_allclose(px, want_px, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(py, want_py, rtol=1e-12, atol=1e-12)


def test_hat_reduces_to_softmax_builder_on_its_non_blank_part():
    """With the blank logit at -40, 1 - sigmoid = 1 to fp64 precision and the HAT px equals the
    plain pruned px computed on the row whose column 0 cannot win any mass."""
    rng = np.random.default_rng(32)
    B, T, S, R, C = 2, 8, 4, 2, 5
    logits = rng.standard_normal((B, T, R, C))
    logits[..., 0] = -40.0
    symbols = rng.integers(1, C, (B, S)).astype(np.int64)
    ranges = _random_band(rng, B, T, S, R)
    bd = np.array([[0, 0, S, T], [0, 0, S, T - 1]], dtype=np.int64)
    px_hat, py_hat = orn.hat_logprobs_pruned(logits, symbols, ranges, 0, bd, "modified")
    px, _ = orn.logprobs_pruned(logits, symbols, ranges, 0, bd, "modified")
    np.testing.assert_allclose(px_hat, px, rtol=0, atol=1e-12)
    finite = np.isfinite(py_hat)
    np.testing.assert_allclose(py_hat[finite], -40.0, atol=1e-12)


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_smoothed_with_zero_scales_is_the_simple_loss(rnnt_type):
    # k2/python/tests/rnnt_loss_test.py:167-178
    c = cases.rnnt_case(41, B=3, T=9, S=4, C=6, dtype=np.float64, t_lo=6, s_lo=2,
                        modified=rnnt_type != "regular")
    a = orn.rnnt_loss_smoothed(c["lm"], c["am"], c["symbols"], 0, 0.0, 0.0, c["boundary"], rnnt_type,
                               reduction="none")
    b = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], rnnt_type,
                             reduction="none")
    np.testing.assert_allclose(a, b, rtol=1e-10)


def test_smoothed_parts_are_normalised_distributions_and_shift_invariant():
    """With all the weight on one part, exp(py) + sum over the vocabulary of exp(px-like terms) is
    1 for that part's distribution: checked for the lm-only part (softmax of lm) and the am-only
    part (softmax of am + log unigram) by rebuilding them symbol by symbol; then the invariance
    the reference asserts (k2/python/tests/rnnt_loss_test.py:436-485)."""
    lm, am, symbols, blank = _fixture()
    lm = lm.astype(np.float64); am = am.astype(np.float64)
    B, S1, C = lm.shape
    T = am.shape[1]
    # lm-only: scale 1 on the lm part
    tot_lm = np.zeros((S1,))
    tot_am = np.zeros((T,))
    for sym in range(C):
        if sym == blank:
            continue
        sy = np.full((1, S1 - 1), sym, dtype=np.int64)
        px, _ = orn.logprobs_smoothed(lm, am, sy, blank, 1.0, 0.0, None, "modified")
        tot_lm[:S1 - 1] += np.exp(px[0, :, 0])
        px, _ = orn.logprobs_smoothed(lm, am, sy, blank, 0.0, 1.0, None, "modified")
        tot_am += np.exp(px[0, 0, :])
    _, py = orn.logprobs_smoothed(lm, am, symbols, blank, 1.0, 0.0, None, "modified")
    np.testing.assert_allclose(tot_lm[:S1 - 1] + np.exp(py[0, :S1 - 1, 0]), 1.0, rtol=1e-10)
    _, py = orn.logprobs_smoothed(lm, am, symbols, blank, 0.0, 1.0, None, "modified")
    np.testing.assert_allclose(tot_am + np.exp(py[0, 0, :]), 1.0, rtol=1e-10)
    # and the lm-only symbol probabilities are softmax(lm)
    px, _ = orn.logprobs_smoothed(lm, am, symbols, blank, 1.0, 0.0, None, "modified")
    soft = lm[0] - np.log(np.exp(lm[0]).sum(-1, keepdims=True))
    np.testing.assert_allclose(px[0, :, 0], soft[np.arange(S1 - 1), symbols[0]], rtol=1e-10)

    base = orn.rnnt_loss_smoothed(lm, am, symbols, blank, 0.0, 0.333, None, reduction="none")
    rng = np.random.default_rng(3)
    am2 = am + rng.standard_normal((1, T, 1))
    got = orn.rnnt_loss_smoothed(lm, am2, symbols, blank, 0.0, 0.333, None, reduction="none")
    np.testing.assert_allclose(got, base, rtol=1e-10)


@pytest.mark.parametrize("modified", [False, True])
def test_deprecated_ranges_invariants(modified):
    from oracle import mi as omi
    rt = "modified" if modified else "regular"
    for seed in range(4):
        B, T, S, C = 3, 40 + 7 * seed, 9 + seed, 8
        c = cases.rnnt_case(seed, B, T, S, C, dtype=np.float64, t_lo=T // 2, s_lo=S // 2,
                            modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        for R in (2, 4, S + 3):
            r = orn.prune_ranges_deprecated(gx, gy, c["boundary"], R)
            Reff = min(R, S + 1) if R <= S else S + 1
            assert r.shape == (B, T, Reff) and r.dtype == np.int64
            s0 = r[:, :, 0]
            assert (np.diff(r, axis=2) == 1).all()
            assert (s0 >= 0).all() and (r[:, :, -1] <= S).all()
            d = np.diff(s0, axis=1)
            assert (d >= 0).all() and (d < (2 if modified else Reff)).all()
            # the windows of the true arg-max occupation, before the adjustment, on live frames
            tot = np.concatenate([gx, np.zeros((B, 1, gx.shape[2]))], axis=1)
            tot[:, :, :T] += gy
            for b in range(B):
                t = 0
                best = max(range(S + 2 - Reff), key=lambda s: (tot[b, s:s + Reff, t].sum(), -s))
                assert s0[b, 0] == 0 or s0[b, 0] <= best


def test_joiner_pruned_logits_against_torch_ops_and_loops():
    """oracle.rnnt.joiner_pruned_logits is the joiner the reference's recipes put between
    do_rnnt_pruning and rnnt_loss_pruned, tanh(am_pruned + lm_pruned) through a linear layer.  Pinned
    by torch's own ops on the same numbers (torch.gather as in k2/python/k2/rnnt_loss.py:947-953,
    torch.tanh, torch.nn.functional.linear) and by explicit loops on a tiny case."""
    rng = np.random.default_rng(21)
    B, T, S, R, D, C = 2, 7, 4, 3, 5, 6
    am = rng.standard_normal((B, T, D))
    lm = rng.standard_normal((B, S + 1, D))
    weight = rng.standard_normal((C, D))
    bias = rng.standard_normal(C)
    start = np.sort(rng.integers(0, S + 2 - R, size=(B, T)), axis=1)
    ranges = (start[:, :, None] + np.arange(R)).astype(np.int64)
    got = orn.joiner_pruned_logits(am, lm, ranges, weight, bias)
    tam, tlm, trg = torch.from_numpy(am), torch.from_numpy(lm), torch.from_numpy(ranges)
    am_pruned = tam.unsqueeze(2).expand(B, T, R, D)
    lm_pruned = torch.gather(tlm.unsqueeze(1).expand(B, T, S + 1, D), dim=2,
                             index=trg.reshape(B, T, R, 1).expand(B, T, R, D))
    want = torch.nn.functional.linear(torch.tanh(am_pruned + lm_pruned), torch.from_numpy(weight),
                                      torch.from_numpy(bias)).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
    for b, t, k, c in itertools.product(range(B), range(T), range(R), range(C)):
        z = bias[c] + sum(math.tanh(am[b, t, d] + lm[b, ranges[b, t, k], d]) * weight[c, d] for d in range(D))
        assert abs(got[b, t, k, c] - z) < 1e-12
    no_bias = orn.joiner_pruned_logits(am, lm, ranges, weight)
    np.testing.assert_allclose(no_bias + bias, got, rtol=1e-12, atol=1e-12)
