"""Pins tests/closed_forms.py (the fp64 closed-form gradients the GPU tests use at full size)
against torch autograd over the plain-torch definitions of tests/torch_ref.py at small sizes."""
import numpy as np
import pytest
import torch

import cases
import closed_forms as cf
import torch_ref
from oracle import mi as omi
from oracle import rnnt as orn

TYPES = ["regular", "modified", "constrained"]


def _random_ranges(rng, B, T, S, R):
    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    start[:, 0] = 0
    start[:, -2:] = S - R + 1
    return (np.maximum.accumulate(start, axis=1)[:, :, None] + np.arange(R)).astype(np.int64)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_simple_and_joint_closed_forms_equal_autograd(rnnt_type):
    B, T, S, C = 3, 9, 4, 6
    c = cases.rnnt_case(61, B, T, S, C, dtype=np.float64, t_lo=6, s_lo=2, modified=rnnt_type != "regular")
    bd = torch.from_numpy(c["boundary"])
    sym = torch.from_numpy(c["symbols"])
    w = np.linspace(0.5, 1.5, B)
    lm = torch.from_numpy(c["lm"]).requires_grad_(True)
    am = torch.from_numpy(c["am"]).requires_grad_(True)
    px, py = torch_ref.logprobs_simple(lm, am, sym, 0, rnnt_type, bd)
    (-torch_ref.mi_scores(px, py, bd) * torch.from_numpy(w)).sum().backward()
    opx, opy = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rnnt_type, c["boundary"])
    _, gx, gy = omi.mi(opx, opy, c["boundary"])
    lm_g, am_g = cf.simple_grads(c["lm"], c["am"], c["symbols"], 0, gx, gy, w, rnnt_type)
    np.testing.assert_allclose(lm_g, lm.grad.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(am_g, am.grad.numpy(), rtol=1e-9, atol=1e-12)

    logits = np.random.default_rng(62).standard_normal((B, T, S + 1, C))
    lg = torch.from_numpy(logits).requires_grad_(True)
    px, py = torch_ref.logprobs_from_logits(lg, sym, 0, rnnt_type, bd)
    (-torch_ref.mi_scores(px, py, bd) * torch.from_numpy(w)).sum().backward()
    opx, opy = orn.logprobs_joint(logits, c["symbols"], 0, rnnt_type, c["boundary"])
    _, gx, gy = omi.mi(opx, opy, c["boundary"])
    got = cf.joint_logits_grad(logits, c["symbols"], 0, gx, gy, w, rnnt_type)
    np.testing.assert_allclose(got, lg.grad.numpy(), rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("hat", [False, True])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_pruned_closed_form_equals_autograd(rnnt_type, hat):
    B, T, S, R, C = 3, 10, 5, 3, 7
    c = cases.rnnt_case(63, B, T, S, C, dtype=np.float64, t_lo=8, s_lo=3, modified=rnnt_type != "regular")
    rng = np.random.default_rng(64)
    ranges = _random_ranges(rng, B, T, S, R)
    logits = rng.standard_normal((B, T, R, C))
    bd = torch.from_numpy(c["boundary"])
    w = np.linspace(0.5, 1.5, B)
    lg = torch.from_numpy(logits).requires_grad_(True)
    px, py = torch_ref.logprobs_pruned(lg, torch.from_numpy(c["symbols"]), torch.from_numpy(ranges), 0, bd,
                                       rnnt_type, hat=hat)
    scores = torch_ref.mi_scores(px, py, bd)
    ok = torch.isfinite(scores)
    assert ok.any()
    (-scores[ok] * torch.from_numpy(w)[ok]).sum().backward()
    builder = orn.hat_logprobs_pruned if hat else orn.logprobs_pruned
    opx, opy = builder(logits, c["symbols"], ranges, 0, c["boundary"], rnnt_type)
    _, gx, gy = omi.mi(opx, opy, c["boundary"])
    got = cf.pruned_logits_grad(logits, c["symbols"], ranges, 0, gx, gy, np.where(ok.numpy(), w, 0.0),
                                rnnt_type, hat=hat)
    np.testing.assert_allclose(got, lg.grad.numpy(), rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("scales", [(0.25, 0.1), (0.0, 0.3), (0.4, 0.0)])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_smoothed_closed_form_equals_autograd(rnnt_type, scales):
    B, T, S, C = 3, 9, 4, 6
    c = cases.rnnt_case(65, B, T, S, C, dtype=np.float64, t_lo=6, s_lo=2, modified=rnnt_type != "regular")
    bd = torch.from_numpy(c["boundary"])
    w = np.linspace(0.5, 1.5, B)
    lm = torch.from_numpy(c["lm"]).requires_grad_(True)
    am = torch.from_numpy(c["am"]).requires_grad_(True)
    px, py = torch_ref.logprobs_smoothed(lm, am, torch.from_numpy(c["symbols"]), 0, scales[0], scales[1],
                                         rnnt_type, bd)
    (-torch_ref.mi_scores(px, py, bd) * torch.from_numpy(w)).sum().backward()
    opx, opy = orn.logprobs_smoothed(c["lm"], c["am"], c["symbols"], 0, scales[0], scales[1], c["boundary"],
                                     rnnt_type)
    _, gx, gy = omi.mi(opx, opy, c["boundary"])
    lm_g, am_g = cf.smoothed_grads(c["lm"], c["am"], c["symbols"], 0, scales[0], scales[1], gx, gy, w, rnnt_type)
    np.testing.assert_allclose(lm_g, lm.grad.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(am_g, am.grad.numpy(), rtol=1e-9, atol=1e-12)


def test_hat_closed_form_with_a_label_equal_to_zero():
    """A label equal to 0 under HAT is outside what the variant is meant for (0 is the blank), and
    there k2's code (px = logits[symbol] - logsumexp(logits[1:]) + log(1 - sigmoid(logits[0])),
    rnnt_loss.py:1115-1160) and the textbook distribution part ways; the kernels and the closed
    form follow k2's code.  Pinned by central differences over the oracle's restatement of it."""
    B, T, S, R, C = 2, 6, 4, 2, 5
    c = cases.rnnt_case(66, B, T, S, C, dtype=np.float64, t_lo=5, s_lo=3)
    c["symbols"][:, 1] = 0
    rng = np.random.default_rng(67)
    ranges = _random_ranges(rng, B, T, S, R)
    logits = rng.standard_normal((B, T, R, C))
    px, py = orn.hat_logprobs_pruned(logits, c["symbols"], ranges, 0, c["boundary"], "regular")
    fx, fy = np.isfinite(px), np.isfinite(py)
    wx, wy = np.where(fx, rng.uniform(0.1, 1.0, px.shape), 0.0), np.where(fy, rng.uniform(0.1, 1.0, py.shape), 0.0)

    def value(x):
        a, b = orn.hat_logprobs_pruned(x, c["symbols"], ranges, 0, c["boundary"], "regular")
        return (np.where(fx, a, 0.0) * wx).sum() + (np.where(fy, b, 0.0) * wy).sum()

    got = cf.pruned_logits_grad(logits, c["symbols"], ranges, 0, wx, wy, -np.ones(B), "regular", hat=True)
    want = np.zeros_like(logits)
    eps = 1e-6
    for i in np.ndindex(logits.shape):
        up, down = logits.copy(), logits.copy()
        up[i] += eps
        down[i] -= eps
        want[i] = (value(up) - value(down)) / (2 * eps)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-8)
