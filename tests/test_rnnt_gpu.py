"""Parity of the fused RNN-T kernels (log-prob builders, prune ranges, pruning gather) and of the
k2-style Python API against the CPU oracle, plus gradients against plain-torch autograd.

Tolerances: fp32 |a-b| <= 1e-5 + 1e-4*|b|; fp64 1e-10; integer outputs bit-exact."""
import numpy as np
import pytest
import torch

import cases
import closed_forms as cf
import tolerance
import torch_ref
from oracle import mi as omi
from oracle import rnnt as orn

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): dict(rtol=1e-4, atol=1e-5), np.dtype(np.float64): dict(rtol=1e-10, atol=1e-10)}
TYPES = ["regular", "modified", "constrained"]


def three_way(name, got, cpu32, cpu64, max_arbitrated=0.05, mode="relative"):
    """The stated tolerance against the fp32 CPU oracle; elements that miss it (where |p| reaches
    the thousands one fp32 ulp of p is ~1e-4, and the fp32 oracle's own gradients carry that much
    rounding noise) are arbitrated one by one by the fp64 oracle (tolerance.py)."""
    st = tolerance.close_f32(name, got, cpu32, cpu64, max_arbitrated=max_arbitrated, mode=mode)
    print(f"{name}: max|gpu-fp64|={st.get('max_gpu_vs_fp64', 0):.3e} max|cpu32-fp64|={st.get('max_cpu32_vs_fp64', 0):.3e} "
          f"max|gpu-cpu32|={st['max_gpu_vs_cpu32']:.3e} arbitrated {st['arbitrated']} of {st['n']} "
          f"({100 * st['arbitrated_frac']:.4f} %), reference's own 99.9th-percentile error "
          f"{st.get('reference_error_quantile_max', 0):.3e} ({mode})")
    return st


def dev(x, device):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(device)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_logprobs_simple_forward(device, dtype, rnnt_type):
    from k2_amd import capi
    for seed, (B, T, S, C), bd in ((1, (3, 37, 9, 50), True), (2, (2, 70, 66, 130), False), (3, (1, 5, 0, 4), True)):
        c = cases.rnnt_case(seed, B, T, S, C, dtype=dtype, t_lo=max(T // 2, S if rnnt_type != "regular" else 1),
                            s_lo=S // 2, with_boundary=bd, modified=rnnt_type != "regular")
        want = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rnnt_type, c["boundary"])
        px, py, _ = capi.logprobs_simple_forward(dev(c["lm"], device), dev(c["am"], device), dev(c["symbols"], device),
                                                 0, capi.RNNT_TYPES[rnnt_type], dev(c["boundary"], device))
        np.testing.assert_allclose(px.cpu().numpy(), want[0], **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(py.cpu().numpy(), want[1], **TOL[np.dtype(dtype)])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_logprobs_joint_forward(device, dtype, rnnt_type):
    from k2_amd import capi
    rng = np.random.default_rng(11)
    for (B, T, S, C), bd in (((2, 21, 6, 40), True), ((1, 9, 8, 600), False), ((2, 12, 3, 513), True)):
        c = cases.rnnt_case(5, B, T, S, C, dtype=dtype, t_lo=max(T // 2, S), s_lo=S // 2, with_boundary=bd,
                            modified=rnnt_type != "regular")
        logits = rng.standard_normal((B, T, S + 1, C)).astype(dtype)
        logits[0, 0, 0, :] = -np.inf  # an all -inf row: logsumexp must give -inf, not NaN
        logits[0, 0, 0, 1] = 0.5
        want = orn.logprobs_joint(logits, c["symbols"], 0, rnnt_type, c["boundary"])
        px, py, _ = capi.logprobs_joint_forward(dev(logits, device), dev(c["symbols"], device), 0,
                                                capi.RNNT_TYPES[rnnt_type], dev(c["boundary"], device))
        np.testing.assert_allclose(px.cpu().numpy(), want[0], **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(py.cpu().numpy(), want[1], **TOL[np.dtype(dtype)])


def _random_ranges(rng, B, T, S, R):
    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    return (start[:, :, None] + np.arange(R)).astype(np.int64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_logprobs_pruned_forward(device, dtype, rnnt_type):
    from k2_amd import capi
    rng = np.random.default_rng(12)
    for (B, T, S, R, C) in ((2, 30, 10, 4, 33), (3, 17, 5, 6, 100), (1, 8, 7, 2, 500)):
        c = cases.rnnt_case(6, B, T, S, C, dtype=dtype, t_lo=max(T // 2, S), s_lo=S // 2,
                            modified=rnnt_type != "regular")
        logits = rng.standard_normal((B, T, R, C)).astype(dtype)
        ranges = _random_ranges(rng, B, T, S, R)
        want = orn.logprobs_pruned(logits, c["symbols"], ranges, 0, c["boundary"], rnnt_type)
        px, py, _ = capi.logprobs_pruned_forward(dev(logits, device), dev(c["symbols"], device), dev(ranges, device),
                                                 0, dev(c["boundary"], device), capi.RNNT_TYPES[rnnt_type])
        np.testing.assert_allclose(px.cpu().numpy(), want[0], **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(py.cpu().numpy(), want[1], **TOL[np.dtype(dtype)])


@pytest.mark.parametrize("modified", [False, True])
def test_prune_ranges_bit_exact(device, modified):
    from k2_amd import capi
    for seed in range(8):
        B, T, S, C = 4, 60 + 13 * seed, 14 + seed, 12
        c = cases.rnnt_case(seed, B, T, S, C, t_lo=T // 2, s_lo=S // 2, modified=modified)
        rt = "modified" if modified else "regular"
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        for R in (2, 3, 4, 5, 6, 7, 8, 9, S + 1):  # 2..8: kernels specialised on the window length
            want = orn.prune_ranges(gx, gy, c["boundary"], R)
            got = capi.prune_ranges(dev(gx, device), dev(gy, device), dev(c["boundary"], device), want.shape[2])
            assert got.dtype == torch.int64
            assert np.array_equal(got.cpu().numpy(), want), (seed, R)


def test_prune_ranges_widens_a_range_too_small_for_the_boundary(device, capsys):
    """k2/python/k2/rnnt_loss.py:694-729: a regular lattice needs s_range >= (S_b - 1) / T_b + 2
    for every sequence, and never more than S + 1 rows."""
    import k2_amd as k2
    B, T, S = 3, 6, 17
    rng = np.random.default_rng(5)
    boundary = np.array([[0, 0, 17, 4], [0, 0, 9, 6], [0, 0, 1, 3]], np.int64)
    gx = rng.random((B, S, T + 1)).astype(np.float32)
    gy = rng.random((B, S + 1, T)).astype(np.float32)
    bd = dev(boundary, device)
    for R, R_eff in ((2, 6), (6, 6), (7, 7), (18, 18), (40, 18)):
        want = orn.prune_ranges(gx, gy, boundary, R)
        assert want.shape == (B, T, R_eff)
        got = k2.get_rnnt_prune_ranges(dev(gx, device), dev(gy, device), bd, R)
        assert np.array_equal(got.cpu().numpy(), want), R
        # the reference also prints when s_range is S + 1 already (rnnt_loss.py:711-716)
        assert ("Adjusting" in capsys.readouterr().out) == (R != R_eff or R > S)
    bd[0, 3] = 2                                            # written in place: read again
    assert k2.get_rnnt_prune_ranges(dev(gx, device), dev(gy, device), bd, 2).shape[-1] == 10


def test_prune_gather_and_its_gradient(device):
    from k2_amd import capi
    rng = np.random.default_rng(3)
    for dtype in (np.float32, np.float64):
        lm = rng.standard_normal((3, 11, 37)).astype(dtype)
        ranges = _random_ranges(rng, 3, 20, 10, 4)
        _, want = orn.do_pruning(np.zeros((3, 20, 5), dtype), lm, ranges)
        got = capi.prune_gather(dev(lm, device), dev(ranges, device))
        assert np.array_equal(got.cpu().numpy(), want)
        g = rng.standard_normal(want.shape).astype(dtype)
        want_g = np.zeros_like(lm)
        np.add.at(want_g, (np.arange(3)[:, None, None], ranges), g)
        got_g = capi.prune_gather_backward(dev(g, device), dev(ranges, device), 11)
        np.testing.assert_allclose(got_g.cpu().numpy(), want_g, rtol=1e-5 if dtype == np.float32 else 1e-12,
                                   atol=1e-5 if dtype == np.float32 else 1e-12)
    # config 3's shape (T * s_range = 2500 rows per sequence, D = 512), with ranges that stay on one
    # row for many frames as a real lattice's do: the order of the additions is fixed by ranges, so
    # two runs give the same bits
    B, T, S, R, D = 32, 500, 100, 5, 512
    ranges = _random_ranges(rng, B, T, S, R)
    ranges[: B // 2, : T // 2] = np.arange(R)       # 250 frames of 16 sequences on rows 0..4
    g = rng.standard_normal((B, T, R, D)).astype(np.float32)
    first = capi.prune_gather_backward(dev(g, device), dev(ranges, device), S + 1)
    again = capi.prune_gather_backward(dev(g, device), dev(ranges, device), S + 1)
    assert torch.equal(first, again)
    want_g = np.zeros((B, S + 1, D), np.float64)
    np.add.at(want_g, (np.arange(B)[:, None, None], ranges), g.astype(np.float64))
    np.testing.assert_allclose(first.cpu().numpy(), want_g, rtol=1e-5, atol=1e-4)
    for D in (1, 6, 36, 1100):                       # columns that are no multiple of four; more than 1024
        ranges = _random_ranges(rng, 2, 9, 5, 3)
        g = rng.standard_normal((2, 9, 3, D))
        want_g = np.zeros((2, 6, D))
        np.add.at(want_g, (np.arange(2)[:, None, None], ranges), g)
        got_g = capi.prune_gather_backward(dev(g, device), dev(ranges, device), 6)
        np.testing.assert_allclose(got_g.cpu().numpy(), want_g, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_api_losses_and_gradients_vs_autograd(device, rnnt_type):
    """End-to-end through the k2-style API in fp64 against plain torch autograd on the CPU:
    rnnt_loss_simple (grads to lm, am), rnnt_loss (grads to logits), rnnt_loss_pruned."""
    import k2_amd as k2
    B, T, S, C = 3, 11, 4, 7
    c = cases.rnnt_case(21, B, T, S, C, dtype=np.float64, t_lo=7, s_lo=2, modified=rnnt_type != "regular")
    bd_cpu = torch.from_numpy(c["boundary"])
    sym_cpu = torch.from_numpy(c["symbols"])
    w = torch.linspace(0.5, 1.5, B, dtype=torch.float64)

    # --- simple
    lm_r = torch.from_numpy(c["lm"]).requires_grad_(True)
    am_r = torch.from_numpy(c["am"]).requires_grad_(True)
    px, py = torch_ref.logprobs_simple(lm_r, am_r, sym_cpu, 0, rnnt_type, bd_cpu)
    loss_r = -torch_ref.mi_scores(px, py, bd_cpu)
    (loss_r * w).sum().backward()
    lm_g = dev(c["lm"], device).requires_grad_(True)
    am_g = dev(c["am"], device).requires_grad_(True)
    loss_g = k2.rnnt_loss_simple(lm_g, am_g, dev(c["symbols"], device), 0, dev(c["boundary"], device),
                                 rnnt_type=rnnt_type, reduction="none")
    (loss_g * w.to(device)).sum().backward()
    np.testing.assert_allclose(loss_g.detach().cpu().numpy(), loss_r.detach().numpy(), rtol=1e-10)
    np.testing.assert_allclose(lm_g.grad.cpu().numpy(), lm_r.grad.numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(am_g.grad.cpu().numpy(), am_r.grad.numpy(), rtol=1e-8, atol=1e-10)

    # --- joint
    rng = np.random.default_rng(8)
    logits = rng.standard_normal((B, T, S + 1, C))
    lg_r = torch.from_numpy(logits).requires_grad_(True)
    px, py = torch_ref.logprobs_from_logits(lg_r, sym_cpu, 0, rnnt_type, bd_cpu)
    loss_r = -torch_ref.mi_scores(px, py, bd_cpu)
    (loss_r * w).sum().backward()
    lg_g = dev(logits, device).requires_grad_(True)
    loss_g = k2.rnnt_loss(lg_g, dev(c["symbols"], device), 0, dev(c["boundary"], device), rnnt_type=rnnt_type,
                          reduction="none")
    (loss_g * w.to(device)).sum().backward()
    np.testing.assert_allclose(loss_g.detach().cpu().numpy(), loss_r.detach().numpy(), rtol=1e-10)
    np.testing.assert_allclose(lg_g.grad.cpu().numpy(), lg_r.grad.numpy(), rtol=1e-8, atol=1e-10)

    # --- pruned (ranges from the simple pass, as in training)
    loss_s, (gx, gy) = k2.rnnt_loss_simple(lm_g.detach(), am_g.detach(), dev(c["symbols"], device), 0,
                                           dev(c["boundary"], device), rnnt_type=rnnt_type, reduction="none",
                                           return_grad=True)
    ranges = k2.get_rnnt_prune_ranges(gx, gy, dev(c["boundary"], device), 3)
    R = ranges.shape[2]
    am_p, lm_p = k2.do_rnnt_pruning(am_g.detach(), lm_g.detach(), ranges)
    assert am_p.shape == (B, T, R, C) and lm_p.shape == (B, T, R, C)
    plog = rng.standard_normal((B, T, R, C))
    pl_r = torch.from_numpy(plog).requires_grad_(True)
    px, py = torch_ref.logprobs_pruned(pl_r, sym_cpu, ranges.cpu(), 0, bd_cpu, rnnt_type)
    loss_r = -torch_ref.mi_scores(px, py, bd_cpu)
    pl_g = dev(plog, device).requires_grad_(True)
    loss_g = k2.rnnt_loss_pruned(pl_g, dev(c["symbols"], device), ranges, 0, dev(c["boundary"], device),
                                 rnnt_type=rnnt_type, reduction="none")
    np.testing.assert_allclose(loss_g.detach().cpu().numpy(), loss_r.detach().numpy(), rtol=1e-10)
    ok = torch.isfinite(loss_r)
    if ok.any():
        (loss_r[ok] * w[ok]).sum().backward()
        (loss_g[ok.to(device)] * w[ok].to(device)).sum().backward()
        np.testing.assert_allclose(pl_g.grad.cpu().numpy(), pl_r.grad.numpy(), rtol=1e-8, atol=1e-10)


def test_hand_fixture_and_identities(device):
    """k2/python/tests/rnnt_loss_test.py:120-244: simple == joint(am+lm); invariant to per-frame
    constants; the value itself is pinned by brute force in the oracle tests."""
    import k2_amd as k2
    lm = torch.tensor([[[0, 0, 1], [0, 1, 1], [1, 0, 1], [2, 2, 0]]], dtype=torch.float, device=device)
    am = torch.tensor([[[0, 1, 2], [0, 0, 0], [0, 2, 4], [0, 3, 3]]], dtype=torch.float, device=device)
    symbols = torch.tensor([[0, 1, 0]], dtype=torch.long, device=device)
    want = orn.rnnt_loss_simple(lm.cpu().numpy(), am.cpu().numpy(), symbols.cpu().numpy(), 2, reduction="none")
    px, py = k2.get_rnnt_logprobs(lm=lm, am=am, symbols=symbols, termination_symbol=2)
    assert px.shape == (1, 3, 5) and py.shape == (1, 4, 4)
    m = k2.mutual_information_recursion(px=px, py=py, boundary=None)
    np.testing.assert_allclose(-m.cpu().numpy(), want, rtol=1e-5)
    m = k2.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=2, boundary=None, reduction="none")
    np.testing.assert_allclose(m.cpu().numpy(), want, rtol=1e-5)
    logits = am.unsqueeze(2) + lm.unsqueeze(1)
    m = k2.rnnt_loss(logits=logits, symbols=symbols, termination_symbol=2, boundary=None, reduction="none")
    np.testing.assert_allclose(m.cpu().numpy(), want, rtol=1e-5)
    lm2 = lm + torch.randn(1, 4, 1, device=device)
    am2 = am + torch.randn(1, 4, 1, device=device)
    m = k2.rnnt_loss_simple(lm=lm2, am=am2, symbols=symbols, termination_symbol=2, boundary=None, reduction="none")
    np.testing.assert_allclose(m.cpu().numpy(), want, rtol=1e-5)
    with pytest.raises(ValueError):
        k2.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=2, reduction="bogus")
    with pytest.raises(AssertionError):
        k2.get_rnnt_logprobs(lm=lm, am=am[:, :, :2], symbols=symbols, termination_symbol=2)


def test_config2_rnnt_loss_simple_full_size(device):
    """BASELINE config 2: B=16, T=250, S=50, V=500, boundary T_b in [150,250], S_b in [20,50]."""
    import k2_amd as k2
    c = cases.rnnt_case(2, 16, 250, 50, 500, t_lo=150, s_lo=20)
    want, (gx_w, gy_w) = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="none",
                                               return_grad=True)
    got, (gx, gy) = k2.rnnt_loss_simple(dev(c["lm"], device), dev(c["am"], device), dev(c["symbols"], device), 0,
                                        dev(c["boundary"], device), reduction="none", return_grad=True)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=1e-5)
    f64 = lambda a: a.astype(np.float64)
    want64, (gx64, gy64) = orn.rnnt_loss_simple(f64(c["lm"]), f64(c["am"]), c["symbols"], 0, c["boundary"],
                                                 reduction="none", return_grad=True)
    np.testing.assert_allclose(got.cpu().numpy(), want64, rtol=1e-4, atol=1e-5)
    three_way("c2 px_grad", gx.cpu().numpy(), gx_w, gx64)
    three_way("c2 py_grad", gy.cpu().numpy(), gy_w, gy64)


def test_config3_prune_and_pruned_loss_full_size(device):
    """BASELINE config 3: B=32, T=500, S=100, V=500, s_range=5, regular."""
    import k2_amd as k2
    B, T, S, C, R = 32, 500, 100, 500, 5
    c = cases.rnnt_case(3, B, T, S, C, t_lo=300, s_lo=50)
    _, (gx_w, gy_w) = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="none",
                                            return_grad=True)
    # integer output from identical grads: bit-exact
    want_ranges = orn.prune_ranges(gx_w, gy_w, c["boundary"], R)
    got_ranges = k2.get_rnnt_prune_ranges(dev(gx_w, device), dev(gy_w, device), dev(c["boundary"], device), R)
    assert np.array_equal(got_ranges.cpu().numpy(), want_ranges)
    # And through the device pipeline end to end (occupation probabilities from the HIP kernels).
    # Two fp32 pipelines round differently, and a frame whose two best windows are within that
    # noise may go either way: the yardstick is the fp64 pipeline, with which the device's ranges
    # must agree about as often as the reference's own fp32 pipeline does (within one per cent).
    _, (gx, gy) = k2.rnnt_loss_simple(dev(c["lm"], device), dev(c["am"], device), dev(c["symbols"], device), 0,
                                      dev(c["boundary"], device), reduction="none", return_grad=True)
    dev_ranges = k2.get_rnnt_prune_ranges(gx, gy, dev(c["boundary"], device), R).cpu().numpy()
    f64 = lambda a: a.astype(np.float64)
    _, (gx64, gy64) = orn.rnnt_loss_simple(f64(c["lm"]), f64(c["am"]), c["symbols"], 0, c["boundary"],
                                            reduction="none", return_grad=True)
    ranges64 = orn.prune_ranges(gx64, gy64, c["boundary"], R)
    frac_dev, frac_cpu = (dev_ranges == ranges64).mean(), (want_ranges == ranges64).mean()
    print("ranges identical to the fp64 pipeline's: device", frac_dev, " fp32 CPU", frac_cpu,
          " device vs fp32 CPU", (dev_ranges == want_ranges).mean())
    assert frac_dev > frac_cpu - 0.01
    logits = np.random.default_rng(33).standard_normal((B, T, R, C)).astype(np.float32)
    want = orn.rnnt_loss_pruned(logits, c["symbols"], want_ranges, 0, c["boundary"], reduction="none")
    got = k2.rnnt_loss_pruned(dev(logits, device), dev(c["symbols"], device), dev(want_ranges, device), 0,
                              dev(c["boundary"], device), reduction="none")
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=1e-5)


def test_config5_rnnt_loss_full_size(device):
    """BASELINE config 5: B=8, T=300, S=75, V=500, joiner logits [8,300,76,500]."""
    import k2_amd as k2
    B, T, S, C = 8, 300, 75, 500
    c = cases.rnnt_case(5, B, T, S, C, t_lo=200, s_lo=40)
    logits = np.random.default_rng(55).standard_normal((B, T, S + 1, C)).astype(np.float32)
    want = orn.rnnt_loss(logits, c["symbols"], 0, c["boundary"], reduction="none")
    got = k2.rnnt_loss(dev(logits, device), dev(c["symbols"], device), 0, dev(c["boundary"], device),
                       reduction="none")
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=1e-5)


# ---- the variants next to the path -------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_hat_logprobs_pruned_forward(device, dtype, rnnt_type):
    """get_hat_logprobs_pruned through the C-ABI against the oracle: vectorised rows (C % 4 == 0),
    odd row lengths, rows longer than the register path and rows of 2 and 3 columns."""
    from k2_amd import capi
    rng = np.random.default_rng(52)
    for (B, T, S, R, C) in ((2, 30, 10, 4, 33), (3, 17, 5, 6, 100), (1, 8, 7, 2, 500), (2, 9, 4, 3, 2),
                            (2, 9, 4, 3, 3), (1, 6, 3, 2, 1100)):
        c = cases.rnnt_case(6, B, T, S, max(C, 2), dtype=dtype, t_lo=max(T // 2, S), s_lo=S // 2,
                            modified=rnnt_type != "regular")
        symbols = np.minimum(c["symbols"], C - 1)
        logits = (3 * rng.standard_normal((B, T, R, C))).astype(dtype)
        ranges = _random_ranges(rng, B, T, S, R)
        want = orn.hat_logprobs_pruned(logits, symbols, ranges, 0, c["boundary"], rnnt_type)
        px, py, _ = capi.logprobs_pruned_forward(dev(logits, device), dev(symbols, device), dev(ranges, device),
                                                 0, dev(c["boundary"], device), capi.RNNT_TYPES[rnnt_type],
                                                 hat=True)
        np.testing.assert_allclose(px.cpu().numpy(), want[0], **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(py.cpu().numpy(), want[1], **TOL[np.dtype(dtype)])


@pytest.mark.parametrize("C", [3, 7, 12])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_hat_loss_and_gradient_vs_autograd(device, rnnt_type, C):
    """rnnt_loss_pruned(use_hat_loss=True) in fp64 against torch autograd on the CPU over the
    probability-space definition; C = 3 takes the one-kernel backward, 12 the vectorised one."""
    import k2_amd as k2
    B, T, S, R = 3, 11, 4, 3
    c = cases.rnnt_case(23, B, T, S, C, dtype=np.float64, t_lo=7, s_lo=2, modified=rnnt_type != "regular")
    rng = np.random.default_rng(9)
    ranges = _random_ranges(rng, B, T, S, R)
    ranges[:, -3:, :] = np.arange(S - R + 1, S + 1)  # the band reaches the last symbol
    ranges[:, 0, :] = np.arange(R)
    ranges = np.maximum.accumulate(ranges, axis=1)
    plog = rng.standard_normal((B, T, R, C))
    w = torch.linspace(0.5, 1.5, B, dtype=torch.float64)
    bd_cpu = torch.from_numpy(c["boundary"])
    pl_r = torch.from_numpy(plog).requires_grad_(True)
    px, py = torch_ref.logprobs_pruned(pl_r, torch.from_numpy(c["symbols"]), torch.from_numpy(ranges), 0,
                                       bd_cpu, rnnt_type, hat=True)
    loss_r = -torch_ref.mi_scores(px, py, bd_cpu)
    pl_g = dev(plog, device).requires_grad_(True)
    loss_g = k2.rnnt_loss_pruned(pl_g, dev(c["symbols"], device), dev(ranges, device), 0,
                                 dev(c["boundary"], device), rnnt_type=rnnt_type, reduction="none",
                                 use_hat_loss=True)
    np.testing.assert_allclose(loss_g.detach().cpu().numpy(), loss_r.detach().numpy(), rtol=1e-10)
    ok = torch.isfinite(loss_r)
    assert ok.any()
    (loss_r[ok] * w[ok]).sum().backward()
    (loss_g[ok.to(device)] * w[ok].to(device)).sum().backward()
    np.testing.assert_allclose(pl_g.grad.cpu().numpy(), pl_r.grad.numpy(), rtol=1e-8, atol=1e-10)
    with pytest.raises(AssertionError):
        k2.get_hat_logprobs_pruned(pl_g, dev(c["symbols"], device), dev(ranges, device), 1,
                                   dev(c["boundary"], device), rnnt_type)


def test_hat_gradient_fp32_vectorised_rows(device):
    """fp32, C = 500 (the 16-byte path of the row kernels) against the fp64 result of the same
    kernels, whose gradient the test above ties to autograd."""
    import k2_amd as k2
    B, T, S, R, C = 4, 40, 12, 4, 500
    c = cases.rnnt_case(29, B, T, S, C, t_lo=T, s_lo=S)  # full lengths: the band below ends at (S, T)
    rng = np.random.default_rng(10)
    start = np.minimum(np.arange(T)[None, :] * (S - R + 2) // T, S - R + 1)
    ranges = (np.repeat(start, B, axis=0)[:, :, None] + np.arange(R)).astype(np.int64)
    plog = rng.standard_normal((B, T, R, C)).astype(np.float32)
    res = {}
    for dt in (torch.float32, torch.float64):
        x = dev(plog, device).to(dt).requires_grad_(True)
        loss = k2.rnnt_loss_pruned(x, dev(c["symbols"], device), dev(ranges, device), 0,
                                   dev(c["boundary"], device), reduction="sum", use_hat_loss=True)
        loss.backward()
        res[dt] = (loss.item(), x.grad.double().cpu().numpy())
    assert np.isfinite(res[torch.float64][0])
    assert res[torch.float32][0] == pytest.approx(res[torch.float64][0], rel=1e-4)
    np.testing.assert_allclose(res[torch.float32][1], res[torch.float64][1], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_smoothed_loss_values_gradients_and_identities(device, rnnt_type):
    """rnnt_loss_smoothed: fp64 values against the oracle, gradients against torch autograd over
    the three-distribution definition, scales (0, 0) == rnnt_loss_simple
    (k2/python/tests/rnnt_loss_test.py:167-178) and invariance to per-frame constants (:436-485)."""
    import k2_amd as k2
    B, T, S, C = 3, 10, 4, 6
    c = cases.rnnt_case(61, B, T, S, C, dtype=np.float64, t_lo=7, s_lo=2, modified=rnnt_type != "regular")
    sym, bd = dev(c["symbols"], device), dev(c["boundary"], device)
    want = orn.rnnt_loss_smoothed(c["lm"], c["am"], c["symbols"], 0, 0.25, 0.1, c["boundary"], rnnt_type,
                                  reduction="none")
    lm_g = dev(c["lm"], device).requires_grad_(True)
    am_g = dev(c["am"], device).requires_grad_(True)
    got = k2.rnnt_loss_smoothed(lm_g, am_g, sym, 0, lm_only_scale=0.25, am_only_scale=0.1, boundary=bd,
                                rnnt_type=rnnt_type, reduction="none")
    np.testing.assert_allclose(got.detach().cpu().numpy(), want, rtol=1e-10)
    px, py = k2.get_rnnt_logprobs_smoothed(lm_g, am_g, sym, 0, 0.25, 0.1, bd, rnnt_type)
    wpx, wpy = orn.logprobs_smoothed(c["lm"], c["am"], c["symbols"], 0, 0.25, 0.1, c["boundary"], rnnt_type)
    np.testing.assert_allclose(px.detach().cpu().numpy(), wpx, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(py.detach().cpu().numpy(), wpy, rtol=1e-10, atol=1e-10)

    w = torch.linspace(0.5, 1.5, B, dtype=torch.float64)
    lm_r = torch.from_numpy(c["lm"]).requires_grad_(True)
    am_r = torch.from_numpy(c["am"]).requires_grad_(True)
    bd_cpu = torch.from_numpy(c["boundary"])
    rpx, rpy = torch_ref.logprobs_smoothed(lm_r, am_r, torch.from_numpy(c["symbols"]), 0, 0.25, 0.1,
                                           rnnt_type, bd_cpu)
    loss_r = -torch_ref.mi_scores(rpx, rpy, bd_cpu)
    np.testing.assert_allclose(loss_r.detach().numpy(), want, rtol=1e-10)
    (loss_r * w).sum().backward()
    (got * w.to(device)).sum().backward()
    np.testing.assert_allclose(lm_g.grad.cpu().numpy(), lm_r.grad.numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(am_g.grad.cpu().numpy(), am_r.grad.numpy(), rtol=1e-8, atol=1e-10)

    plain = k2.rnnt_loss_simple(lm_g.detach(), am_g.detach(), sym, 0, bd, rnnt_type=rnnt_type, reduction="none")
    zero = k2.rnnt_loss_smoothed(lm_g.detach(), am_g.detach(), sym, 0, lm_only_scale=0.0, am_only_scale=0.0,
                                 boundary=bd, rnnt_type=rnnt_type, reduction="none")
    np.testing.assert_allclose(zero.cpu().numpy(), plain.cpu().numpy(), rtol=1e-10)
    shifted = k2.rnnt_loss_smoothed(lm_g.detach(), am_g.detach() + torch.randn(B, T, 1, device=device, dtype=torch.float64),
                                    sym, 0, lm_only_scale=0.0, am_only_scale=0.333, boundary=bd,
                                    rnnt_type=rnnt_type, reduction="none")
    base = k2.rnnt_loss_smoothed(lm_g.detach(), am_g.detach(), sym, 0, lm_only_scale=0.0, am_only_scale=0.333,
                                 boundary=bd, rnnt_type=rnnt_type, reduction="none")
    np.testing.assert_allclose(shifted.cpu().numpy(), base.cpu().numpy(), rtol=1e-9)
    loss, (gx, gy) = k2.rnnt_loss_smoothed(lm_g.detach(), am_g.detach(), sym, 0, boundary=bd, rnnt_type=rnnt_type,
                                           return_grad=True)
    assert loss.ndim == 0 and gx.shape == px.shape and gy.shape == py.shape


@pytest.mark.parametrize("modified", [False, True])
def test_deprecated_prune_ranges_matches_oracle(device, modified):
    import k2_amd as k2
    rt = "modified" if modified else "regular"
    for seed in range(3):
        B, T, S, C = 3, 50 + 9 * seed, 11 + seed, 9
        c = cases.rnnt_case(seed, B, T, S, C, dtype=np.float64, t_lo=T // 2, s_lo=S // 2, modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        for R in (2, 5, S + 2):
            want = orn.prune_ranges_deprecated(gx, gy, c["boundary"], R)
            got = k2.get_rnnt_prune_ranges_deprecated(dev(gx, device), dev(gy, device),
                                                      dev(c["boundary"], device), R)
            assert got.dtype == torch.int64
            assert np.array_equal(got.cpu().numpy(), want), (seed, R)


def test_variants_degenerate_shapes(device):
    """S = 0 (no symbols), s_range = S + 1 (no pruning) and an empty batch through the HAT and
    smoothed builders."""
    import k2_amd as k2
    B, T, C = 2, 5, 4
    logits = torch.randn(B, T, 1, C, device=device, dtype=torch.float64)
    sym0 = torch.zeros(B, 0, dtype=torch.long, device=device)
    ranges0 = torch.zeros(B, T, 1, dtype=torch.long, device=device)
    bd = torch.tensor([[0, 0, 0, T], [0, 0, 0, T - 1]], device=device)
    loss = k2.rnnt_loss_pruned(logits, sym0, ranges0, 0, bd, reduction="none", use_hat_loss=True)
    want = -torch.nn.functional.logsigmoid(logits[..., 0, 0])  # only blanks: sum of log sigmoid
    assert loss[0].item() == pytest.approx(want[0].sum().item(), rel=1e-10)
    assert loss[1].item() == pytest.approx(want[1, :T - 1].sum().item(), rel=1e-10)
    S = 3
    c = cases.rnnt_case(77, B, T, S, C, dtype=np.float64)
    full = torch.randn(B, T, S + 1, C, device=device, dtype=torch.float64)
    ranges = torch.arange(S + 1, device=device).expand(B, T, S + 1).contiguous()
    a = k2.rnnt_loss_pruned(full, dev(c["symbols"], device), ranges, 0, dev(c["boundary"], device), reduction="none")
    b = k2.rnnt_loss(full, dev(c["symbols"], device), 0, dev(c["boundary"], device), reduction="none")
    np.testing.assert_allclose(a.cpu().numpy(), b.cpu().numpy(), rtol=1e-12)
    lm = torch.randn(0, S + 1, C, device=device)
    am = torch.randn(0, T, C, device=device)
    e = k2.rnnt_loss_smoothed(lm, am, torch.zeros(0, S, dtype=torch.long, device=device), 0, reduction="none")
    assert e.shape == (0,)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_logprobs_simple_fp32_products_vs_fp64(device, rnnt_type):
    """The fp32 batched products run on the matrix cores (two kernels by size, 16-byte and scalar
    operand loads, ragged edges in M, N and K); fp64 runs on the vector ALUs and is tied to autograd
    by test_api_losses_and_gradients_vs_autograd.  Same inputs, same incoming gradients: px, py and
    the gradients with respect to lm and am must agree to the fp32 tolerance (1e-4 relative; the
    1e-5 absolute part is taken relative to the tensor's largest magnitude, the gradients being
    sums over up to 500 frames)."""
    from k2_amd import capi, native
    code = capi.RNNT_TYPES[rnnt_type]
    rng = np.random.default_rng(91)
    shapes = ((3, 37, 9, 50),        # small, rows not a multiple of four: split-K kernel, scalar loads
              (2, 70, 66, 132),      # split-K kernel, 16-byte loads, K = 132 = 8 x 16 + 4
              (16, 250, 50, 500),    # config 2: split-K kernel everywhere (the am gradient's K is short)
              (96, 203, 70, 130),    # LDS kernel everywhere, scalar loads, ragged in every axis
              (32, 500, 100, 500))   # config 3: LDS kernel, 16-byte loads
    for (B, T, S, C) in shapes:
        c = cases.rnnt_case(B + T, B, T, S, C, t_lo=max(T // 2, S), s_lo=S // 2, modified=rnnt_type != "regular")
        sym, bd = dev(c["symbols"], device), dev(c["boundary"], device)
        T1 = T + 1 if rnnt_type == "regular" else T
        gpx = rng.random((B, S, T1)).astype(np.float32)
        gpy = rng.random((B, S + 1, T)).astype(np.float32)
        res = {}
        for dt in (torch.float32, torch.float64):
            lm, am = dev(c["lm"], device).to(dt), dev(c["am"], device).to(dt)
            px, py, saved = native.logprobs_simple_forward(lm, am, sym, 0, code, bd)
            lm_g, am_g = native.logprobs_simple_backward(dev(gpx, device).to(dt), dev(gpy, device).to(dt), sym, bd,
                                                         saved, 0, code)
            res[dt] = [t.double().cpu().numpy() for t in (px, py, lm_g, am_g)]
        for name, a, b in zip(("px", "py", "lm_grad", "am_grad"), res[torch.float32], res[torch.float64]):
            scale = max(1.0, float(np.abs(b[np.isfinite(b)]).max()))
            with np.errstate(invalid="ignore"):
                ok = np.isclose(a, b, rtol=1e-4, atol=1e-5 * scale, equal_nan=True) | (a == b)
            assert ok.all(), (name, (B, T, S, C), int((~ok).sum()), a[~ok][:4], b[~ok][:4])


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_simple_gradients_with_often_repeated_symbols(device, rnnt_type):
    """Two non-blank classes and nine symbols: every symbol repeats more often than the am
    gradient's epilogue lists per column, so it takes its rescanning path; fp64 against torch
    autograd on the CPU, fp32 against fp64."""
    import k2_amd as k2
    B, T, S, C = 2, 13, 9, 3
    c = cases.rnnt_case(31, B, T, S, C, dtype=np.float64, t_lo=11, s_lo=7, modified=rnnt_type != "regular")
    assert max(np.bincount(c["symbols"][0])) > 4
    bd_cpu, sym_cpu = torch.from_numpy(c["boundary"]), torch.from_numpy(c["symbols"])
    lm_r = torch.from_numpy(c["lm"]).requires_grad_(True)
    am_r = torch.from_numpy(c["am"]).requires_grad_(True)
    px, py = torch_ref.logprobs_simple(lm_r, am_r, sym_cpu, 0, rnnt_type, bd_cpu)
    loss_r = -torch_ref.mi_scores(px, py, bd_cpu)
    loss_r.sum().backward()
    grads = {}
    for dt in (torch.float64, torch.float32):
        lm_g = dev(c["lm"], device).to(dt).requires_grad_(True)
        am_g = dev(c["am"], device).to(dt).requires_grad_(True)
        loss_g = k2.rnnt_loss_simple(lm_g, am_g, dev(c["symbols"], device), 0, dev(c["boundary"], device),
                                     rnnt_type=rnnt_type, reduction="none")
        loss_g.sum().backward()
        grads[dt] = (loss_g.detach().double().cpu().numpy(), lm_g.grad.double().cpu().numpy(),
                     am_g.grad.double().cpu().numpy())
    np.testing.assert_allclose(grads[torch.float64][0], loss_r.detach().numpy(), rtol=1e-10)
    np.testing.assert_allclose(grads[torch.float64][1], lm_r.grad.numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(grads[torch.float64][2], am_r.grad.numpy(), rtol=1e-8, atol=1e-10)
    for a, b in zip(grads[torch.float32], grads[torch.float64]):
        np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_loss_nodes_equal_the_builder_then_recursion_chain(device, rnnt_type):
    """The loss functions run builder + recursion as one autograd node and scale the gradients per
    sequence inside the builders' gradient kernels; chaining the public builder, the public
    recursion and torch's own products (what the reference does, k2/python/k2/rnnt_loss.py:
    300-338, 520-540, 1430-1468) must give the same bits: per-sequence losses, gradients under
    arbitrary per-sequence weights, with a delay penalty, and the returned occupation
    probabilities."""
    import k2_amd as k2
    from k2_amd.rnnt_loss import _delay_penalty
    B, T, S, C, R = 5, 37, 11, 23, 4
    c = cases.rnnt_case(41, B, T, S, C, t_lo=20, s_lo=5, modified=rnnt_type != "regular")
    sym = torch.from_numpy(c["symbols"]).to(device)
    bd = torch.from_numpy(c["boundary"]).to(device)
    w = torch.tensor([0.3, -1.7, 2.0, 0.0, 1.0], device=device)
    rng = np.random.default_rng(7)

    def leaf(shape):
        return torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to(device).requires_grad_(True)

    def compare(node, chain, leaves):
        for fn, out in ((node, []), (chain, [])):
            pass
        results = []
        for fn in (node, chain):
            for x in leaves:
                x.grad = None
            loss = fn()
            (loss * w).sum().backward()
            results.append((loss.detach().clone(), [x.grad.clone() for x in leaves]))
        assert torch.equal(results[0][0], results[1][0])
        for a, b in zip(results[0][1], results[1][1]):
            assert torch.equal(a, b)

    for penalty in (0.0, 0.01):
        lm, am = leaf((B, S + 1, C)), leaf((B, T, C))

        def chain_simple():
            px, py = k2.get_rnnt_logprobs(lm, am, sym, 0, rnnt_type, bd)
            if penalty:
                px = _delay_penalty(px, bd, rnnt_type, penalty)
            return -k2.mutual_information_recursion(px, py, bd)
        compare(lambda: k2.rnnt_loss_simple(lm, am, sym, 0, bd, rnnt_type, penalty, "none"),
                chain_simple, [lm, am])

        logits = leaf((B, T, S + 1, C))

        def chain_joint():
            px, py = k2.get_rnnt_logprobs_joint(logits, sym, 0, rnnt_type, bd)
            if penalty:
                px = _delay_penalty(px, bd, rnnt_type, penalty)
            return -k2.mutual_information_recursion(px, py, bd)
        compare(lambda: k2.rnnt_loss(logits, sym, 0, bd, rnnt_type, penalty, "none"), chain_joint, [logits])

        _, (gx, gy) = k2.rnnt_loss_simple(lm.detach(), am.detach(), sym, 0, bd, rnnt_type, 0.0, "sum",
                                          return_grad=True)
        ranges = k2.get_rnnt_prune_ranges(gx, gy, bd, R)
        pruned = leaf((B, T, R, C))
        for hat, builder in ((False, k2.get_rnnt_logprobs_pruned), (True, k2.get_hat_logprobs_pruned)):
            def chain_pruned():
                px, py = builder(pruned, sym, ranges, 0, bd, rnnt_type)
                if penalty:
                    px = _delay_penalty(px, bd, rnnt_type, penalty)
                return -k2.mutual_information_recursion(px, py, bd)
            compare(lambda: k2.rnnt_loss_pruned(pruned, sym, ranges, 0, bd, rnnt_type, penalty, "none", hat),
                    chain_pruned, [pruned])

    # return_grad hands out the same occupation probabilities as the recursion does
    lm, am = leaf((B, S + 1, C)), leaf((B, T, C))
    loss, (gx, gy) = k2.rnnt_loss_simple(lm, am, sym, 0, bd, rnnt_type, 0.0, "sum", return_grad=True)
    px, py = k2.get_rnnt_logprobs(lm, am, sym, 0, rnnt_type, bd)
    scores, (hx, hy) = k2.mutual_information_recursion(px, py, bd, return_grad=True)
    assert torch.equal(gx, hx) and torch.equal(gy, hy) and torch.equal(loss, -scores.sum())
    assert not gx.requires_grad and not gy.requires_grad
    # and without gradients nothing of the backward machinery runs
    with torch.no_grad():
        plain = k2.rnnt_loss_simple(lm, am, sym, 0, bd, rnnt_type, 0.0, "none")
    assert torch.equal(plain, -scores.detach()) and not plain.requires_grad


def test_random_shapes_through_the_api(device):
    """Random small shapes, lattice types, boundaries, dtypes and delay penalties through the
    k2-style API against the oracle: rnnt_loss_simple with gradients, get_rnnt_prune_ranges
    (bit-exact, from the oracle's gradients), rnnt_loss_pruned (and a finite gradient), rnnt_loss."""
    import k2_amd as k2

    def close(name, seed, got, want, tol):
        got = got.detach().cpu().numpy()
        ok = np.isclose(got, want, equal_nan=True, **tol) | (got == want)
        assert ok.all(), (name, seed, got[~ok][:4], want[~ok][:4])

    for seed in range(7000, 7080):
        rng = np.random.default_rng(seed)
        rt = TYPES[int(rng.integers(0, 3))]
        B, S, C = int(rng.integers(1, 6)), int(rng.integers(1, 40)), int(rng.integers(2, 60))
        t_min = S if rt != "regular" else 1
        T = int(rng.integers(t_min, S + 90))
        dtype = np.float32 if rng.random() < 0.8 else np.float64
        c = cases.rnnt_case(seed, B, T, S, C, dtype=dtype, t_lo=max(T // 2, t_min), s_lo=S // 2,
                            with_boundary=bool(rng.random() < 0.7), modified=(rt != "regular"))
        pen = float(rng.choice([0.0, 0.0, 0.01]))
        tol, bd, sym = TOL[np.dtype(dtype)], c["boundary"], c["symbols"]
        want, (gx_w, gy_w) = orn.rnnt_loss_simple(c["lm"], c["am"], sym, 0, bd, rt, pen, "none", True)
        got, (gx, gy) = k2.rnnt_loss_simple(dev(c["lm"], device), dev(c["am"], device), dev(sym, device), 0,
                                            dev(bd, device), rt, pen, "none", True)
        close("simple", seed, got, want, tol)
        if dtype == np.float64:
            close("px_grad", seed, gx, gx_w, tol)
            close("py_grad", seed, gy, gy_w, tol)
        R = int(rng.integers(2 if rt == "regular" else 1, S + 3))
        bd_full = np.tile(np.array([[0, 0, S, T]], np.int64), (B, 1)) if bd is None else bd
        ranges_w = orn.prune_ranges(gx_w, gy_w, bd_full, R)
        ranges = k2.get_rnnt_prune_ranges(dev(gx_w, device), dev(gy_w, device), dev(bd_full, device), R)
        assert np.array_equal(ranges.cpu().numpy(), ranges_w), ("ranges", seed)
        logits = rng.standard_normal((B, T, ranges_w.shape[2], C)).astype(dtype)
        want = orn.rnnt_loss_pruned(logits, sym, ranges_w, 0, bd, rt, pen, "none")
        lg = dev(logits, device).requires_grad_(True)
        got = k2.rnnt_loss_pruned(lg, dev(sym, device), dev(ranges_w, device), 0, dev(bd, device), rt, pen, "none")
        close("pruned", seed, got, want, tol)
        fin = np.isfinite(want)
        if fin.any():
            (got * dev(fin.astype(dtype), device)).sum().backward()
            # the closed form of the gradient from the oracle's occupation probabilities
            opx, opy = orn.logprobs_pruned(logits, sym, ranges_w, 0, bd, rt)
            opx = orn.apply_delay_penalty(opx, bd, rt, pen)
            (_, ogx, ogy), (a64, ogx64, ogy64) = _occupation_oracles(opx, opy, bd)
            g32, g64 = cf.pruned_logits_grad(logits, sym, ranges_w, 0, (ogx, ogx64), (ogy, ogy64),
                                             fin.astype(np.float64), rt)
            if dtype == np.float64:
                close("pruned gradient", seed, lg.grad, g64, tol)
            else:
                tolerance.close_f32(f"pruned gradient {seed}", lg.grad.cpu().numpy(), g32, g64, max_arbitrated=0.05)
        full = rng.standard_normal((B, T, S + 1, C)).astype(dtype)
        want = orn.rnnt_loss(full, sym, 0, bd, rt, pen, "none")
        got = k2.rnnt_loss(dev(full, device), dev(sym, device), 0, dev(bd, device), rt, pen, "none")
        close("joint", seed, got, want, tol)


# ---- gradients to the network outputs at the full BASELINE sizes ---------------------------------

def _occupation_oracles(px32, py32, boundary):
    """(ans, gx, gy) of the fp32 oracle and of the fp64 oracle on the same fp32 px / py."""
    a32, gx32, gy32 = omi.mi(px32, py32, boundary)
    a64, gx64, gy64 = omi.mi(px32.astype(np.float64), py32.astype(np.float64), boundary)
    return (a32, gx32, gy32), (a64, gx64, gy64)


def test_config2_network_gradients_full_size(device):
    """BASELINE config 2 (B=16, T=250, S=50, V=500, fp32): lm.grad and am.grad of
    rnnt_loss_simple against the fp64 closed form (tests/closed_forms.py).  First with the
    occupation probabilities the GPU itself returned, which isolates the builder's backward
    kernels (batched products, symbol and blank terms) at the stated tolerance; then end to end
    against the oracle's occupation probabilities, fp32 and fp64."""
    import k2_amd as k2
    B = 16
    c = cases.rnnt_case(2, B, 250, 50, 500, t_lo=150, s_lo=20)
    w = np.linspace(0.5, 1.5, B).astype(np.float32)
    lm = dev(c["lm"], device).requires_grad_(True)
    am = dev(c["am"], device).requires_grad_(True)
    loss, (gx, gy) = k2.rnnt_loss_simple(lm, am, dev(c["symbols"], device), 0, dev(c["boundary"], device),
                                         reduction="none", return_grad=True)
    (loss * dev(w, device)).sum().backward()
    gx, gy = gx.cpu().numpy(), gy.cpu().numpy()
    opx, opy = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, "regular", c["boundary"])
    (a32, gx32, gy32), (a64, gx64, gy64) = _occupation_oracles(opx, opy, c["boundary"])
    own, f32, f64 = cf.simple_grads(c["lm"], c["am"], c["symbols"], 0, (gx, gx32, gx64), (gy, gy32, gy64), w)
    for name, got, k in (("lm.grad", lm.grad.cpu().numpy(), 0), ("am.grad", am.grad.cpu().numpy(), 1)):
        np.testing.assert_allclose(got, own[k], rtol=1e-4, atol=1e-5, err_msg="c2 " + name)
        # signed sums of ~100 occupation probabilities: the arbitration's percentile is absolute
        three_way("c2 " + name, got, f32[k], f64[k], mode="absolute")


@pytest.mark.parametrize("few_symbols", [False, True])
def test_simple_gradients_where_the_am_gradient_takes_the_larger_tiles(device, few_symbols):
    """B=32, T=250, S=33, V=500: 1024 tiles of 64 x 64 in the am gradient, the fewest with which
    its product of K = S + 1 = 34 takes the LDS kernel (sixteen elements per thread in the
    epilogue's load rounds, ragged tiles in T and V, two groups of rows in the blank column's
    sums).  With the symbols as drawn (a column lists 0-3 positions) and with two classes only
    (every list overflows: the rescanning path).  lm.grad / am.grad against the fp64 closed form
    (tests/closed_forms.py) on the occupation probabilities that the GPU itself returned."""
    import k2_amd as k2
    B, T, S, C = 32, 250, 33, 500
    c = cases.rnnt_case(77, B, T, S, C, t_lo=150, s_lo=20)
    symbols = 1 + c["symbols"] % 2 if few_symbols else c["symbols"]
    w = np.linspace(0.5, 1.5, B).astype(np.float32)
    lm = dev(c["lm"], device).requires_grad_(True)
    am = dev(c["am"], device).requires_grad_(True)
    loss, (gx, gy) = k2.rnnt_loss_simple(lm, am, dev(symbols, device), 0, dev(c["boundary"], device),
                                         reduction="none", return_grad=True)
    (loss * dev(w, device)).sum().backward()
    gx, gy = gx.cpu().numpy(), gy.cpu().numpy()
    (want,) = cf.simple_grads(c["lm"], c["am"], symbols, 0, (gx,), (gy,), w)
    for name, got, k in (("lm.grad", lm.grad.cpu().numpy(), 0), ("am.grad", am.grad.cpu().numpy(), 1)):
        np.testing.assert_allclose(got, want[k], rtol=1e-4, atol=1e-5, err_msg=name)


def test_config3_logits_gradient_full_size(device):
    """BASELINE config 3 (B=32, T=500, S=100, V=500, s_range=5, fp32): the gradient of
    rnnt_loss_pruned w.r.t. the pruned logits [32,500,5,500] from the vectorised row kernel
    (C % 4 == 0, softmax blank term) against the fp64 closed form, isolated and end to end as in
    the config 2 test."""
    import k2_amd as k2
    B, T, S, C, R = 32, 500, 100, 500, 5
    c = cases.rnnt_case(3, B, T, S, C, t_lo=300, s_lo=50)
    _, (gx_s, gy_s) = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], reduction="none",
                                            return_grad=True)
    ranges = orn.prune_ranges(gx_s, gy_s, c["boundary"], R)
    logits = np.random.default_rng(33).standard_normal((B, T, R, C)).astype(np.float32)
    w = np.linspace(0.5, 1.5, B).astype(np.float32)
    sym_d, rng_d, bd_d = dev(c["symbols"], device), dev(ranges, device), dev(c["boundary"], device)
    lg = dev(logits, device).requires_grad_(True)
    loss = k2.rnnt_loss_pruned(lg, sym_d, rng_d, 0, bd_d, reduction="none")
    (loss * dev(w, device)).sum().backward()
    got = lg.grad.cpu().numpy()
    with torch.no_grad():
        px, py = k2.get_rnnt_logprobs_pruned(lg.detach(), sym_d, rng_d, 0, bd_d)
        _, (gx, gy) = k2.mutual_information_recursion(px, py, bd_d, return_grad=True)
    opx, opy = orn.logprobs_pruned(logits, c["symbols"], ranges, 0, c["boundary"], "regular")
    (a32, gx32, gy32), (a64, gx64, gy64) = _occupation_oracles(opx, opy, c["boundary"])
    three_way("c3 px_grad", gx.cpu().numpy(), gx32, gx64)
    three_way("c3 py_grad", gy.cpu().numpy(), gy32, gy64)
    own, f32, f64 = cf.pruned_logits_grad(logits, c["symbols"], ranges, 0, (gx.cpu().numpy(), gx32, gx64),
                                          (gy.cpu().numpy(), gy32, gy64), w)
    np.testing.assert_allclose(got, own, rtol=1e-4, atol=1e-5)
    three_way("c3 logits.grad", got, f32, f64)


def test_config5_logits_gradient_full_size(device):
    """BASELINE config 5 (B=8, T=300, S=75, V=500, fp32): the gradient of rnnt_loss w.r.t. the
    joiner logits [8,300,76,500], as in the config 3 test."""
    import k2_amd as k2
    B, T, S, C = 8, 300, 75, 500
    c = cases.rnnt_case(5, B, T, S, C, t_lo=200, s_lo=40)
    logits = np.random.default_rng(55).standard_normal((B, T, S + 1, C)).astype(np.float32)
    w = np.linspace(0.5, 1.5, B).astype(np.float32)
    sym_d, bd_d = dev(c["symbols"], device), dev(c["boundary"], device)
    lg = dev(logits, device).requires_grad_(True)
    loss = k2.rnnt_loss(lg, sym_d, 0, bd_d, reduction="none")
    (loss * dev(w, device)).sum().backward()
    got = lg.grad.cpu().numpy()
    with torch.no_grad():
        px, py = k2.get_rnnt_logprobs_joint(lg.detach(), sym_d, 0, boundary=bd_d)
        _, (gx, gy) = k2.mutual_information_recursion(px, py, bd_d, return_grad=True)
    opx, opy = orn.logprobs_joint(logits, c["symbols"], 0, "regular", c["boundary"])
    (a32, gx32, gy32), (a64, gx64, gy64) = _occupation_oracles(opx, opy, c["boundary"])
    three_way("c5 px_grad", gx.cpu().numpy(), gx32, gx64)
    three_way("c5 py_grad", gy.cpu().numpy(), gy32, gy64)
    own, f32, f64 = cf.joint_logits_grad(logits, c["symbols"], 0, (gx.cpu().numpy(), gx32, gx64),
                                         (gy.cpu().numpy(), gy32, gy64), w)
    np.testing.assert_allclose(got, own, rtol=1e-4, atol=1e-5)
    three_way("c5 logits.grad", got, f32, f64)


# ---- what the reference's own Python chain computes (tests/golden/rnnt_ref_fixtures.npz) ---------

def _fixtures():
    import os
    f = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rnnt_ref_fixtures.npz"))
    get = lambda name, key: f[f"{name}/{key}"] if f"{name}/{key}" in f.files else None
    return [str(n) for n in f["names"]], get


def test_reference_chain_fixtures(device, every=1):
    """Every function of the path on the inputs recorded with the reference's outputs: losses,
    occupation probabilities and network-output gradients within the fp32 tolerance, prune ranges
    (both rules) bit for bit from the reference's own gradients."""
    import k2_amd as k2
    names, get = _fixtures()
    tol = dict(rtol=1e-4, atol=1e-5)
    # (every: the host-build run of this body, tests/test_cpu_build_host_layer.py, takes every second chain)
    for name in [n for n in names if n.startswith("chain")][::every]:
        am, lm, sym, bd = (get(name, k) for k in ("am", "lm", "symbols", "boundary"))
        rt, dp, R = str(get(name, "rnnt_type")), float(get(name, "delay_penalty")), int(get(name, "s_range"))
        w = dev(get(name, "weights"), device)
        B, T, _ = am.shape
        S = sym.shape[1]
        sym_d, bd_d = dev(sym, device), dev(bd, device)
        lm_d = dev(lm, device).requires_grad_(True)
        am_d = dev(am, device).requires_grad_(True)
        loss, (gx, gy) = k2.rnnt_loss_simple(lm_d, am_d, sym_d, 0, bd_d, rt, dp, "none", True)
        (loss * w).sum().backward()
        np.testing.assert_allclose(loss.detach().cpu().numpy(), get(name, "simple_loss"), err_msg=name, **tol)
        np.testing.assert_allclose(gx.cpu().numpy(), get(name, "px_grad"), err_msg=name, **tol)
        np.testing.assert_allclose(gy.cpu().numpy(), get(name, "py_grad"), err_msg=name, **tol)
        np.testing.assert_allclose(lm_d.grad.cpu().numpy(), get(name, "lm_grad"), err_msg=name, **tol)
        np.testing.assert_allclose(am_d.grad.cpu().numpy(), get(name, "am_grad"), err_msg=name, **tol)
        bd_r = bd if bd is not None else np.tile(np.array([[0, 0, S, T]], np.int64), (B, 1))
        want = get(name, "ranges")
        ranges = k2.get_rnnt_prune_ranges(dev(get(name, "px_grad"), device), dev(get(name, "py_grad"), device),
                                          dev(bd_r, device), R)
        assert ranges.dtype == torch.int64 and tuple(ranges.shape) == want.shape, name
        assert np.array_equal(ranges.cpu().numpy(), want), name
        old = k2.get_rnnt_prune_ranges_deprecated(dev(get(name, "px_grad"), device),
                                                  dev(get(name, "py_grad"), device), dev(bd_r, device), R)
        assert np.array_equal(old.cpu().numpy(), get(name, "ranges_deprecated")), name
        am_p, lm_p = k2.do_rnnt_pruning(am_d.detach(), lm_d.detach(), ranges)
        logits = (am_p + lm_p).detach().requires_grad_(True)
        pruned = k2.rnnt_loss_pruned(logits, sym_d, ranges, 0, bd_d, rt, dp, "none")
        (pruned * w).sum().backward()
        np.testing.assert_allclose(pruned.detach().cpu().numpy(), get(name, "pruned_loss"), err_msg=name, **tol)
        np.testing.assert_allclose(logits.grad.cpu().numpy(), get(name, "pruned_logits_grad"), err_msg=name, **tol)
        hat = k2.rnnt_loss_pruned(logits.detach(), sym_d, ranges, 0, bd_d, rt, dp, "none", use_hat_loss=True)
        np.testing.assert_allclose(hat.cpu().numpy(), get(name, "hat_loss"), err_msg=name, **tol)
        full_logits = (am_d.detach().unsqueeze(2) + lm_d.detach().unsqueeze(1)).requires_grad_(True)
        full = k2.rnnt_loss(full_logits, sym_d, 0, bd_d, rt, dp, "none")
        (full * w).sum().backward()
        np.testing.assert_allclose(full.detach().cpu().numpy(), get(name, "full_loss"), err_msg=name, **tol)
        np.testing.assert_allclose(full_logits.grad.cpu().numpy(), get(name, "full_logits_grad"), err_msg=name, **tol)
        smoothed = k2.rnnt_loss_smoothed(lm_d.detach(), am_d.detach(), sym_d, 0, 0.2, 0.1, bd_d, rt, dp, "none")
        np.testing.assert_allclose(smoothed.cpu().numpy(), get(name, "smoothed_loss"), err_msg=name, **tol)


def test_reference_prune_ranges_on_ties_and_near_ties(device):
    """Gradients whose window sums tie exactly, or differ in the last bits so that the order of
    the additions decides the arg-max: the kernel must return the reference's integers."""
    import k2_amd as k2
    names, get = _fixtures()
    for name in names:
        if not name.startswith("ties"):
            continue
        gx, gy, bd, R = get(name, "px_grad"), get(name, "py_grad"), get(name, "boundary"), int(get(name, "s_range"))
        got = k2.get_rnnt_prune_ranges(dev(gx, device), dev(gy, device), dev(bd, device), R)
        assert np.array_equal(got.cpu().numpy(), get(name, "ranges")), name
        old = k2.get_rnnt_prune_ranges_deprecated(dev(gx, device), dev(gy, device), dev(bd, device), R)
        assert np.array_equal(old.cpu().numpy(), get(name, "ranges_deprecated")), name


def test_reference_logprobs_where_the_shifted_exponentials_underflow(device):
    """get_rnnt_logprobs on inputs scaled until exp(lm - max) * exp(am - max) underflows for some
    cells, where the reference's `+ tiny` decides the normaliser (k2/python/k2/rnnt_loss.py:172-184)."""
    import k2_amd as k2
    names, get = _fixtures()
    for name in names:
        if not name.startswith("floor"):
            continue
        px, py = k2.get_rnnt_logprobs(dev(get(name, "lm"), device), dev(get(name, "am"), device),
                                      dev(get(name, "symbols"), device), 0, str(get(name, "rnnt_type")),
                                      dev(get(name, "boundary"), device))
        want_px, want_py = get(name, "px"), get(name, "py")
        px, py = px.cpu().numpy(), py.cpu().numpy()
        assert np.array_equal(np.isfinite(px), np.isfinite(want_px)), name
        fin = np.isfinite(want_px)
        np.testing.assert_allclose(px[fin], want_px[fin], rtol=1e-4, atol=1e-5, err_msg=name)
        np.testing.assert_allclose(py, want_py, rtol=1e-4, atol=1e-5, err_msg=name)


def test_reference_joint_recursion_fixtures(device):
    """joint_mutual_information_recursion (k2/python/k2/mutual_information.py:314-423) on inputs
    recorded with the reference's own outputs: the split of the score over N = 1, 2, 3 pairs of
    inputs, and the gradient of a weighted sum of its elements to every input."""
    import k2_amd as k2
    names, get = _fixtures()
    tol = dict(rtol=1e-4, atol=1e-5)
    seen = 0
    for name in names:
        if not name.startswith("joint"):
            continue
        seen += 1
        N = int(get(name, "n"))
        bd = dev(get(name, "boundary"), device)
        pxs = [dev(get(name, f"px{i}"), device).requires_grad_(True) for i in range(N)]
        pys = [dev(get(name, f"py{i}"), device).requires_grad_(True) for i in range(N)]
        prods = k2.joint_mutual_information_recursion(pxs, pys, bd)
        assert tuple(prods.shape) == get(name, "prods").shape, name
        np.testing.assert_allclose(prods.detach().cpu().numpy(), get(name, "prods"), err_msg=name, **tol)
        w = get(name, "weights")
        (prods * dev(w, device)).sum().backward()
        # the gradients are weighted occupation probabilities: where an element misses the plain
        # bar against the reference's fp32 result the fp64 oracle arbitrates (tolerance.py)
        _, gx64, gy64 = omi.joint_mi([get(name, f"px{i}").astype(np.float64) for i in range(N)],
                                     [get(name, f"py{i}").astype(np.float64) for i in range(N)], get(name, "boundary"))
        lo = np.finfo(np.float32).min
        for i in range(N):
            for what, t, occ in (("px", pxs[i], gx64), ("py", pys[i], gy64)):
                want = get(name, f"{what}{i}_grad")
                want64 = np.where(get(name, f"{what}{i}") > lo, w[i].astype(np.float64)[:, None, None] * occ, 0.0)
                tolerance.close_f32(f"{name} {what}{i}.grad", t.grad.cpu().numpy(), want, want64, max_arbitrated=0.01)
    assert seen >= 6


def test_reference_smoothed_and_hat_gradient_fixtures(device):
    """The gradients of rnnt_loss_smoothed to lm / am and of rnnt_loss_pruned(use_hat_loss=True) to
    the logits (k2/python/k2/rnnt_loss.py:1471-1829, 992-1177), against what the reference's chain
    and torch's autograd gave on the same inputs."""
    import k2_amd as k2
    names, get = _fixtures()
    tol = dict(rtol=1e-4, atol=1e-5)
    seen = 0
    for name in names:
        if not name.startswith("grad"):
            continue
        seen += 1
        rt = str(get(name, "rnnt_type"))
        sym_d, bd_d, w = dev(get(name, "symbols"), device), dev(get(name, "boundary"), device), dev(get(name, "weights"), device)
        lm_d = dev(get(name, "lm"), device).requires_grad_(True)
        am_d = dev(get(name, "am"), device).requires_grad_(True)
        smoothed = k2.rnnt_loss_smoothed(lm_d, am_d, sym_d, 0, float(get(name, "lm_only_scale")),
                                         float(get(name, "am_only_scale")), bd_d, rt, 0.0, "none")
        (smoothed * w).sum().backward()
        np.testing.assert_allclose(smoothed.detach().cpu().numpy(), get(name, "smoothed_loss"), err_msg=name, **tol)
        np.testing.assert_allclose(lm_d.grad.cpu().numpy(), get(name, "smoothed_lm_grad"), err_msg=name, **tol)
        np.testing.assert_allclose(am_d.grad.cpu().numpy(), get(name, "smoothed_am_grad"), err_msg=name, **tol)
        logits = dev(get(name, "hat_logits"), device).requires_grad_(True)
        ranges = dev(get(name, "ranges"), device)
        hat = k2.rnnt_loss_pruned(logits, sym_d, ranges, 0, bd_d, rt, 0.0, "none", use_hat_loss=True)
        (hat * w).sum().backward()
        np.testing.assert_allclose(hat.detach().cpu().numpy(), get(name, "hat_loss"), err_msg=name, **tol)
        np.testing.assert_allclose(logits.grad.cpu().numpy(), get(name, "hat_logits_grad"), err_msg=name, **tol)
    assert seen >= 4
