"""The smoothed builder's own kernels (K2AMD_SMOOTHED_KERNELS=1) on the GPU: px / py against the
oracle, losses and gradients against torch autograd over the three-distribution definition and
against the reference's recorded outputs, the torch-op implementation of the same functions on
the same device, and the two host layers against each other.

These kernels have not run on a GPU yet (their host-thread build is what
tests/test_cpu_build_smoothed.py checks), so the library leaves them switched off and this file
is skipped unless K2AMD_SMOOTHED_KERNELS=1 is set in the environment of the test run.  The file's
name puts it after every validated test and before the no-allocation one."""
import os

import numpy as np
import pytest
import torch

import cases
import torch_ref
from oracle import rnnt as orn

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("K2AMD_SMOOTHED_KERNELS", "0") != "1",
                                 reason="the smoothed builder's kernels are opt-in until they have run on a GPU: "
                                        "set K2AMD_SMOOTHED_KERNELS=1")]

TYPES = ["regular", "modified", "constrained"]


def dev(x, device):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(device)


def _loss_and_grads(k2, c, device, rnnt_type, scales, weights, use_boundary=True):
    lm = dev(c["lm"], device).requires_grad_(True)
    am = dev(c["am"], device).requires_grad_(True)
    bd = dev(c["boundary"], device) if use_boundary else None
    px, py = k2.get_rnnt_logprobs_smoothed(lm, am, dev(c["symbols"], device), 0, scales[0], scales[1], bd, rnnt_type)
    loss = k2.rnnt_loss_smoothed(lm, am, dev(c["symbols"], device), 0, scales[0], scales[1], bd, rnnt_type,
                                 reduction="none")
    (loss * dev(weights, device)).sum().backward()
    return [t.detach().cpu().numpy() for t in (px, py, loss, lm.grad, am.grad)]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_kernels_against_oracle_autograd_and_the_torch_ops(device, rnnt_type, dtype, monkeypatch):
    import k2_amd as k2
    from k2_amd import rnnt_loss
    B, T, S, C = 3, 37, 9, 70
    c = cases.rnnt_case(81, B, T, S, C, dtype=dtype, t_lo=20, s_lo=4, modified=rnnt_type != "regular")
    c["symbols"][:, 1] = c["symbols"][:, 0]
    c["symbols"][:, 3] = 0
    w = np.linspace(0.5, 1.5, B).astype(dtype)
    tol = dict(rtol=1e-10, atol=1e-10) if dtype == np.float64 else dict(rtol=1e-4, atol=1e-5)
    for scales, use_boundary in (((0.25, 0.1), True), ((0.0, 0.3), False)):
        assert rnnt_loss.smoothed_kernels_enabled()
        got = _loss_and_grads(k2, c, device, rnnt_type, scales, w, use_boundary)
        bd = c["boundary"] if use_boundary else None
        wpx, wpy = orn.logprobs_smoothed(c["lm"], c["am"], c["symbols"], 0, scales[0], scales[1], bd, rnnt_type)
        np.testing.assert_allclose(got[0], wpx, **tol)
        np.testing.assert_allclose(got[1], wpy, **tol)
        # autograd over the definition, in fp64 on the CPU
        lm_r = torch.from_numpy(c["lm"].astype(np.float64)).requires_grad_(True)
        am_r = torch.from_numpy(c["am"].astype(np.float64)).requires_grad_(True)
        bd_r = None if bd is None else torch.from_numpy(bd)
        rpx, rpy = torch_ref.logprobs_smoothed(lm_r, am_r, torch.from_numpy(c["symbols"]), 0, scales[0], scales[1],
                                               rnnt_type, bd_r)
        loss_r = -torch_ref.mi_scores(rpx, rpy, bd_r)
        (loss_r * torch.from_numpy(w.astype(np.float64))).sum().backward()
        np.testing.assert_allclose(got[2], loss_r.detach().numpy(), **tol)
        gtol = dict(rtol=1e-8, atol=1e-10) if dtype == np.float64 else dict(rtol=1e-3, atol=1e-5)
        np.testing.assert_allclose(got[3], lm_r.grad.numpy(), **gtol)
        np.testing.assert_allclose(got[4], am_r.grad.numpy(), **gtol)
        # the torch-op implementation on the same device
        monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "0")
        assert not rnnt_loss.smoothed_kernels_enabled()
        ops = _loss_and_grads(k2, c, device, rnnt_type, scales, w, use_boundary)
        monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1")
        for a, b in zip(got, ops):
            np.testing.assert_allclose(a, b, **gtol)


def test_reference_fixtures_of_the_smoothed_loss(device):
    import k2_amd as k2
    f = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rnnt_ref_fixtures.npz"))
    tol = dict(rtol=1e-4, atol=1e-5)
    seen = 0
    for name in (str(n) for n in f["names"]):
        if not name.startswith("grad"):
            continue
        seen += 1
        get = lambda key: f[f"{name}/{key}"]
        lm = dev(get("lm"), device).requires_grad_(True)
        am = dev(get("am"), device).requires_grad_(True)
        loss = k2.rnnt_loss_smoothed(lm, am, dev(get("symbols"), device), 0, float(get("lm_only_scale")),
                                     float(get("am_only_scale")), dev(get("boundary"), device),
                                     str(get("rnnt_type")), 0.0, "none")
        (loss * dev(get("weights"), device)).sum().backward()
        np.testing.assert_allclose(loss.detach().cpu().numpy(), get("smoothed_loss"), err_msg=name, **tol)
        np.testing.assert_allclose(lm.grad.cpu().numpy(), get("smoothed_lm_grad"), err_msg=name, **tol)
        np.testing.assert_allclose(am.grad.cpu().numpy(), get("smoothed_am_grad"), err_msg=name, **tol)
    assert seen >= 4


def test_config2_shape_and_the_two_host_layers(device):
    """BASELINE config 2's shape (B=16 T=250 S=50 V=500): the kernels against the torch ops, and
    the extension's host functions against the ctypes ones bit for bit (same C-ABI calls)."""
    import k2_amd as k2
    from k2_amd import capi, native
    B, T, S, C = 16, 250, 50, 500
    c = cases.rnnt_case(2, B, T, S, C, t_lo=150, s_lo=20)
    lm, am, sym, bd = (dev(c[k], device) for k in ("lm", "am", "symbols", "boundary"))
    px, py, saved = native.logprobs_smoothed_forward(lm, am, sym, 0, 0.25, 0.1, 0, bd)
    px2, py2, saved2 = capi.logprobs_smoothed_forward(lm, am, sym, 0, 0.25, 0.1, 0, bd)
    assert torch.equal(px, px2) and torch.equal(py, py2)
    for a, b in zip(saved, saved2):
        assert torch.equal(a, b)
    g = torch.Generator(device="cpu").manual_seed(5)
    gx, gy = torch.rand(px.shape, generator=g).to(device), torch.rand(py.shape, generator=g).to(device)
    scale = torch.linspace(0.5, 1.5, B, device=device)
    for seq in (None, scale):
        a = native.logprobs_smoothed_backward(gx, gy, sym, bd, saved, 0, 0.25, 0.1, 0, seq)
        b = capi.logprobs_smoothed_backward(gx, gy, sym, bd, saved2, 0, 0.25, 0.1, 0, seq)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        assert torch.isfinite(a[0]).all() and torch.isfinite(a[1]).all()
    wpx, wpy = orn.logprobs_smoothed(c["lm"], c["am"], c["symbols"], 0, 0.25, 0.1, c["boundary"], "regular")
    np.testing.assert_allclose(px.cpu().numpy(), wpx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(py.cpu().numpy(), wpy, rtol=1e-4, atol=1e-5)
