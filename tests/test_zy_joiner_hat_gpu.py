"""rnnt_loss_pruned_joiner(use_hat_loss=True) on the GPU: the hybrid autoregressive transducer's
log-probs inside the fused joiner kernels (a template flag of joiner.hip's forward and backward
row kernels; the other instantiations are unchanged).

Not run on a GPU yet (its host-thread build is checked in tests/test_cpu_build_host_layer.py), so
the library refuses the variant unless K2AMD_JOINER_HAT=1 is set and this file is skipped without
it.  Collected after every test that has run on a GPU."""
import os

import numpy as np
import pytest
import torch

import test_joiner_gpu as tj
from oracle import mi as omi

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("K2AMD_JOINER_HAT", "0") != "1",
                                 reason="the HAT variant of the fused joiner is opt-in until it has run on a GPU: "
                                        "set K2AMD_JOINER_HAT=1")]


@pytest.mark.parametrize("precision", ["fp32", "bf16"])
@pytest.mark.parametrize("rnnt_type", tj.TYPES)
def test_forward_and_gradients(device, rnnt_type, precision):
    for seed, B, T, S, C, D, R, with_bias in tj.SMALL:
        c = tj.joiner_case(seed, B, T, S, C, D, R, rnnt_type, with_bias)
        logits, px, py = tj.chain_fp64(c, hat=True)
        gpx, gpy, norm = tj.run_forward(c, device, precision, hat=True)
        torch.cuda.synchronize()
        tag = f"hat {rnnt_type} {precision} seed {seed}"
        if precision == "fp32":
            tj.close(tag + " px", gpx.cpu().numpy(), px, 1e-4, 1e-5 / max(np.abs(px[np.isfinite(px)]).max(), 1e-30))
            tj.close(tag + " py", gpy.cpu().numpy(), py, 1e-4, 1e-5 / max(np.abs(py[np.isfinite(py)]).max(), 1e-30))
        else:
            fin = np.isfinite(px)
            assert np.array_equal(np.isfinite(gpx.cpu().numpy()), fin)
            assert np.abs(gpx.cpu().numpy()[fin] - px[fin]).max() < 5e-2
        if precision != "fp32":
            continue
        _, gx, gy = omi.mi(px, py, c["boundary"])
        gx, gy = gx.astype(np.float32), gy.astype(np.float32)
        scale = np.linspace(0.5, 1.5, B).astype(np.float32)
        want = tj.closed_form_grads(c, logits, gx, gy, scale, hat=True)
        got = tj.run_backward(c, device, precision, norm, gx, gy, scale, hat=True)
        for name, g, w in zip(("am_grad", "lm_grad", "weight_grad", "bias_grad"), got, want):
            if g is not None:
                tj.close(f"{tag} {name}", g, w, 1e-4, 1e-5)


def test_loss_against_the_three_steps(device):
    import k2_amd as k2
    c = tj.joiner_case(9, 4, 60, 15, 200, 256, 5, "regular", True)
    t = lambda k, grad=False: tj.dev(c[k], device).requires_grad_(grad)
    sym, bd, ranges = t("symbols"), t("boundary"), t("ranges")
    a1, l1, w1, b1 = t("am", True), t("lm", True), t("weight", True), t("bias", True)
    fused = k2.rnnt_loss_pruned_joiner(a1, l1, ranges, w1, b1, sym, 0, bd, reduction="sum", use_hat_loss=True)
    fused.backward()
    a2, l2, w2, b2 = t("am", True), t("lm", True), t("weight", True), t("bias", True)
    am_p, lm_p = k2.do_rnnt_pruning(a2, l2, ranges)
    logits = torch.nn.functional.linear(torch.tanh(am_p + lm_p), w2, b2)
    steps = k2.rnnt_loss_pruned(logits, sym, ranges, 0, bd, reduction="sum", use_hat_loss=True)
    steps.backward()
    np.testing.assert_allclose(fused.item(), steps.item(), rtol=1e-4)
    for name, x, y in (("am", a1, a2), ("lm", l1, l2), ("weight", w1, w2), ("bias", b1, b2)):
        scale = float(y.grad.abs().max())
        np.testing.assert_allclose(x.grad.cpu().numpy(), y.grad.cpu().numpy(), rtol=1e-3, atol=1e-4 * scale, err_msg=name)
