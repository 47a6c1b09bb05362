"""Parity of the fused pruned joiner (k2amd_rnnt_joiner_pruned_forward / _backward) against the
chain it replaces, do_rnnt_pruning -> tanh -> linear -> get_rnnt_logprobs_pruned
(k2/python/k2/rnnt_loss.py:913-954, 1180-1348), evaluated by the CPU oracle in fp64.

Tolerances.  precision "fp32": px / py within 1e-5 + 1e-4 |want| of the fp64 chain (the same -inf
pattern); gradients within 1e-4 |want| + 1e-5 max|want| of the fp64 closed form evaluated on the
occupation probabilities the entry point was given (sums over up to B*T*R rows: the absolute term
scales with the tensor).  precision "bf16" rounds the operands of the three matrix products to 8
significant bits; its bounds are stated where it is tested."""
import numpy as np
import pytest
import torch

import cases
import closed_forms as cf
from oracle import mi as omi
from oracle import rnnt as orn

pytestmark = pytest.mark.gpu

TYPES = ["regular", "modified", "constrained"]


def dev(x, device):
    return None if x is None else torch.from_numpy(np.ascontiguousarray(x)).to(device)


def joiner_case(seed, B, T, S, C, D, R, rnnt_type="regular", with_bias=True, t_lo=None, s_lo=None):
    """Projected encoder / decoder outputs, an output layer, and ranges as the pipeline makes them
    (from the occupation probabilities of a simple loss over random lm / am)."""
    modified = rnnt_type != "regular"
    c = cases.rnnt_case(seed, B, T, S, C, t_lo=t_lo if t_lo is not None else max(T // 2, S if modified else 1),
                        s_lo=s_lo if s_lo is not None else S // 2, modified=modified)
    _, (gx, gy) = orn.rnnt_loss_simple(c["lm"], c["am"], c["symbols"], 0, c["boundary"], rnnt_type=rnnt_type,
                                       reduction="none", return_grad=True)
    ranges = orn.prune_ranges(gx, gy, c["boundary"], R)
    rng = np.random.default_rng(seed + 1000)
    return dict(am=(0.8 * rng.standard_normal((B, T, D))).astype(np.float32),
                lm=(0.8 * rng.standard_normal((B, S + 1, D))).astype(np.float32),
                weight=(2.0 / np.sqrt(D) * rng.standard_normal((C, D))).astype(np.float32),
                bias=(0.5 * rng.standard_normal(C)).astype(np.float32) if with_bias else None,
                ranges=ranges, symbols=c["symbols"], boundary=c["boundary"], rnnt_type=rnnt_type)


def chain_fp64(c, hat=False):
    """logits, px, py of the chain in fp64 on the fp32 inputs."""
    f = lambda x: None if x is None else x.astype(np.float64)
    logits = orn.joiner_pruned_logits(f(c["am"]), f(c["lm"]), c["ranges"], f(c["weight"]), f(c["bias"]))
    builder = orn.hat_logprobs_pruned if hat else orn.logprobs_pruned
    px, py = builder(logits, c["symbols"], c["ranges"], 0, c["boundary"], c["rnnt_type"])
    return logits, px, py


def closed_form_grads(c, logits, gx, gy, scale, hat=False):
    """fp64 gradients of sum_b scale[b] * score_b w.r.t. am, lm, weight, bias, given the gradients
    gx, gy of the scores w.r.t. px, py: the closed form for the logits, then the chain rule through
    the linear layer, tanh and the gather."""
    B, T, R = c["ranges"].shape
    d_logits = -cf.pruned_logits_grad(logits, c["symbols"], c["ranges"], 0, gx.astype(np.float64),
                                      gy.astype(np.float64), scale.astype(np.float64), c["rnnt_type"], hat=hat)
    am, lm, w = c["am"].astype(np.float64), c["lm"].astype(np.float64), c["weight"].astype(np.float64)
    h = np.tanh(am[:, :, None, :] + lm[np.arange(B)[:, None, None], c["ranges"], :])
    d_w = np.einsum("btkc,btkd->cd", d_logits, h, optimize=True)
    d_b = d_logits.sum(axis=(0, 1, 2))
    d_pre = (d_logits @ w) * (1.0 - h * h)
    d_am = d_pre.sum(axis=2)
    d_lm = np.zeros_like(lm)
    np.add.at(d_lm, (np.arange(B)[:, None, None], c["ranges"]), d_pre)
    return d_am, d_lm, d_w, d_b


def close(name, got, want, rtol, atol_of_max):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert np.array_equal(np.isneginf(got), np.isneginf(want)), name
    fin = np.isfinite(want)
    assert np.isfinite(got[fin]).all(), name
    scale = max(np.abs(want[fin]).max(), 1e-30) if fin.any() else 1.0
    err = np.abs(got[fin] - want[fin])
    bound = rtol * np.abs(want[fin]) + atol_of_max * scale
    worst = float((err / bound).max()) if err.size else 0.0
    print(f"{name}: max err {err.max() if err.size else 0:.3e} (scale {scale:.3e}), worst err/bound {worst:.3f}")
    assert worst <= 1.0, (name, worst)


def run_forward(c, device, precision, hat=False):
    from k2_amd import capi
    return capi.joiner_pruned_forward(dev(c["am"], device), dev(c["lm"], device), dev(c["ranges"], device),
                                      dev(c["weight"], device), dev(c["bias"], device), dev(c["symbols"], device),
                                      0, dev(c["boundary"], device), capi.RNNT_TYPES[c["rnnt_type"]],
                                      capi.JOINER_PRECISIONS[precision], hat)


def run_backward(c, device, precision, norm, gx, gy, scale, hat=False):
    from k2_amd import capi
    out = capi.joiner_pruned_backward(dev(c["am"], device), dev(c["lm"], device), dev(c["ranges"], device),
                                      dev(c["weight"], device), dev(c["bias"], device), dev(c["symbols"], device),
                                      0, dev(c["boundary"], device), capi.RNNT_TYPES[c["rnnt_type"]], norm,
                                      dev(gx, device), dev(gy, device), dev(scale, device),
                                      capi.JOINER_PRECISIONS[precision], hat)
    torch.cuda.synchronize()
    return [None if t is None else t.cpu().numpy() for t in out]


SMALL = [  # seed, B, T, S, C, D, R, bias
    (1, 2, 23, 9, 37, 64, 3, True),     # one column tile, rows that do not fill a tile
    (2, 3, 40, 12, 130, 128, 5, False),  # two column tiles, the second nearly empty; no bias
    (3, 1, 70, 30, 500, 192, 4, True),   # C = 500 as in the configs; D not a multiple of 128
    (4, 4, 33, 6, 64, 320, 2, True),     # smallest window
    (5, 2, 50, 20, 257, 512, 7, True),   # largest D; R does not divide the tile rows
    (6, 1, 30, 12, 700, 64, 4, True),    # three tiles of 256 columns, smallest D
]


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_forward_small_shapes_fp32(device, rnnt_type):
    for seed, B, T, S, C, D, R, with_bias in SMALL:
        c = joiner_case(seed, B, T, S, C, D, R, rnnt_type, with_bias)
        logits, px, py = chain_fp64(c)
        gpx, gpy, norm = run_forward(c, device, "fp32")
        torch.cuda.synchronize()
        tag = f"{rnnt_type} seed {seed}"
        close(tag + " px", gpx.cpu().numpy(), px, 1e-4, 1e-5 / max(np.abs(px[np.isfinite(px)]).max(), 1e-30))
        close(tag + " py", gpy.cpu().numpy(), py, 1e-4, 1e-5 / max(np.abs(py[np.isfinite(py)]).max(), 1e-30))
        want_norm = np.log(np.exp(logits - logits.max(-1, keepdims=True)).sum(-1)) + logits.max(-1)
        np.testing.assert_allclose(norm.cpu().numpy(), want_norm, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_backward_in_several_passes(device, precision, monkeypatch):
    """The backward keeps the activations and the logits' gradients of the rows it has gone through
    in its workspace, up to a bound; beyond it, it goes through the rows in passes.  With the
    bound lowered (the library reads K2AMD_JOINER_PASS_ELEMS at every call) a small shape takes
    several passes: same gradients as in one pass, up to the order of the sums."""
    from k2_amd import capi
    seed, B, T, S, C, D, R, with_bias = 7, 3, 57, 14, 300, 128, 4, True
    c = joiner_case(seed, B, T, S, C, D, R, "regular", with_bias)
    logits, px, py = chain_fp64(c)
    _, gx, gy = omi.mi(px, py, c["boundary"])
    gx, gy = gx.astype(np.float32), gy.astype(np.float32)
    scale = np.linspace(0.5, 1.5, B).astype(np.float32)
    _, _, norm = run_forward(c, device, precision)
    args = (B, S, T, R, C, D, capi.JOINER_PRECISIONS[precision])
    whole = capi.lib().k2amd_rnnt_joiner_pruned_workspace_bytes(*args)
    one = run_backward(c, device, precision, norm, gx, gy, scale)
    rows_tile = 64 if precision == "bf16" else 32
    monkeypatch.setenv("K2AMD_JOINER_PASS_ELEMS", str(2 * rows_tile * (D + 512)))  # two tiles a pass
    assert capi.lib().k2amd_rnnt_joiner_pruned_workspace_bytes(*args) < whole
    several = run_backward(c, device, precision, norm, gx, gy, scale)
    monkeypatch.delenv("K2AMD_JOINER_PASS_ELEMS")
    for name, g, w in zip(("am_grad", "lm_grad", "weight_grad", "bias_grad"), several, one):
        close(f"{precision} {name}", g, w, 1e-5, 1e-6)
    if precision == "fp32":
        for name, g, w in zip(("am_grad", "lm_grad", "weight_grad", "bias_grad"), several,
                              closed_form_grads(c, logits, gx, gy, scale)):
            close(name, g, w, 1e-4, 1e-5)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_backward_small_shapes_fp32(device, rnnt_type):
    for seed, B, T, S, C, D, R, with_bias in SMALL:
        c = joiner_case(seed, B, T, S, C, D, R, rnnt_type, with_bias)
        logits, px, py = chain_fp64(c)
        _, gx, gy = omi.mi(px, py, c["boundary"])
        gx, gy = gx.astype(np.float32), gy.astype(np.float32)
        scale = np.linspace(0.5, 1.5, B).astype(np.float32)
        _, _, norm = run_forward(c, device, "fp32")
        d_am, d_lm, d_w, d_b = run_backward(c, device, "fp32", norm, gx, gy, scale)
        w_am, w_lm, w_w, w_b = closed_form_grads(c, logits, gx, gy, scale)
        tag = f"{rnnt_type} seed {seed}"
        close(tag + " am_grad", d_am, w_am, 1e-4, 1e-5)
        close(tag + " lm_grad", d_lm, w_lm, 1e-4, 1e-5)
        close(tag + " weight_grad", d_w, w_w, 1e-4, 1e-5)
        if with_bias:
            close(tag + " bias_grad", d_b, w_b, 1e-4, 1e-5)
        else:
            assert d_b is None


def test_bf16_small_shapes(device):
    """bfloat16 operands (8 significant bits) for the three products, fp32 sums: the log-probs move
    by a few 1e-2 at most and the gradients by a few per cent of their largest element; the
    bounds below are what that rounding allows at these sizes, not a parity claim."""
    for seed, B, T, S, C, D, R, with_bias in SMALL:
        c = joiner_case(seed, B, T, S, C, D, R, "regular", with_bias)
        logits, px, py = chain_fp64(c)
        gpx, gpy, norm = run_forward(c, device, "bf16")
        torch.cuda.synchronize()
        close(f"bf16 seed {seed} px", gpx.cpu().numpy(), px, 0.0, 0.05 / max(np.abs(px[np.isfinite(px)]).max(), 1e-30))
        close(f"bf16 seed {seed} py", gpy.cpu().numpy(), py, 0.0, 0.05 / max(np.abs(py[np.isfinite(py)]).max(), 1e-30))
        _, gx, gy = omi.mi(px, py, c["boundary"])
        gx, gy = gx.astype(np.float32), gy.astype(np.float32)
        scale = np.ones(B, np.float32)
        got = run_backward(c, device, "bf16", norm, gx, gy, scale)
        want = closed_form_grads(c, logits, gx, gy, scale)
        for name, g, w in zip(("am_grad", "lm_grad", "weight_grad", "bias_grad"), got, want):
            if g is not None:
                close(f"bf16 seed {seed} {name}", g, w, 0.0, 0.03)


def test_refusals(device):
    """Shapes the kernels are not built for, wrong dtypes and shapes: RuntimeError, nothing launched."""
    from k2_amd import capi
    c = joiner_case(1, 2, 23, 9, 37, 64, 3)
    args = lambda **kw: [dev(kw.get(k, c[k]), device) for k in ("am", "lm", "ranges", "weight", "bias", "symbols")]
    with pytest.raises(RuntimeError):   # D not a multiple of 64
        capi.joiner_pruned_forward(*args(am=c["am"][:, :, :48], lm=c["lm"][:, :, :48], weight=c["weight"][:, :48]),
                                   0, None, 0)
    with pytest.raises(RuntimeError):   # fp64
        capi.joiner_pruned_forward(*[t.double() if t.is_floating_point() else t for t in args()], 0, None, 0)
    with pytest.raises(RuntimeError):   # bias of the wrong length
        capi.joiner_pruned_forward(*args(bias=c["bias"][:-1]), 0, None, 0)
    with pytest.raises(RuntimeError):   # termination symbol outside the vocabulary
        capi.joiner_pruned_forward(*args(), 37, None, 0)


def test_config3_shape_through_the_api(device):
    """BASELINE config 3's shape (B=32, T=500, S=100, V=500, s_range=5) with a joiner of D=512,
    through k2_amd.rnnt_loss_pruned_joiner and autograd: the loss per utterance against the fp64
    chain + fp64 recursion; am.grad, lm.grad, weight.grad, bias.grad against the fp64 closed form on
    the occupation probabilities the device's own recursion returned (which isolates the joiner's
    three products from the recursion's fp32 noise, bounded elsewhere)."""
    import k2_amd as k2
    B, T, S, C, D, R = 32, 500, 100, 500, 512, 5
    c = joiner_case(3, B, T, S, C, D, R, "regular", True, t_lo=300, s_lo=50)
    logits, px, py = chain_fp64(c)
    scores64, _, _ = omi.mi(px, py, c["boundary"])
    w = np.linspace(0.5, 1.5, B).astype(np.float32)
    t = {k: dev(c[k], device) for k in ("am", "lm", "weight", "bias", "ranges", "symbols", "boundary")}
    for k in ("am", "lm", "weight", "bias"):
        t[k].requires_grad_(True)
    loss = k2.rnnt_loss_pruned_joiner(t["am"], t["lm"], t["ranges"], t["weight"], t["bias"], t["symbols"], 0,
                                      t["boundary"], reduction="none")
    (loss * dev(w, device)).sum().backward()
    np.testing.assert_allclose(loss.detach().cpu().numpy(), -scores64, rtol=1e-4, atol=1e-4)
    with torch.no_grad():
        gpx, gpy, _ = run_forward(c, device, "fp32")
        _, (gx, gy) = k2.mutual_information_recursion(gpx, gpy, t["boundary"], return_grad=True)
    close("c3 px", gpx.cpu().numpy(), px, 1e-4, 1e-5 / np.abs(px[np.isfinite(px)]).max())
    close("c3 py", gpy.cpu().numpy(), py, 1e-4, 1e-5 / np.abs(py[np.isfinite(py)]).max())
    want = closed_form_grads(c, logits, gx.cpu().numpy(), gy.cpu().numpy(), -w)  # loss = -score
    for name, key, wv in zip(("am.grad", "lm.grad", "weight.grad", "bias.grad"), ("am", "lm", "weight", "bias"), want):
        close("c3 " + name, t[key].grad.cpu().numpy(), wv, 1e-4, 1e-5)


def test_config3_shape_bf16(device):
    """The same through the bfloat16 products: loss within 1e-3 relative of the fp64 chain."""
    import k2_amd as k2
    B, T, S, C, D, R = 32, 500, 100, 500, 512, 5
    c = joiner_case(3, B, T, S, C, D, R, "regular", True, t_lo=300, s_lo=50)
    _, px, py = chain_fp64(c)
    scores64, _, _ = omi.mi(px, py, c["boundary"])
    t = {k: dev(c[k], device) for k in ("am", "lm", "weight", "bias", "ranges", "symbols", "boundary")}
    for k in ("am", "lm", "weight", "bias"):
        t[k].requires_grad_(True)
    loss = k2.rnnt_loss_pruned_joiner(t["am"], t["lm"], t["ranges"], t["weight"], t["bias"], t["symbols"], 0,
                                      t["boundary"], reduction="none", precision="bf16")
    loss.sum().backward()
    got = loss.detach().cpu().numpy()
    print("bf16 c3 loss: max relative error", np.abs(got + scores64).max() / np.abs(scores64).max())
    np.testing.assert_allclose(got, -scores64, rtol=1e-3)
    for k in ("am", "lm", "weight", "bias"):
        assert torch.isfinite(t[k].grad).all()
