"""The Python host layer (k2_amd/capi.py's wrappers, k2_amd/rnnt_loss.py's autograd Functions)
run on CPU tensors against the host build of the kernels (tests/cpu_kernels.py).

The product never does this: it takes device tensors and fails without the GPU library.  Here a
fixture swaps, for the duration of a test, the library handle for the host build and the three
places where the wrappers touch the device (the device check, the stream, the device guard), so
that the very code that marshals arguments on the GPU box is exercised without one: argument
order and count of every C-ABI call, the buffers it allocates and their shapes, what is saved for
the backward, and the chaining of the autograd Functions.  Gradients are compared with torch
autograd over the plain-torch definitions (tests/torch_ref.py)."""
import contextlib
import os
import types

import numpy as np
import pytest
import torch

import cases
import cpu_kernels as ck
import torch_ref
from oracle import mi as omi
from oracle import rnnt as orn

TYPES = ["regular", "modified", "constrained"]
# what takes a quarter of a minute and more on eight cores runs with K2AMD_SLOW_CPU_TESTS=1 only
slow = pytest.mark.skipif(os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1",
                          reason="slow on the host: run with K2AMD_SLOW_CPU_TESTS=1")


@pytest.fixture
def host_on_cpu(monkeypatch):
    from k2_amd import capi, native
    cpu_lib = ck.lib()
    monkeypatch.setattr(capi, "lib", lambda: cpu_lib)
    monkeypatch.setattr(capi, "_on_device", lambda t: True)
    monkeypatch.setattr(capi, "stream_ptr", lambda device: None)
    monkeypatch.setattr(torch.cuda, "device", lambda device: contextlib.nullcontext())
    # (for the workspace cache of the pipelined kernels, which is kept per device and stream)
    monkeypatch.setattr(torch.cuda, "current_stream", lambda device=None: types.SimpleNamespace(cuda_stream=0))
    monkeypatch.setattr(torch.cuda, "current_device", lambda: 0)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda device=None: None)
    monkeypatch.setattr(capi, "_workspaces", {})
    monkeypatch.setattr(native, "_ext", None)              # the ctypes host: same C-ABI calls as the extension's
    monkeypatch.setattr(native, "_require_device", lambda t: None)
    return capi


def _weighted(px, py, seed):
    """A scalar function of the lattice's log-probs with fixed random weights (zero where px is
    -inf: the last column of a regular lattice and the boundary cut)."""
    g = torch.Generator().manual_seed(seed)
    wx = torch.rand(px.shape, generator=g, dtype=torch.float64).to(px.dtype)
    wy = torch.rand(py.shape, generator=g, dtype=torch.float64).to(py.dtype)
    finite = torch.isfinite(px)
    return (torch.where(finite, px, torch.zeros_like(px)) * wx).sum() + (py * wy).sum()


def _case(seed, B, T, S, C, rnnt_type, dtype=np.float64):
    c = cases.rnnt_case(seed, B, T, S, C, dtype=dtype, t_lo=max(S, T - 3), s_lo=max(1, S - 2),
                        modified=rnnt_type != "regular")
    c["symbols"][:, 1] = c["symbols"][:, 0]
    return c


def _t(c, *keys):
    return [None if c[k] is None else torch.from_numpy(c[k]) for k in keys]


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_simple_and_smoothed_builders_through_autograd(host_on_cpu, rnnt_type, monkeypatch):
    import k2_amd as k2
    c = _case(801, 3, 11, 6, 70, rnnt_type)
    sym, bd = _t(c, "symbols", "boundary")
    for smoothed in (False, True):
        for kernels in ((False, True) if smoothed else (False,)):
            monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1" if kernels else "0")
            lm, am = (x.requires_grad_(True) for x in _t(c, "lm", "am"))
            lm_r, am_r = (x.requires_grad_(True) for x in _t(c, "lm", "am"))
            if smoothed:
                px, py = k2.get_rnnt_logprobs_smoothed(lm, am, sym, 0, 0.25, 0.1, boundary=bd, rnnt_type=rnnt_type)
                rpx, rpy = torch_ref.logprobs_smoothed(lm_r, am_r, sym, 0, 0.25, 0.1, rnnt_type, bd)
            else:
                px, py = k2.get_rnnt_logprobs(lm, am, sym, 0, rnnt_type=rnnt_type, boundary=bd)
                rpx, rpy = torch_ref.logprobs_simple(lm_r, am_r, sym, 0, rnnt_type, bd)
            np.testing.assert_allclose(px.detach().numpy(), rpx.detach().numpy(), rtol=1e-10, atol=1e-10)
            np.testing.assert_allclose(py.detach().numpy(), rpy.detach().numpy(), rtol=1e-10, atol=1e-10)
            _weighted(px, py, 5).backward()
            _weighted(rpx, rpy, 5).backward()
            np.testing.assert_allclose(lm.grad.numpy(), lm_r.grad.numpy(), rtol=1e-8, atol=1e-10)
            np.testing.assert_allclose(am.grad.numpy(), am_r.grad.numpy(), rtol=1e-8, atol=1e-10)


def test_smoothed_kernels_with_float32_and_a_per_sequence_scale(host_on_cpu, monkeypatch):
    """The smoothed wrappers directly, fp32, with seq_scale (the loss functions' way of passing
    the gradient that reaches each score)."""
    capi = host_on_cpu
    c = _case(802, 3, 13, 5, 33, "regular", np.float32)
    lm, am, sym, bd = _t(c, "lm", "am", "symbols", "boundary")
    assert capi.smoothed_supported(lm, am)
    px, py, saved = capi.logprobs_smoothed_forward(lm, am, sym, 0, 0.25, 0.1, 0, bd)
    wpx, wpy = orn.logprobs_smoothed(c["lm"], c["am"], c["symbols"], 0, 0.25, 0.1, c["boundary"], "regular")
    np.testing.assert_allclose(px.numpy(), wpx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(py.numpy(), wpy, rtol=1e-4, atol=1e-5)
    _, gx, gy = omi.mi(wpx.astype(np.float64), wpy.astype(np.float64), c["boundary"])
    scale = torch.linspace(0.5, 1.5, 3)
    lm_g, am_g = capi.logprobs_smoothed_backward(torch.from_numpy(gx.astype(np.float32)),
                                                 torch.from_numpy(gy.astype(np.float32)), sym, bd, saved, 0, 0.25,
                                                 0.1, 0, scale)
    import closed_forms as cf
    want_lm, want_am = cf.smoothed_grads(c["lm"], c["am"], c["symbols"], 0, 0.25, 0.1, gx, gy, -scale.numpy(),
                                         "regular")
    np.testing.assert_allclose(lm_g.numpy(), want_lm, rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(am_g.numpy(), want_am, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_joint_and_pruned_builders_through_autograd(host_on_cpu, rnnt_type):
    import k2_amd as k2
    B, T, S, C, R = 2, 9, 5, 37, 3
    c = _case(803, B, T, S, C, rnnt_type)
    sym, bd = _t(c, "symbols", "boundary")
    rng = np.random.default_rng(804)
    logits = torch.from_numpy(rng.standard_normal((B, T, S + 1, C))).requires_grad_(True)
    ref = logits.detach().clone().requires_grad_(True)
    px, py = k2.get_rnnt_logprobs_joint(logits, sym, 0, rnnt_type=rnnt_type, boundary=bd)
    rpx, rpy = torch_ref.logprobs_from_logits(ref, sym, 0, rnnt_type, bd)
    np.testing.assert_allclose(px.detach().numpy(), rpx.detach().numpy(), rtol=1e-10, atol=1e-10)
    _weighted(px, py, 6).backward()
    _weighted(rpx, rpy, 6).backward()
    np.testing.assert_allclose(logits.grad.numpy(), ref.grad.numpy(), rtol=1e-8, atol=1e-10)

    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    start[:, 0], start[:, -2:] = 0, S - R + 1
    ranges = torch.from_numpy((np.maximum.accumulate(start, axis=1)[:, :, None] + np.arange(R)).astype(np.int64))
    for hat in (False, True):
        logits = torch.from_numpy(rng.standard_normal((B, T, R, C))).requires_grad_(True)
        ref = logits.detach().clone().requires_grad_(True)
        builder = k2.get_hat_logprobs_pruned if hat else k2.get_rnnt_logprobs_pruned
        px, py = builder(logits, sym, ranges, 0, boundary=bd, rnnt_type=rnnt_type)
        rpx, rpy = torch_ref.logprobs_pruned(ref, sym, ranges, 0, bd, rnnt_type, hat=hat)
        finite = torch.isfinite(rpx)
        assert torch.equal(torch.isfinite(px), finite)
        np.testing.assert_allclose(px.detach()[finite].numpy(), rpx.detach()[finite].numpy(), rtol=1e-10, atol=1e-10)
        # py outside the band is -inf on both sides: weigh the band only
        band = torch.isfinite(rpy)
        assert torch.equal(torch.isfinite(py), band)
        g = torch.Generator().manual_seed(7)
        wx, wy = torch.rand(px.shape, generator=g, dtype=torch.float64), torch.rand(py.shape, generator=g, dtype=torch.float64)
        zero = torch.zeros((), dtype=torch.float64)
        for a, b in ((px, py), (rpx, rpy)):
            (torch.where(finite, a, zero) * wx).sum().add((torch.where(band, b, zero) * wy).sum()).backward()
        np.testing.assert_allclose(logits.grad.numpy(), ref.grad.numpy(), rtol=1e-8, atol=1e-10)


def test_prune_ranges_pruning_and_lattice(host_on_cpu):
    import k2_amd as k2
    capi = host_on_cpu
    B, T, S, C, R = 3, 17, 8, 12, 4
    c = _case(805, B, T, S, C, "regular", np.float32)
    px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, "regular", c["boundary"])
    _, gx, gy = omi.mi(px, py, c["boundary"])
    bd = torch.from_numpy(c["boundary"])
    ranges = k2.get_rnnt_prune_ranges(torch.from_numpy(gx), torch.from_numpy(gy), bd, R)
    want = orn.prune_ranges(gx, gy, c["boundary"], R)
    assert np.array_equal(ranges.numpy(), want)

    D = 24
    rng = np.random.default_rng(806)
    am = torch.from_numpy(rng.standard_normal((B, T, D)).astype(np.float32)).requires_grad_(True)
    lm = torch.from_numpy(rng.standard_normal((B, S + 1, D)).astype(np.float32)).requires_grad_(True)
    am_p, lm_p = k2.do_rnnt_pruning(am, lm, ranges)
    want_lm = torch.gather(lm.detach().unsqueeze(1).expand(B, T, S + 1, D), 2,
                           ranges.reshape(B, T, R, 1).expand(B, T, R, D))
    assert torch.equal(lm_p.detach(), want_lm)
    assert torch.equal(am_p.detach(), am.detach().unsqueeze(2).expand(B, T, R, D))
    w = torch.from_numpy(rng.standard_normal((B, T, R, D)).astype(np.float32))
    (lm_p * w).sum().backward()
    want_g = torch.zeros(B, S + 1, D).index_put_(
        (torch.arange(B).reshape(B, 1, 1).expand(B, T, R), ranges), w, accumulate=True)
    np.testing.assert_allclose(lm.grad.numpy(), want_g.numpy(), rtol=1e-5, atol=1e-5)

    from oracle import lattice as olat
    logits = rng.standard_normal((B, T, ranges.shape[2], C)).astype(np.float32)
    frames = c["boundary"][:, 3].astype(np.int32)
    state_splits, arc_splits, arcs, arc_map = capi.pruned_ranges_to_lattice(
        ranges.to(torch.int32), torch.from_numpy(frames), torch.from_numpy(c["symbols"]), torch.from_numpy(logits))
    w_state, w_arc, w_arcs, w_scores, w_map = olat.pruned_ranges_to_lattice(
        ranges.numpy().astype(np.int32), frames, c["symbols"], logits)
    assert np.array_equal(state_splits.numpy(), w_state) and np.array_equal(arc_splits.numpy(), w_arc)
    assert np.array_equal(arcs.numpy()[:, :3], w_arcs) and np.array_equal(arc_map.numpy(), w_map)
    assert np.array_equal(arcs.numpy()[:, 3].copy().view(np.float32), w_scores.astype(np.float32))


def test_joint_products_wrapper(host_on_cpu):
    capi = host_on_cpu
    rng = np.random.default_rng(807)
    N, B, S, T = 3, 2, 4, 7
    pxs = [torch.from_numpy(-rng.uniform(0, 3, (B, S, T + 1))) for _ in range(N)]
    pys = [torch.from_numpy(-rng.uniform(0, 3, (B, S + 1, T))) for _ in range(N)]
    gx, gy = torch.from_numpy(rng.uniform(0, 1, (B, S, T + 1))), torch.from_numpy(rng.uniform(0, 1, (B, S + 1, T)))
    prods = capi.mi_joint_products(pxs, pys, gx, gy)
    want = torch.stack([(x * gx).sum(dim=(1, 2)) + (y * gy).sum(dim=(1, 2)) for x, y in zip(pxs, pys)])
    np.testing.assert_allclose(prods.numpy(), want.numpy(), rtol=1e-12)


# ---- the whole Python API on the host: the GPU tests' own bodies, with device = cpu --------------
# mutual_information_recursion and every loss function run end to end, on the kernels that the
# library would take on the device for the same shape and dtype.

def _gpu_test(name):
    import test_rnnt_gpu
    return getattr(test_rnnt_gpu, name)


@pytest.mark.parametrize("modified", [False, True])
def test_deprecated_prune_ranges_through_the_api(host_on_cpu, modified):
    _gpu_test("test_deprecated_prune_ranges_matches_oracle")(torch.device("cpu"), modified)


@pytest.mark.parametrize("name", ["test_reference_chain_fixtures",
                                  "test_reference_prune_ranges_on_ties_and_near_ties",
                                  "test_reference_logprobs_where_the_shifted_exponentials_underflow",
                                  pytest.param("test_reference_joint_recursion_fixtures", marks=slow),
                                  "test_reference_smoothed_and_hat_gradient_fixtures"])
def test_reference_fixtures_through_the_api(host_on_cpu, name, monkeypatch):
    """Everything recorded from the reference's own Python chain (tests/golden/rnnt_ref_fixtures.npz)
    through k2_amd's API on CPU tensors: losses, occupation probabilities, gradients to the network
    outputs, prune ranges bit for bit; the smoothed loss with the library's kernels for
    its marginal terms."""
    if "chain" in name:  # every fourth chain (every second with the slow switch), the smoothed loss in it with the library's kernels
        monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1")
        _gpu_test(name)(torch.device("cpu"), every=2 if os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") == "1" else 4)
        return
    if "smoothed" in name:  # (with torch ops for the marginal terms this test runs on the GPU)
        monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1")
    _gpu_test(name)(torch.device("cpu"))


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_smoothed_loss_with_the_kernels(host_on_cpu, rnnt_type, monkeypatch):
    """rnnt_loss_smoothed end to end (values against the oracle, gradients against autograd over the
    definition, scales (0, 0) == rnnt_loss_simple, invariance to per-frame constants) with the
    marginal terms in the library's kernels."""
    monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1")
    _gpu_test("test_smoothed_loss_values_gradients_and_identities")(torch.device("cpu"), rnnt_type)


@pytest.mark.parametrize("name", [pytest.param("test_rnnt_loss_gradient", marks=slow), "test_rnnt_loss_empty_reference",
                                  "test_mutual_information_against_itself_and_finite_differences"])
def test_reference_scenarios_through_the_api(host_on_cpu, name):
    """Scenarios of the reference's own tests (rnnt_loss_test.py, mutual_information_test.py) as
    tests/test_reference_scenarios_gpu.py restates them, at the sizes the host build can afford."""
    import test_reference_scenarios_gpu
    getattr(test_reference_scenarios_gpu, name)(torch.device("cpu"))


@slow
def test_joint_recursion_split_through_the_api(host_on_cpu):
    import test_mi_gpu
    test_mi_gpu.test_joint_recursion_split_matches_the_torch_chain(torch.device("cpu"), torch.float32)


def test_no_allocation_entry_point(host_on_cpu):
    """k2amd_mi_forward_noalloc gives what k2amd_mi_forward gives (the same kernels; the scratch of
    the pipelined ones is the library's static array), is not refused for that array's size where
    the shape is served without scratch, and its status call answers.  (Two calls in a row on
    shapes that the pipelined kernels serve: tests/test_cpu_build_pipelined.py.)"""
    capi = host_on_cpu
    lib = capi.lib()
    c = cases.mi_case(901, dtype=np.float32, max_B=3, max_S=20, max_T=40)
    px, py = torch.from_numpy(c["px"]), torch.from_numpy(c["py"])
    bd = None if c["boundary"] is None else torch.from_numpy(c["boundary"])
    B, S, T = c["B"], c["S"], c["T"]
    p1, p2 = torch.empty(B, S + 1, T + 1), torch.empty(B, S + 1, T + 1)
    want = capi.mi_forward(px, py, bd, p1)
    got = capi.mi_forward_noalloc(px, py, bd, p2, torch.empty(B))
    assert torch.equal(got, want)
    ans, _ = omi.mi_forward(c["px"], c["py"], c["boundary"])
    np.testing.assert_allclose(got.numpy(), ans, rtol=1e-4, atol=1e-5)
    # a lattice of 2 GiB and more: not refused for scratch, turned down for its null pointers
    assert lib.k2amd_mi_forward_noalloc(None, None, None, None, None, 4096, 200, 1000, 1, 0, None) == 1
    assert lib.k2amd_mi_forward_noalloc(None, None, None, None, None, 0, 3, 3, 0, 0, None) == 0
    assert lib.k2amd_mi_noalloc_status(None) == 0


@pytest.mark.parametrize("modified", [False, True])
def test_fp64_pipelined_kernels(host_on_cpu, modified):
    """mi_wave.hip (one wavefront per chunk of 64 rows, chunks of a sequence handing their border
    over through words in the workspace, lane shifts by DPP) against the fp64 oracle: lattices of
    one to three chunks, boundaries, both lattice types; the workspace is back in its initial
    state after every call.  Workgroups run one after the other here, in ticket order, which the
    kernels' own rule (a chunk waits only for chunks with earlier tickets) makes sufficient."""
    capi = host_on_cpu
    seen_chunks = set()
    for seed, max_s in ((910, 20), (912, 190), (913, 130)):
        c = cases.mi_case(seed, dtype=np.float64, max_B=3, max_S=max_s, max_T=60,
                          force={"modified": modified, "rand_bd": seed % 2 == 0})
        B, S, T = c["B"], c["S"], c["T"]
        seen_chunks.add(S // 64 + 1)
        px, py = torch.from_numpy(c["px"]), torch.from_numpy(c["py"])
        bd = None if c["boundary"] is None else torch.from_numpy(c["boundary"])
        assert capi.lib().k2amd_mi_workspace_bytes(B, S, T, int(modified), 1) > 0
        p = torch.empty(B, S + 1, T + 1, dtype=torch.float64)
        ans = capi.mi_forward(px, py, bd, p)
        want_ans, want_p = omi.mi_forward(c["px"], c["py"], c["boundary"])
        np.testing.assert_allclose(ans.numpy(), want_ans, rtol=1e-10, atol=1e-10)
        g = torch.full((B,), 1.0, dtype=torch.float64)
        gx, gy = capi.mi_backward(px, py, bd, p, g, overwrite_ans_grad=True)
        want_gx, want_gy = omi.mi_backward(c["px"], c["py"], c["boundary"], want_p)
        np.testing.assert_allclose(gx.numpy(), want_gx, rtol=1e-9, atol=1e-10)
        np.testing.assert_allclose(gy.numpy(), want_gy, rtol=1e-9, atol=1e-10)
        finite = np.isfinite(want_ans)
        np.testing.assert_allclose(g.numpy()[finite], 1.0, rtol=1e-9)
        assert capi.mi_workspace_is_clean(px.device)
    assert len(seen_chunks) >= 2, seen_chunks


def test_smoke_entry_point_runs(host_on_cpu, capsys):
    """__graft_entry__.smoke()'s own body on CPU tensors, over the host build of the kernels."""
    import __graft_entry__
    __graft_entry__.smoke("cpu")
    assert "smoke ok" in capsys.readouterr().out


# ---- the fused joiner: built for the host from a copy of joiner.hip in which the three lines that
# spell bfloat16 vectors and aligned dynamic LDS are replaced (tests/cpu_kernels.py); the matrix
# instructions of both operand types and the quad DPP moves come from the stand-in -----------------

@pytest.mark.parametrize("rnnt_type,hat", [("regular", False), ("constrained", True),
                                           pytest.param("modified", True, marks=slow),
                                           pytest.param("modified", False, marks=slow),
                                           pytest.param("constrained", False, marks=slow),
                                           pytest.param("regular", True, marks=slow)])
def test_fused_joiner_fp32(host_on_cpu, rnnt_type, hat):
    """hat: the hybrid autoregressive transducer's log-probs inside the fused kernels (column 0 with
    its own sigmoid, the normaliser over the other columns)."""
    import test_joiner_gpu as tj
    cpu = torch.device("cpu")
    # the second shape has more than one tile of 256 columns: column 0 is left out of the
    # normaliser in the first tile only
    for seed, B, T, S, C, D, R, with_bias in ((1, 2, 9, 4, 11, 64, 3, True), (2, 1, 7, 3, 300, 128, 2, False)):
        c = tj.joiner_case(seed, B, T, S, C, D, R, rnnt_type, with_bias)
        if hat:
            c["symbols"][:, 0] = 0  # the blank's column as an ordinary symbol
        logits, px, py = tj.chain_fp64(c, hat)
        gpx, gpy, norm = tj.run_forward(c, cpu, "fp32", hat)
        tag = f"{rnnt_type} seed {seed}"
        tj.close(tag + " px", gpx.numpy(), px, 1e-4, 1e-5 / max(np.abs(px[np.isfinite(px)]).max(), 1e-30))
        tj.close(tag + " py", gpy.numpy(), py, 1e-4, 1e-5 / max(np.abs(py[np.isfinite(py)]).max(), 1e-30))
        _, gx, gy = omi.mi(px, py, c["boundary"])
        gx, gy = gx.astype(np.float32), gy.astype(np.float32)
        scale = np.linspace(0.5, 1.5, B).astype(np.float32)
        want = tj.closed_form_grads(c, logits, gx, gy, scale, hat)
        got = tj.run_backward(c, cpu, "fp32", norm, gx, gy, scale, hat)
        for name, g, w in zip(("am_grad", "lm_grad", "weight_grad", "bias_grad"), got, want):
            if g is None:
                assert name == "bias_grad" and not with_bias
                continue
            tj.close(f"{tag} {name}", g, w, 1e-4, 1e-5)


def test_fused_joiner_bf16_and_no_frames(host_on_cpu):
    import test_joiner_gpu as tj
    from k2_amd import capi
    cpu = torch.device("cpu")
    c = tj.joiner_case(3, 2, 9, 4, 11, 64, 3, "regular", True)
    logits, px, py = tj.chain_fp64(c)
    gpx, gpy, norm = tj.run_forward(c, cpu, "bf16")
    fin = np.isfinite(px)
    assert np.array_equal(np.isfinite(gpx.numpy()), fin)
    assert np.abs(gpx.numpy()[fin] - px[fin]).max() < 3e-2 and np.abs(gpy.numpy()[np.isfinite(py)] - py[np.isfinite(py)]).max() < 3e-2
    # no frames at all: py is empty, px is its one -inf column
    B, S, R, C, D = 2, 5, 3, 11, 64
    rng = np.random.default_rng(3)
    lm = torch.from_numpy(rng.standard_normal((B, S + 1, D)).astype(np.float32))
    px0, py0, _ = capi.joiner_pruned_forward(torch.zeros(B, 0, D), lm, torch.zeros(B, 0, R, dtype=torch.int64),
                                             torch.from_numpy(rng.standard_normal((C, D)).astype(np.float32)), None,
                                             torch.from_numpy(rng.integers(1, C, (B, S)).astype(np.int64)), 0, None, 0)
    assert tuple(px0.shape) == (B, S, 1) and tuple(py0.shape) == (B, S + 1, 0) and torch.isneginf(px0).all()


def test_hat_loss_through_the_fused_joiner(host_on_cpu, monkeypatch):
    """rnnt_loss_pruned_joiner(use_hat_loss=True) against the three steps it replaces
    (do_rnnt_pruning, tanh + linear, rnnt_loss_pruned(use_hat_loss=True)): loss and the gradients
    to am, lm, weight and bias; refused while its switch is off."""
    import k2_amd as k2
    import test_joiner_gpu as tj
    c = tj.joiner_case(5, 2, 9, 4, 11, 64, 3, "regular", True)
    t = lambda k, grad=False: torch.from_numpy(c[k]).requires_grad_(grad)
    sym, bd, ranges = t("symbols"), t("boundary"), t("ranges")
    a1, l1, w1, b1 = t("am", True), t("lm", True), t("weight", True), t("bias", True)
    with pytest.raises(RuntimeError, match="K2AMD_JOINER_HAT"):
        k2.rnnt_loss_pruned_joiner(a1, l1, ranges, w1, b1, sym, 0, bd, reduction="sum", use_hat_loss=True)
    monkeypatch.setenv("K2AMD_JOINER_HAT", "1")
    fused = k2.rnnt_loss_pruned_joiner(a1, l1, ranges, w1, b1, sym, 0, bd, reduction="sum", use_hat_loss=True)
    fused.backward()
    a2, l2, w2, b2 = t("am", True), t("lm", True), t("weight", True), t("bias", True)
    am_p, lm_p = k2.do_rnnt_pruning(a2, l2, ranges)
    logits = torch.nn.functional.linear(torch.tanh(am_p + lm_p), w2, b2)
    steps = k2.rnnt_loss_pruned(logits, sym, ranges, 0, bd, reduction="sum", use_hat_loss=True)
    steps.backward()
    np.testing.assert_allclose(fused.item(), steps.item(), rtol=1e-5)
    for name, x, y in (("am", a1, a2), ("lm", l1, l2), ("weight", w1, w2), ("bias", b1, b2)):
        scale = float(y.grad.abs().max())
        np.testing.assert_allclose(x.grad.numpy(), y.grad.numpy(), rtol=1e-4, atol=1e-5 * scale, err_msg=name)
