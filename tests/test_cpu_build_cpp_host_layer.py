"""The C++ host layer (k2_amd/csrc/pybind.cpp) on CPU tensors: a copy in which only the places
that touch the device are replaced (tests/cpu_kernels.py::HOST_LAYER_EDITS: the device guard,
torch's current stream, the event behind the boundary copy, pinned memory, "is on the device"),
built against the host build of the kernels.  Everything else of that file runs as it runs on the
GPU box: the checks, the allocations and their shapes, the order and count of the arguments of
every C-ABI call, what comes back.

It is compared with the ctypes host layer (k2_amd/capi.py), function by function and bit for
bit, as tests/test_zw_host_layers_gpu.py and tests/test_mi_gpu.py compare the two on the GPU, and
the loss functions run end to end through it against the reference's fixtures."""
import os

import numpy as np
import pytest
import torch

import cases
import cpu_kernels as ck
from test_cpu_build_host_layer import host_on_cpu  # noqa: F401  (a fixture)

slow = pytest.mark.skipif(os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1",
                          reason="slow on the host: run with K2AMD_SLOW_CPU_TESTS=1")
CPU = torch.device("cpu")


@pytest.fixture
def hosts(host_on_cpu, monkeypatch):  # noqa: F811
    """(native with the C++ host layer behind it, capi), both over the host build of the kernels."""
    from k2_amd import native
    monkeypatch.setattr(native, "_ext", ck.host_layer())
    return native, host_on_cpu


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("rnnt_type,dtype", [
    ("regular", np.float32), ("constrained", np.float64),
    ("modified", np.float32), pytest.param("regular", np.float64, marks=slow),
    pytest.param("constrained", np.float32, marks=slow), pytest.param("modified", np.float64, marks=slow)])
def test_builders_of_both_hosts(hosts, rnnt_type, dtype):
    import test_zw_host_layers_gpu as zw
    zw.test_builders(CPU, hosts, rnnt_type, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pruning_and_lattice_of_both_hosts(hosts, dtype):
    import test_zw_host_layers_gpu as zw
    zw.test_pruning_and_lattice(CPU, hosts, dtype)


@pytest.mark.parametrize("modified", [False, True])
def test_deprecated_ranges_of_both_hosts(hosts, modified):
    import test_zw_host_layers_gpu as zw
    zw.test_deprecated_ranges(CPU, hosts, modified)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", ["regular", "modified"])
def test_smoothed_builder_of_both_hosts(hosts, rnnt_type, dtype):
    import test_zw_host_layers_gpu as zw
    zw.test_smoothed_builder(CPU, hosts, rnnt_type, dtype)


def test_recursion_of_both_hosts(hosts):
    """The functions of the reference's names (mutual_information.cu:26-67) in both hosts: the pair,
    the pair that hands the log-derivatives on, the single launch, a strided px made contiguous
    by the C++ host, ans_grad overwritten."""
    native, capi = hosts
    ext = native._ext
    rng = np.random.default_rng(77)
    B, S, T = 2, 70, 40
    px = _t(rng.standard_normal((B, S, T + 1)).astype(np.float32))
    py = _t(rng.standard_normal((B, S + 1, T)).astype(np.float32))
    bd = torch.tensor([[0, 0, S, T], [3, 5, 66, 33]], dtype=torch.int64)
    p1, p2 = torch.empty(B, S + 1, T + 1), torch.empty(B, S + 1, T + 1)
    ans1 = capi.mi_forward(px, py, bd, p1)
    px_strided = torch.empty(B, S, 2 * px.shape[2])[:, :, ::2]
    px_strided.copy_(px)
    ans2 = ext.mutual_information_forward(px=px_strided, py=py, boundary=bd, p=p2)
    g1, g2 = torch.full((B,), 2.0), torch.full((B,), 2.0)
    gx1, gy1 = capi.mi_backward(px, py, bd, p1, g1, overwrite_ans_grad=True)
    gx2, gy2 = ext.mutual_information_backward(px=px, py=py, boundary=bd, p=p2, ans_grad=g2)
    for x, y in ((ans1, ans2), (gx1, gx2), (gy1, gy2), (g1, g2)):  # (p is undefined outside the boxes)
        assert torch.equal(x, y)
    assert ext.mutual_information_keeps_log_deriv(px=px, py=py) == bool(capi.mi_keeps_log_deriv(px, py))
    if ext.mutual_information_keeps_log_deriv(px=px, py=py):
        p3, kept = torch.empty(B, S + 1, T + 1), torch.full((B, S + 1, T + 1), float("nan"))
        ans3 = ext.mutual_information_forward(px=px_strided, py=py, boundary=bd, p=p3, log_deriv=kept)
        g3 = torch.full((B,), 2.0)
        gx3, gy3 = ext.mutual_information_backward(px=px, py=py, boundary=bd, p=p3, ans_grad=g3, log_deriv=kept)
        assert torch.equal(ans3, ans2) and torch.equal(gx3, gx2) and torch.equal(gy3, gy2) and torch.equal(g3, g2)
        with pytest.raises(RuntimeError):  # wrong shape
            ext.mutual_information_forward(px=px, py=py, boundary=bd, p=p3, log_deriv=kept[:, :-1])
    assert ext.mutual_information_forward_backward_supported(px=px, py=py) == bool(capi.mi_forward_backward_supported(px, py))
    if ext.mutual_information_forward_backward_supported(px=px, py=py):
        g5, g6 = torch.full((B,), 2.0), torch.full((B,), 2.0)
        ans5, gx5, gy5 = ext.mutual_information_forward_backward(px=px_strided, py=py, boundary=bd, ans_grad=g5)
        ans6, gx6, gy6 = capi.mi_forward_backward(px, py, bd, g6, overwrite_ans_grad=True)
        assert torch.equal(ans5, ans6) and torch.equal(gx5, gx6) and torch.equal(gy5, gy6) and torch.equal(g5, g6)
        np.testing.assert_allclose(ans5.numpy(), ans2.numpy(), rtol=1e-4, atol=1e-5)
    rows = ext.BoundaryRead(bd).rows()
    assert rows == tuple(tuple(r) for r in bd.tolist())
    ws = ext.mutual_information_workspace(px)
    assert ws is not None and ws.dtype == torch.uint8
    assert ext.mutual_information_recover_workspaces() == 0


def test_joint_products_of_both_hosts(hosts):
    native, capi = hosts
    rng = np.random.default_rng(807)
    N, B, S, T = 3, 2, 4, 7
    pxs = [_t(-rng.uniform(0, 3, (B, S, T + 1))) for _ in range(N)]
    pys = [_t(-rng.uniform(0, 3, (B, S + 1, T))) for _ in range(N)]
    gx, gy = _t(rng.uniform(0, 1, (B, S, T + 1))), _t(rng.uniform(0, 1, (B, S + 1, T)))
    assert torch.equal(native._ext.mutual_information_joint_products(pxs, pys, gx, gy),
                       capi.mi_joint_products(pxs, pys, gx, gy))


@pytest.mark.parametrize("name", ["test_reference_chain_fixtures",
                                  "test_reference_prune_ranges_on_ties_and_near_ties",
                                  pytest.param("test_reference_smoothed_and_hat_gradient_fixtures", marks=slow)])
def test_reference_fixtures_through_the_api_over_the_cpp_host(hosts, name, monkeypatch):
    """What was recorded from the reference's own Python chain, through k2_amd's API with the C++
    host layer underneath: losses, occupation probabilities, gradients, both kinds of prune
    ranges (every eighth chain; every second with the slow switch)."""
    import test_rnnt_gpu
    if "chain" in name:
        monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1")
        getattr(test_rnnt_gpu, name)(CPU, every=2 if os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") == "1" else 8)
        return
    if "smoothed" in name:
        monkeypatch.setenv("K2AMD_SMOOTHED_KERNELS", "1")
    getattr(test_rnnt_gpu, name)(CPU)


def test_recursion_scenario_over_the_cpp_host(hosts):
    """mutual_information_recursion through its autograd Function with the C++ host layer
    underneath (boundary read, workspace cache, the single launch or the pair as advised)."""
    import k2_amd as k2
    from oracle import mi as omi
    c = cases.mi_case(41, dtype=np.float32, max_B=3, max_S=20, max_T=40, force={"rand_bd": True})
    px, py = _t(c["px"]).requires_grad_(True), _t(c["py"]).requires_grad_(True)
    scores = k2.mutual_information_recursion(px, py, _t(c["boundary"]))
    want, gx, gy = omi.mi(c["px"], c["py"], c["boundary"])
    np.testing.assert_allclose(scores.detach().numpy(), want, rtol=1e-4, atol=1e-5)
    finite = np.isfinite(want)
    scores[torch.from_numpy(finite)].sum().backward()
    for b in np.nonzero(finite)[0]:
        np.testing.assert_allclose(px.grad.numpy()[b], gx[b], rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(py.grad.numpy()[b], gy[b], rtol=1e-4, atol=1e-5)


def test_error_flag_rides_with_the_cpp_hosts_boundary_read(hosts):
    """The error flag of the stream's workspace rides with the C++ host's boundary read: forced
    from the host, it turns the next read into a RuntimeError that names the timeout, once, and
    the workspace is initialised again, so that the call after that works.  (Through the API this
    runs on the GPU, tests/test_mi_gpu.py::test_a_wait_that_gave_up_raises_at_the_next_call: the
    Python layer reads a host tensor's rows without this class.)"""
    native, capi = hosts
    ext = native._ext
    rng = np.random.default_rng(19)
    B, S, T = 2, 70, 40
    px = _t(rng.normal(-2, 1, (B, S, T + 1)).astype(np.float32))
    py = _t(rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32))
    bd = torch.tensor([[0, 0, S, T], [1, 2, 60, 33]], dtype=torch.int64)
    p = torch.empty(B, S + 1, T + 1)
    good = ext.mutual_information_forward(px=px, py=py, boundary=bd, p=p).clone()
    assert torch.isfinite(good).all()
    ws = ext.mutual_information_workspace(px)
    assert ws is not None
    ws[:16].view(torch.int32)[2] = 1                         # FastHeader::error
    assert torch.isnan(ext.mutual_information_forward(px=px, py=py, boundary=bd, p=p)).all()
    with pytest.raises(RuntimeError, match="timed out"):
        ext.BoundaryRead(bd).rows()
    assert int(ws[:16].view(torch.int32)[2]) == 0
    assert ext.BoundaryRead(bd).rows() == tuple(tuple(r) for r in bd.tolist())
    assert torch.equal(ext.mutual_information_forward(px=px, py=py, boundary=bd, p=p), good)
    assert ext.mutual_information_recover_workspaces() == 0
