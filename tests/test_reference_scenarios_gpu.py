"""The scenarios of the reference's own tests for this path (k2/python/tests/rnnt_loss_test.py,
mutual_information_test.py), replayed against this package.  Where the reference compares its CUDA
device with its CPU device, the CPU side here is the oracle; its identities are asserted as they
stand.  torch.allclose defaults (rtol 1e-5, atol 1e-8) are the reference's own tolerances."""
import numpy as np
import pytest
import torch

from oracle import rnnt as orn

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("rnnt_type", ["regular", "modified", "constrained"])
def test_rnnt_loss_random(device, rnnt_type):
    """rnnt_loss_test.py:246-376: B=5, S<=20, T<=300, C=100, lengths in the boundary; the simple,
    smoothed(0, 0) and joint losses agree with each other and with the CPU value, and are
    invariant to per-frame constants."""
    import k2_amd as k2
    g = torch.Generator().manual_seed(20)
    B, S, T, C = 5, 20, 300, 100
    frames = torch.randint(S, T, (B,), generator=g)
    seq_length = torch.randint(3, S - 1, (B,), generator=g)
    T, S = int(frames.max()), int(seq_length.max())
    am_ = torch.randn((B, T, C), generator=g)
    lm_ = torch.randn((B, S + 1, C), generator=g)
    symbols_ = torch.randint(0, C - 1, (B, S), generator=g)
    blank = C - 1
    boundary_ = torch.zeros((B, 4), dtype=torch.int64)
    boundary_[:, 2] = seq_length
    boundary_[:, 3] = frames
    expected = torch.tensor(orn.rnnt_loss_simple(_np(lm_), _np(am_), _np(symbols_), blank, _np(boundary_),
                                                 rnnt_type, reduction="mean"))
    lm, am = lm_.to(device), am_.to(device)
    symbols, boundary = symbols_.to(device), boundary_.to(device)
    px, py = k2.get_rnnt_logprobs(lm=lm, am=am, symbols=symbols, termination_symbol=blank, boundary=boundary,
                                  rnnt_type=rnnt_type)
    assert px.shape == ((B, S, T) if rnnt_type != "regular" else (B, S, T + 1))
    assert py.shape == (B, S + 1, T)
    m = k2.mutual_information_recursion(px=px, py=py, boundary=boundary)
    assert torch.allclose(-torch.mean(m).cpu(), expected, rtol=1e-4)

    def all_three(lm, am):
        a = k2.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=blank, boundary=boundary,
                                rnnt_type=rnnt_type)
        b = k2.rnnt_loss_smoothed(lm=lm, am=am, symbols=symbols, termination_symbol=blank, lm_only_scale=0.0,
                                  am_only_scale=0.0, boundary=boundary, rnnt_type=rnnt_type)
        c = k2.rnnt_loss(logits=am.unsqueeze(2) + lm.unsqueeze(1), symbols=symbols, termination_symbol=blank,
                         boundary=boundary, rnnt_type=rnnt_type)
        return a, b, c

    for m in all_three(lm, am):
        assert torch.allclose(m.cpu(), expected, rtol=1e-4), (m, expected)
    lm2 = lm + torch.randn(B, S + 1, 1, device=device)
    am2 = am + torch.randn(B, T, 1, device=device)
    for m in all_three(lm2, am2):
        assert torch.allclose(m.cpu(), expected, rtol=1e-4), (m, expected)


def test_rnnt_loss_gradient(device):
    """rnnt_loss_test.py:378-434 without torchaudio (absent here): the gradients of the simple loss
    with respect to am and lm equal those of the joint loss on am + lm, which autograd pushes
    through the broadcast sum."""
    import k2_amd as k2
    g = torch.Generator().manual_seed(21)
    B, S, T, C = 3, 12, 60, 30
    am_ = torch.randn((B, T, C), generator=g, dtype=torch.float64)
    lm_ = torch.randn((B, S + 1, C), generator=g, dtype=torch.float64)
    symbols = torch.randint(0, C - 1, (B, S), generator=g).to(device)
    boundary = torch.tensor([[0, 0, S, T], [0, 0, S - 3, T - 7], [0, 0, 5, 40]]).to(device)
    grads = []
    for joint in (False, True):
        am = am_.to(device).requires_grad_(True)
        lm = lm_.to(device).requires_grad_(True)
        if joint:
            loss = k2.rnnt_loss(logits=am.unsqueeze(2) + lm.unsqueeze(1), symbols=symbols, termination_symbol=C - 1,
                                boundary=boundary, reduction="sum")
        else:
            loss = k2.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=C - 1,
                                       boundary=boundary, reduction="sum")
        loss.backward()
        grads.append((loss.item(), am.grad.cpu(), lm.grad.cpu()))
    assert grads[0][0] == pytest.approx(grads[1][0], rel=1e-10)
    assert torch.allclose(grads[0][1], grads[1][1], rtol=1e-8, atol=1e-10)
    assert torch.allclose(grads[0][2], grads[1][2], rtol=1e-8, atol=1e-10)


def test_rnnt_loss_pruned_tracks_the_full_loss(device):
    """rnnt_loss_test.py:486-570: with am + lm as the pruned joiner output, the pruned loss
    approaches the simple loss from above as s_range grows and equals it once nothing is pruned;
    the reference prints the values, here the ordering is asserted."""
    import k2_amd as k2
    g = torch.Generator().manual_seed(22)
    B, T, S, C = 4, 300, 50, 10
    frames = torch.randint(S, T, (B,), generator=g)
    seq_length = torch.randint(3, S - 1, (B,), generator=g)
    T, S = int(frames.max()), int(seq_length.max())
    am = torch.randn((B, T, C), generator=g, dtype=torch.float64).to(device)
    lm = torch.randn((B, S + 1, C), generator=g, dtype=torch.float64).to(device)
    symbols = torch.randint(0, C - 1, (B, S), generator=g).to(device)
    boundary = torch.zeros((B, 4), dtype=torch.int64)
    boundary[:, 2] = seq_length
    boundary[:, 3] = frames
    boundary = boundary.to(device)
    for rnnt_type in ("regular", "modified", "constrained"):
        full = k2.rnnt_loss(logits=am.unsqueeze(2) + lm.unsqueeze(1), symbols=symbols, termination_symbol=C - 1,
                            boundary=boundary, rnnt_type=rnnt_type, reduction="none")
        simple, (px_grad, py_grad) = k2.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=C - 1,
                                                         boundary=boundary, rnnt_type=rnnt_type,
                                                         return_grad=True, reduction="none")
        assert torch.allclose(full, simple)
        previous = None
        for r in range(2, 50, 5):
            ranges = k2.get_rnnt_prune_ranges(px_grad=px_grad, py_grad=py_grad, boundary=boundary, s_range=r)
            am_p, lm_p = k2.do_rnnt_pruning(am=am, lm=lm, ranges=ranges)
            pruned = k2.rnnt_loss_pruned(logits=am_p + lm_p, symbols=symbols, ranges=ranges,
                                         termination_symbol=C - 1, boundary=boundary, rnnt_type=rnnt_type,
                                         reduction="none")
            assert torch.isfinite(pruned).all(), (rnnt_type, r, pruned)
            assert (pruned >= simple - 1e-9).all(), (rnnt_type, r)   # pruning only removes paths
            if previous is not None:
                assert (pruned <= previous + 1e-6).all(), (rnnt_type, r)
            previous = pruned
        assert torch.allclose(previous, simple, rtol=1e-6), (rnnt_type, previous, simple)


def test_rnnt_loss_empty_reference(device):
    """rnnt_loss_test.py:927-1050: S = 0 does not crash, and every loss equals the sum of the blank
    log-probabilities."""
    import k2_amd as k2
    lm = torch.tensor([[[0, 0, 1]]], dtype=torch.float, device=device)
    am = torch.tensor([[[0, 1, 2], [0, 0, 0], [0, 2, 4], [0, 3, 3]]], dtype=torch.float, device=device)
    blank = 2
    symbols = torch.zeros((1, 0), dtype=torch.long, device=device)
    expected = -torch.log_softmax(am[0] + lm[0, 0], dim=-1)[:, blank].sum().reshape(1)
    px, py = k2.get_rnnt_logprobs(lm=lm, am=am, symbols=symbols, termination_symbol=blank)
    assert px.shape == (1, 0, 5) and py.shape == (1, 1, 4)
    m = k2.mutual_information_recursion(px=px, py=py, boundary=None)
    assert torch.allclose(-m, expected)
    for _ in range(2):
        m = k2.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=blank, boundary=None,
                                reduction="none")
        assert torch.allclose(m, expected)
        m = k2.rnnt_loss_smoothed(lm=lm, am=am, symbols=symbols, termination_symbol=blank, lm_only_scale=0.0,
                                  am_only_scale=0.0, boundary=None, reduction="none")
        assert torch.allclose(m, expected)
        m = k2.rnnt_loss(logits=am.unsqueeze(2) + lm.unsqueeze(1), symbols=symbols, termination_symbol=blank,
                         boundary=None, reduction="none")
        assert torch.allclose(m, expected)
        # invariant to a constant per frame (second pass)
        lm = lm + torch.randn(1, 1, 1, device=device)
        am = am + torch.randn(1, 4, 1, device=device)


def test_mutual_information_against_itself_and_finite_differences(device):
    """mutual_information_test.py:189-306 in small: the returned occupation gradients equal a
    finite-difference derivative of the scores (fp64, the reference's tolerance 1e-2 relative, here
    far tighter), and autograd's gradient is the occupation scaled by the incoming gradient."""
    import k2_amd as k2
    g = torch.Generator().manual_seed(23)
    for modified in (False, True):
        B, S, T = 2, 5, 9
        T1 = T if modified else T + 1
        px = torch.randn((B, S, T1), generator=g, dtype=torch.float64).to(device).requires_grad_(True)
        py = torch.randn((B, S + 1, T), generator=g, dtype=torch.float64).to(device).requires_grad_(True)
        boundary = torch.tensor([[0, 0, S, T], [1, 2, S - 1, T - 1]]).to(device)
        m, (gx, gy) = k2.mutual_information_recursion(px, py, boundary, return_grad=True)
        w = torch.tensor([0.7, -1.3], dtype=torch.float64, device=device)
        (m * w).sum().backward()
        assert torch.allclose(px.grad, gx * w.reshape(B, 1, 1))
        assert torch.allclose(py.grad, gy * w.reshape(B, 1, 1))
        eps = 1e-6
        for tensor, grad in ((px, gx), (py, gy)):
            for idx in ((0, 2, 3), (1, 3, 4), (1, 1, 2), (0, 0, 0)):
                bumped = tensor.detach().clone()
                bumped[idx] += eps
                args = (bumped, py.detach()) if tensor is px else (px.detach(), bumped)
                m2 = k2.mutual_information_recursion(args[0], args[1], boundary)
                fd = ((m2 - m.detach())[idx[0]] / eps).item()
                assert fd == pytest.approx(grad[idx].item(), abs=1e-5), (modified, idx)
