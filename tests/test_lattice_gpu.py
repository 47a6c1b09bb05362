"""pruned_ranges_to_lattice on the GPU: bit-exact against the reference's golden vectors
(k2/python/tests/pruned_ranges_to_lattice_test.py:45-205) and against the oracle on random bands,
through the k2-style API, the C++ host and the ctypes host."""
import numpy as np
import pytest
import torch

from oracle import lattice as olat
from test_oracle_lattice import golden_case

pytestmark = pytest.mark.gpu

TORCH_DT = {np.float32: torch.float32, np.float64: torch.float64, np.float16: torch.float16}


def _dev(x, device):
    return torch.from_numpy(np.ascontiguousarray(x)).to(device)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_reference_golden_vectors(device, dtype):
    import k2_amd as k2
    c = golden_case(dtype)
    ofsa, arc_map = k2.pruned_ranges_to_lattice(_dev(c["ranges"], device), _dev(c["frames"], device),
                                                _dev(c["symbols"], device), _dev(c["logits"], device))
    assert arc_map.dtype == torch.int32
    assert torch.equal(arc_map.cpu(), torch.from_numpy(c["arc_map"]))
    assert torch.equal(ofsa.values()[:, :3].cpu(), torch.from_numpy(c["arcs"]))
    # scores == index_select(logits.reshape(-1), arc_map) with 0 where the map is -1 (:101-109)
    flat = _dev(c["logits"], device).reshape(-1).to(torch.float32)
    want = torch.where(arc_map >= 0, flat[arc_map.clamp(min=0).long()], torch.zeros((), device=device))
    assert torch.equal(ofsa.scores, want)
    assert ofsa.row_splits(1).tolist() == [0, 21, 37]
    assert ofsa.row_splits(2)[-1].item() == 49 and ofsa.dim0 == 2 and ofsa.num_elements == 49


@pytest.mark.parametrize("host", ["pybind", "ctypes"])
def test_random_bands_match_oracle(device, host):
    from k2_amd import capi, native
    rng = np.random.default_rng(7)
    for case in range(12):
        B = int(rng.integers(1, 6))
        T = int(rng.integers(1, 300 if case % 3 == 0 else 20))
        R = int(rng.integers(1, 6))
        S, C = int(rng.integers(R, R + 30)), int(rng.integers(2, 40))
        start = np.clip(np.cumsum(rng.integers(0, max(R, 2), (B, T)), axis=1) - R, 0, S - R)
        ranges = (start[:, :, None] + np.arange(R)).astype(np.int32)
        frames = rng.integers(1, T + 1, B).astype(np.int32)
        symbols = rng.integers(0, C, (B, S)).astype(np.int64)
        dtype = (np.float32, np.float64, np.float16)[case % 3]
        logits = rng.standard_normal((B, T, R, C)).astype(dtype)
        want = olat.pruned_ranges_to_lattice(ranges, frames, symbols, logits)
        args = (_dev(ranges, device), _dev(frames, device), _dev(symbols, device), _dev(logits, device))
        got = native.pruned_ranges_to_lattice(*args) if host == "pybind" else capi.pruned_ranges_to_lattice(*args)
        state_splits, arc_splits, arcs, arc_map = [g.cpu().numpy() for g in got]
        assert np.array_equal(state_splits, want[0]), case
        assert np.array_equal(arc_splits, want[1]), case
        assert np.array_equal(arcs[:, :3], want[2]), case
        assert np.array_equal(arcs[:, 3].view(np.float32), want[3]), case
        assert np.array_equal(arc_map, want[4]), case


def test_strided_logits_and_errors(device):
    """arc_map follows the strides of the logits it was given (pruned_ranges_to_lattice.cu:172-176),
    and bad inputs raise RuntimeError like the reference's TORCH_CHECKs (:66-77)."""
    import k2_amd as k2
    c = golden_case(np.float32)
    big = torch.zeros(2, 4, 5, 12, device=device)
    big[..., :9] = _dev(c["logits"], device)
    view = big[..., :9]
    ofsa, arc_map = k2.pruned_ranges_to_lattice(_dev(c["ranges"], device), _dev(c["frames"], device),
                                                _dev(c["symbols"], device), view)
    assert torch.equal(ofsa.values()[:, :3].cpu(), torch.from_numpy(c["arcs"]))
    ok = arc_map >= 0
    assert torch.equal(big.reshape(-1)[arc_map[ok].long()], ofsa.scores[ok])
    with pytest.raises(RuntimeError):
        k2.pruned_ranges_to_lattice(_dev(c["ranges"], device).long(), _dev(c["frames"], device),
                                    _dev(c["symbols"], device), view)
    with pytest.raises(RuntimeError):
        k2.pruned_ranges_to_lattice(_dev(c["ranges"], device), _dev(c["frames"], device),
                                    _dev(c["symbols"], device), view[0])
    with pytest.raises(RuntimeError, match="no CPU path"):
        k2.pruned_ranges_to_lattice(torch.from_numpy(c["ranges"]), torch.from_numpy(c["frames"]),
                                    torch.from_numpy(c["symbols"]), torch.from_numpy(c["logits"]))


def test_degenerate_shapes(device):
    """A sequence without frames is a lone final state; an empty batch gives empty outputs."""
    import k2_amd as k2
    ranges = torch.zeros(2, 3, 2, dtype=torch.int32, device=device)
    ranges[..., 1] = 1
    frames = torch.tensor([0, 3], dtype=torch.int32, device=device)
    symbols = torch.tensor([[1, 2], [2, 1]], dtype=torch.long, device=device)
    logits = torch.randn(2, 3, 2, 4, device=device)
    ofsa, arc_map = k2.pruned_ranges_to_lattice(ranges, frames, symbols, logits)
    want = olat.pruned_ranges_to_lattice(ranges.cpu().numpy(), frames.cpu().numpy(), symbols.cpu().numpy(),
                                         logits.cpu().numpy())
    assert ofsa.row_splits(1).tolist() == [0, 1, 8]
    assert np.array_equal(ofsa.row_splits(2).cpu().numpy(), want[1])
    assert np.array_equal(ofsa.values()[:, :3].cpu().numpy(), want[2])
    assert np.array_equal(arc_map.cpu().numpy(), want[4])
    empty = k2.pruned_ranges_to_lattice(ranges[:0], frames[:0], symbols[:0], logits[:0])
    assert empty[0].dim0 == 0 and empty[0].num_elements == 0 and empty[1].numel() == 0
    assert empty[0].row_splits(1).tolist() == [0] and empty[0].row_splits(2).tolist() == [0]
