"""Pins oracle/lattice.py against the golden vectors of the reference's own test
(k2/python/tests/pruned_ranges_to_lattice_test.py:45-205)."""
import json
import os

import numpy as np
import pytest

from oracle import lattice as olat

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "pruned_ranges_to_lattice.json")


def golden_case(dtype=np.float32):
    g = json.load(open(GOLDEN))
    ranges = np.array(g["ranges"], dtype=np.int32)
    B, T, R = ranges.shape
    C = g["C"]
    base = np.array(g["logits_base"], dtype=np.float32)
    # pruned_ranges_to_lattice_test.py:186-197
    logits = np.broadcast_to(base, (B, T, R, C)).copy()
    logits = logits + (10.0 * np.arange(1, B * T + 1, dtype=np.float32)).reshape(B, T, 1, 1)
    logits = logits + np.arange(R, dtype=np.float32).reshape(1, 1, R, 1)
    return dict(ranges=ranges, frames=np.array(g["frames"], dtype=np.int32),
                symbols=np.array(g["symbols"], dtype=np.int64), logits=logits.astype(dtype),
                arc_map=np.array(g["arc_map"], dtype=np.int32),
                arcs=np.array(g["arcs"], dtype=np.int32))


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_oracle_matches_reference_golden(dtype):
    c = golden_case(dtype)
    state_splits, arc_splits, arcs, scores, arc_map = olat.pruned_ranges_to_lattice(
        c["ranges"], c["frames"], c["symbols"], c["logits"])
    assert np.array_equal(arc_map, c["arc_map"])
    assert np.array_equal(arcs, c["arcs"])
    assert list(state_splits) == [0, 21, 37]
    assert arc_splits[-1] == 49 and len(arc_splits) == 38
    # scores are the logits the map points at (:101-109); 0 for the arcs into the final states
    flat = c["logits"].reshape(-1).astype(np.float32)
    want = np.where(arc_map >= 0, flat[np.maximum(arc_map, 0)], 0.0)
    assert np.array_equal(scores, want)


def test_oracle_structure_on_random_bands():
    rng = np.random.default_rng(0)
    for _ in range(10):
        B, T, R, S, C = 3, int(rng.integers(2, 9)), int(rng.integers(2, 5)), 9, 7
        # a valid band: starts at 0 and moves by less than R per frame (k2/python/k2/rnnt_loss.py:583-589)
        start = np.minimum(np.cumsum(rng.integers(0, R, (B, T)), axis=1) - rng.integers(0, R, (B, 1)), S - R + 1)
        start = np.maximum(start, 0)
        ranges = (start[:, :, None] + np.arange(R)).astype(np.int32)
        frames = rng.integers(1, T + 1, B).astype(np.int32)
        symbols = rng.integers(1, C, (B, S)).astype(np.int64)
        logits = rng.standard_normal((B, T, R, C)).astype(np.float32)
        ss, asp, arcs, scores, amap = olat.pruned_ranges_to_lattice(ranges, frames, symbols, logits)
        assert ss[-1] == (frames * R + 1).sum() and asp[-1] == len(arcs)
        for b in range(B):
            lo, hi = asp[ss[b]], asp[ss[b + 1]]
            a = arcs[lo:hi]
            assert (a[:, 1] > a[:, 0]).all()            # acyclic, states in topological order
            assert (a[:, 1] <= frames[b] * R).all()
            assert (a[:, 2] == -1).sum() == 1 and a[-1, 2] == -1
            assert a[-1, 1] == frames[b] * R
