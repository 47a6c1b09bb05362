"""TEST INFRASTRUCTURE ONLY: pure-Python restatement of PrunedRangesToLattice
(k2/python/csrc/torch/pruned_ranges_to_lattice.cu:60-263).

Parity status: **pinned** by the golden vectors of the reference's own test
(k2/python/tests/pruned_ranges_to_lattice_test.py:45-168, committed as
tests/golden/pruned_ranges_to_lattice.json): arc_map and the (src, dest, label) columns of every
arc, for float32, float64 and float16 logits, plus scores == logits.reshape(-1)[arc_map].

Only tests may import this.
"""
import numpy as np


def pruned_ranges_to_lattice(ranges, frames, symbols, logits):
    """ranges int32 [B,T,R], frames int32 [B], symbols int64 [B,S], logits [B,T,R,C].
    Returns (state_splits [B+1], arc_splits [states+1], arcs int32 [N,3], scores f32 [N],
    arc_map int32 [N])."""
    B, T, R = ranges.shape
    st = [s // logits.itemsize for s in logits.strides]
    # fsa -> states (pruned_ranges_to_lattice.cu:109-121): frames * R + 1 (the super-final state)
    state_splits = np.zeros(B + 1, dtype=np.int32)
    for b in range(B):
        assert frames[b] <= T
        state_splits[b + 1] = state_splits[b] + frames[b] * R + 1
    # state -> number of arcs (:123-160)
    counts = []
    for b in range(B):
        F = int(frames[b])
        for s1 in range(F * R + 1):
            t, k = divmod(s1, R)
            if s1 == F * R:
                counts.append(0)
                continue
            n = 1
            horizontal = False
            if t < F - 1:
                horizontal = ranges[b, t, k] >= ranges[b, t + 1, 0]
            if k != R - 1 and horizontal:
                n = 2
            counts.append(n)
    arc_splits = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    # arcs (:183-258)
    arcs, scores, arc_map = [], [], []
    for b in range(B):
        F = int(frames[b])
        for s1 in range(F * R + 1):
            t, k = divmod(s1, R)
            n = counts[state_splits[b] + s1]
            for a in range(n):
                if s1 == F * R - 1:
                    arcs.append((s1, s1 + 1, -1)); scores.append(0.0); arc_map.append(-1)
                    continue
                base = b * st[0] + t * st[1] + k * st[2]
                if k < R - 1:
                    label = int(symbols[b, ranges[b, t, k]])
                    if a == 0:
                        arcs.append((s1, s1 + 1, label))
                        scores.append(float(logits[b, t, k, label]))
                        arc_map.append(base + label * st[3])
                    else:
                        dest = int(ranges[b, t, k]) - int(ranges[b, t + 1, 0]) + (t + 1) * R
                        arcs.append((s1, dest, 0))
                        scores.append(float(logits[b, t, k, 0]))
                        arc_map.append(base)
                else:
                    dest = int(ranges[b, t, k]) - int(ranges[b, t + 1, 0]) + (t + 1) * R
                    arcs.append((s1, dest, 0))
                    scores.append(float(logits[b, t, k, 0]))
                    arc_map.append(base)
    return (state_splits, arc_splits, np.array(arcs, dtype=np.int32).reshape(-1, 3),
            np.array(scores, dtype=np.float32), np.array(arc_map, dtype=np.int32))
