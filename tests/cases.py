"""Seeded input generators shared by the CPU (oracle) and GPU (parity) tests.

The MI cases follow the recipe of the reference's own randomized test
(k2/python/tests/mutual_information_test.py:44-131): zeros or N(0,1) for px / py, optional +15
offsets, an all -inf last px column, random boundaries that include empty sequences and
non-zero begin offsets.
"""
import numpy as np


def random_boundary(rng, B, S, T, modified):
    rows = []
    for _ in range(B):
        this_S = int(rng.integers(0, S + 1))
        lo = this_S if modified else 1
        lo = min(lo, T)
        this_T = int(rng.integers(lo, T + 1))
        s_begin = int(rng.integers(0, S - this_S + 1))
        t_begin = int(rng.integers(0, T - this_T + 1))
        rows.append([s_begin, t_begin, s_begin + this_S, t_begin + this_T])
    return np.array(rows, dtype=np.int64)


def mi_case(seed, dtype=np.float32, max_B=10, max_S=16, max_T=500, force=None):
    """One random case in the style of the reference test.  Returns a dict."""
    rng = np.random.default_rng(seed)
    B = int(rng.integers(1, max_B + 1))
    S = int(rng.integers(1, max_S + 1))
    T = int(rng.integers(1, max_T + 1))
    random_px = rng.random() < 0.5
    random_py = rng.random() < 0.5
    rand_bd = rng.random() < 0.7
    big_px = rng.random() < 0.2
    big_py = rng.random() < 0.2
    modified = bool(rng.random() < 0.5)
    if force is not None:
        modified = bool(force.get("modified", modified))
        rand_bd = force.get("rand_bd", rand_bd)
        big_px = force.get("big_px", big_px)
        big_py = force.get("big_py", big_py)
        random_px = force.get("random_px", random_px)
        random_py = force.get("random_py", random_py)
    if modified and T < S:
        T = S + int(rng.integers(0, 31))
    T1 = T if modified else T + 1
    if random_px:
        px = rng.standard_normal((B, S, T1)).astype(dtype)
        if S > 1 and not rand_bd and not modified:
            px[:, :, -1:] = -np.inf
    else:
        px = np.zeros((B, S, T1), dtype=dtype)
    if big_px:
        px += dtype(15.0)
    py = rng.standard_normal((B, S + 1, T)).astype(dtype) if random_py else np.zeros((B, S + 1, T), dtype=dtype)
    if big_py:
        py += dtype(15.0)
    if rand_bd:
        boundary = random_boundary(rng, B, S, T, modified)
    elif rng.random() < 0.5:
        boundary = np.tile(np.array([[0, 0, S, T]], dtype=np.int64), (B, 1))
    else:
        boundary = None
    return dict(px=px, py=py, boundary=boundary, modified=modified, B=B, S=S, T=T)


def c4_case(seed=4, B=32, S=200, T=1000, dtype=np.float32):
    """The headline stress shape: modified lattice, log-softmax-like values min(N(-3,1), 0),
    T_b in [0.6 T, T], S_b in [0.5 S, S]."""
    rng = np.random.default_rng(seed)
    px = np.minimum(rng.normal(-3.0, 1.0, (B, S, T)), 0.0).astype(dtype)
    py = np.minimum(rng.normal(-3.0, 1.0, (B, S + 1, T)), 0.0).astype(dtype)
    Tb = rng.integers(int(0.6 * T), T + 1, size=B)
    Sb = rng.integers(int(0.5 * S), S + 1, size=B)
    boundary = np.stack([np.zeros(B, np.int64), np.zeros(B, np.int64), Sb, Tb], axis=1).astype(np.int64)
    return dict(px=px, py=py, boundary=boundary, modified=True, B=B, S=S, T=T)


def rnnt_case(seed, B, T, S, C, dtype=np.float32, t_lo=None, s_lo=None, with_boundary=True,
              modified=False):
    """am/lm/symbols/boundary in the style of BASELINE configs 2, 3 and 5: N(0,1) activations,
    symbols uniform in [1, C), blank 0, per-utterance lengths."""
    rng = np.random.default_rng(seed)
    am = rng.standard_normal((B, T, C)).astype(dtype)
    lm = rng.standard_normal((B, S + 1, C)).astype(dtype)
    symbols = rng.integers(1, C, size=(B, S)).astype(np.int64)
    boundary = None
    if with_boundary:
        t_lo = T if t_lo is None else t_lo
        s_lo = S if s_lo is None else s_lo
        Tb = rng.integers(t_lo, T + 1, size=B)
        Sb = rng.integers(s_lo, S + 1, size=B)
        if modified:
            Sb = np.minimum(Sb, Tb)
        boundary = np.stack([np.zeros(B, np.int64), np.zeros(B, np.int64), Sb, Tb], axis=1).astype(np.int64)
    return dict(am=am, lm=lm, symbols=symbols, boundary=boundary, B=B, T=T, S=S, C=C)
