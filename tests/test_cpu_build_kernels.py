"""The library's HIP kernels, compiled for the host (tests/cpu_kernels.py) and run through their
C-ABI on numpy buffers that end at an inaccessible page: the same parity checks as the GPU tests
make, without a GPU, plus the certainty that no kernel reads or writes past the end of a tensor at
these shapes (that would end the run with a segmentation fault).  (The pipelined fp32
mutual-information kernels and the single launch: tests/test_cpu_build_pipelined.py.)

This is a second line behind the GPU tests, not a replacement: the host compiler is not hipcc,
every work-item is a thread here and the workgroups of a launch run one after the other."""
import ctypes
import os

import numpy as np
import pytest

import cases
import closed_forms as cf
import cpu_kernels as ck
from cpu_kernels import Fenced, fenced, p
from oracle import lattice as olat
from oracle import mi as omi
from oracle import rnnt as orn

TYPES = ["regular", "modified", "constrained"]
CODES = {"regular": 0, "modified": 1, "constrained": 2}
TOL = {np.dtype(np.float32): dict(rtol=1e-4, atol=1e-5), np.dtype(np.float64): dict(rtol=1e-10, atol=1e-10)}


@pytest.fixture(scope="module")
def lib():
    return ck.lib()


def dcode(dt):
    return 0 if np.dtype(dt) == np.float32 else 1


class Inputs:
    """Fenced copies of a call's input arrays, kept alive until the case is over (ctypes gets a
    bare address: an array that only lived inside the argument list would be gone by the call)."""

    def __init__(self, at="end"):
        self.kept, self.at = [], at

    def __call__(self, array):
        f = fenced(array, self.at)
        self.kept.append(f)
        return p(f)


# ---- the exact mutual-information kernels ------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_exact_mi_kernels_equal_the_cpu_loops_bit_for_bit(lib, dtype, modified):
    """mi_generic.hip follows k2's CPU loops term for term (mutual_information_cpu.cu:89-123,
    179-266); built for the host with the same libm, it has to give the same bits."""
    for seed in range(6):
        c = cases.mi_case(500 + seed, dtype=dtype, max_B=3, max_S=40, max_T=70,
                          force={"modified": modified, "rand_bd": seed % 3 != 0})
        px, py, bd = c["px"], c["py"], c["boundary"]
        B, S, T = c["B"], c["S"], c["T"]
        want_ans, want_p = omi.mi_forward(px, py, bd)
        want_gx, want_gy = omi.mi_backward(px, py, bd, want_p)
        fpx, fpy, fbd = fenced(px), fenced(py), fenced(bd)
        pp, ans = Fenced((B, S + 1, T + 1), dtype, fill=np.nan), Fenced((B,), dtype, fill=np.nan)
        assert lib.cpu_mi_forward_generic(p(fpx), p(fpy), p(fbd), p(pp), p(ans), B, S, T, int(modified),
                                          dcode(dtype)) == 0
        np.testing.assert_array_equal(ans.a, want_ans)
        box = np.array([[0, 0, S, T]] * B) if bd is None else bd
        for b in range(B):
            s0, t0, s1, t1 = box[b]
            np.testing.assert_array_equal(pp.a[b, s0:s1 + 1, t0:t1 + 1], want_p[b, s0:s1 + 1, t0:t1 + 1])
        gx, gy = Fenced(px.shape, dtype, fill=np.nan), Fenced(py.shape, dtype, fill=np.nan)
        ans_grad = Fenced((B,), dtype, fill=1.0)
        assert lib.cpu_mi_backward_generic(p(fpx), p(pp), p(fbd), p(ans_grad), p(gx), p(gy), B, S, T,
                                           int(modified), 1, dcode(dtype)) == 0
        np.testing.assert_array_equal(gx.a, want_gx)
        np.testing.assert_array_equal(gy.a, want_gy)
        for f in (pp, ans, gx, gy, ans_grad):
            assert f.intact()


def _exact_pair(lib, c, dtype, modified):
    """p, ans, px_grad, py_grad of the exact kernels on fenced buffers."""
    px, py, bd = c["px"], c["py"], c["boundary"]
    B, S, T = c["B"], c["S"], c["T"]
    fpx, fpy, fbd = fenced(px), fenced(py), fenced(bd)
    pp, ans = Fenced((B, S + 1, T + 1), dtype, fill=np.nan), Fenced((B,), dtype, fill=np.nan)
    assert lib.cpu_mi_forward_generic(p(fpx), p(fpy), p(fbd), p(pp), p(ans), B, S, T, int(modified),
                                      dcode(dtype)) == 0
    gx, gy = Fenced(px.shape, dtype, fill=np.nan), Fenced(py.shape, dtype, fill=np.nan)
    ans_grad = Fenced((B,), dtype, fill=1.0)
    assert lib.cpu_mi_backward_generic(p(fpx), p(pp), p(fbd), p(ans_grad), p(gx), p(gy), B, S, T,
                                       int(modified), 1, dcode(dtype)) == 0
    for f in (pp, ans, gx, gy, ans_grad):
        assert f.intact()
    return pp.a.copy(), ans.a.copy(), gx.a.copy(), gy.a.copy(), ans_grad.a.copy()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_exact_mi_kernels_without_lds_rows_give_the_same_bits(lib, dtype, modified, monkeypatch):
    """Sequences with more rows than LDS holds are swept with the previous step read back from p
    and from px_grad / py_grad (mi_generic_impl.h); K2AMD_MI_GENERIC_ROWS=global selects that
    form at any size.  Same bits as the CPU loops and as the form with the rows in LDS,
    -inf entries and boundaries included."""
    for seed in range(3):
        c = cases.mi_case(900 + seed, dtype=dtype, max_B=3, max_S=40, max_T=70,
                          force={"modified": modified, "rand_bd": seed % 3 != 0})
        if seed % 2:
            rng = np.random.default_rng(seed)
            for name in ("px", "py"):
                c[name][rng.random(c[name].shape) < 0.15] = -np.inf
        monkeypatch.delenv("K2AMD_MI_GENERIC_ROWS", raising=False)
        lds = _exact_pair(lib, c, dtype, modified)
        monkeypatch.setenv("K2AMD_MI_GENERIC_ROWS", "global")
        glob = _exact_pair(lib, c, dtype, modified)
        want_ans, want_p = omi.mi_forward(c["px"], c["py"], c["boundary"])
        want_gx, want_gy = omi.mi_backward(c["px"], c["py"], c["boundary"], want_p)
        np.testing.assert_array_equal(glob[1], want_ans)
        np.testing.assert_array_equal(glob[2], want_gx)
        np.testing.assert_array_equal(glob[3], want_gy)
        for a, b in zip(lds, glob):
            np.testing.assert_array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.parametrize("full", [False, pytest.param(True, marks=pytest.mark.skipif(
    os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1", reason="slow on the host: run with K2AMD_SLOW_CPU_TESTS=1"))])
@pytest.mark.parametrize("dtype,S", [(np.float32, 8200), (np.float64, 4100)])
def test_exact_mi_kernels_beyond_the_lds_rows(lib, dtype, S, full, monkeypatch):
    """Tensors with more rows than two LDS rows of 64 KiB hold (S > 8190 in fp32, 4094 in fp64):
    served, and with the bits of the CPU loops.  The quick form sweeps boxes of a hundred rows at
    either end of such a tensor (a barrier per step is what costs time on the host), the full
    form all rows."""
    monkeypatch.delenv("K2AMD_MI_GENERIC_ROWS", raising=False)
    rng = np.random.default_rng(S)
    B, T = 2, 2
    bd = None if full else np.array([[S - 100, 0, S, T], [3, 1, 90, T]], dtype=np.int64)
    c = {"B": B, "S": S, "T": T, "boundary": bd,
         "px": np.minimum(rng.normal(-2, 1, (B, S, T + 1)), 0).astype(dtype),
         "py": np.minimum(rng.normal(-2, 1, (B, S + 1, T)), 0).astype(dtype)}
    pp, ans, gx, gy, _ = _exact_pair(lib, c, dtype, False)
    want_ans, want_p = omi.mi_forward(c["px"], c["py"], bd)
    want_gx, want_gy = omi.mi_backward(c["px"], c["py"], bd, want_p)
    np.testing.assert_array_equal(ans, want_ans)
    np.testing.assert_array_equal(gx, want_gx)
    np.testing.assert_array_equal(gy, want_gy)
    for b in range(B):
        s0, t0, s1, t1 = (0, 0, S, T) if bd is None else bd[b]
        np.testing.assert_array_equal(pp[b, s0:s1 + 1, t0:t1 + 1], want_p[b, s0:s1 + 1, t0:t1 + 1])


# ---- the row kernels: get_rnnt_logprobs_joint / _pruned / HAT -----------------------------------

def _random_ranges(rng, B, T, S, R):
    start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1)
    start[:, 0] = 0
    start[:, -2:] = S - R + 1
    return (np.maximum.accumulate(start, axis=1)[:, :, None] + np.arange(R)).astype(np.int64)


# classes: fewer than a wavefront's lanes; 16-byte rows in registers; scalar rows in registers
# (odd length); beyond the register-resident rows (64 * 8) and vectorisable; beyond and not
ROW_CLASSES = [7, 64, 260, 71, 516, 1030, 1033]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_joint_builder(lib, rnnt_type, dtype):
    # (the stand-in pays for every workgroup of a launch, and the "constrained" pass launches
    # hundreds: the lattice types other than the regular one see three of the classes)
    for k, C in enumerate(ROW_CLASSES[:5] if rnnt_type == "regular" else ROW_CLASSES[2:4]):
        B, T, S = 2, 6 + k, 3
        c = cases.rnnt_case(600 + k, B, T, S, C, dtype=dtype, t_lo=4, s_lo=2, modified=rnnt_type != "regular")
        rng = np.random.default_rng(610 + k)
        at = "start" if rnnt_type == "constrained" else "end"  # the fence in front of the tensors for one type
        keep = Inputs(at)
        logits = (3 * rng.standard_normal((B, T, S + 1, C))).astype(dtype)
        sym, bd = c["symbols"], c["boundary"] if k % 2 == 0 else None
        T1 = T + 1 if rnnt_type == "regular" else T
        fl, fs, fb = fenced(logits, at), fenced(sym, at), fenced(bd, at)
        px, py = Fenced((B, S, T1), dtype, np.nan, at), Fenced((B, S + 1, T), dtype, np.nan, at)
        norm = Fenced((B, T, S + 1), dtype, np.nan, at)
        assert lib.k2amd_rnnt_logprobs_joint_forward(p(fl), p(fs), p(fb), p(px), p(py), p(norm), B, S, T, C, 0,
                                                     CODES[rnnt_type], dcode(dtype), None) == 0
        wpx, wpy = orn.logprobs_joint(logits, sym, 0, rnnt_type, bd)
        np.testing.assert_allclose(px.a, wpx, **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(py.a, wpy, **TOL[np.dtype(dtype)])
        _, gx, gy = omi.mi(wpx.astype(np.float64), wpy.astype(np.float64), bd)
        w = np.linspace(0.5, 1.5, B)
        want = cf.joint_logits_grad(logits, sym, 0, gx, gy, -w, rnnt_type)  # of sum_b w[b] score[b]
        grad = Fenced(logits.shape, dtype, np.nan, at)
        assert lib.k2amd_rnnt_logprobs_joint_backward(
            p(fl), p(norm), keep(gx.astype(dtype)), keep(gy.astype(dtype)), keep(w.astype(dtype)),
            p(fs), p(fb), p(grad), B, S, T, C, 0, CODES[rnnt_type], dcode(dtype), None) == 0
        np.testing.assert_allclose(grad.a, want, **(dict(rtol=1e-8, atol=1e-10) if dtype == np.float64
                                                    else dict(rtol=1e-3, atol=1e-5)))
        for f in (px, py, norm, grad):
            assert f.intact()


@pytest.mark.parametrize("hat", [False, True])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_pruned_builders(lib, rnnt_type, dtype, hat):
    for k, C in enumerate(ROW_CLASSES[::2] + ROW_CLASSES[5:6] if rnnt_type == "regular" else ROW_CLASSES[1:6:2]):
        B, T, S, R = 2, 9 + k, 5, 1 + k % 4
        c = cases.rnnt_case(620 + k, B, T, S, C, dtype=dtype, t_lo=7, s_lo=3, modified=rnnt_type != "regular")
        rng = np.random.default_rng(630 + k)
        at = "start" if rnnt_type == "constrained" else "end"
        keep = Inputs(at)
        logits = (3 * rng.standard_normal((B, T, R, C))).astype(dtype)
        ranges = _random_ranges(rng, B, T, S, R)
        sym, bd = c["symbols"], c["boundary"] if k % 2 == 0 else None
        T1 = T + 1 if rnnt_type == "regular" else T
        fl, fs, fr, fb = fenced(logits, at), fenced(sym, at), fenced(ranges, at), fenced(bd, at)
        px, py = Fenced((B, S, T1), dtype, np.nan, at), Fenced((B, S + 1, T), dtype, np.nan, at)
        norm = Fenced((B, T, R), dtype, np.nan, at)
        code, dc = CODES[rnnt_type], dcode(dtype)
        if hat:
            assert lib.k2amd_rnnt_hat_logprobs_pruned_forward(p(fl), p(fs), p(fr), p(fb), p(px), p(py), p(norm),
                                                              B, S, T, R, C, code, dc, None) == 0
        else:
            assert lib.k2amd_rnnt_logprobs_pruned_forward(p(fl), p(fs), p(fr), p(fb), p(px), p(py), p(norm),
                                                          B, S, T, R, C, 0, code, dc, None) == 0
        builder = orn.hat_logprobs_pruned if hat else orn.logprobs_pruned
        wpx, wpy = builder(logits, sym, ranges, 0, bd, rnnt_type)
        np.testing.assert_allclose(px.a, wpx, **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(py.a, wpy, **TOL[np.dtype(dtype)])
        # any gradients will do for the backward's formulas; these are smooth and nowhere zero
        gx = rng.uniform(0.1, 1.0, wpx.shape)
        gy = rng.uniform(0.1, 1.0, wpy.shape)
        w = np.linspace(0.5, 1.5, B)
        if rnnt_type == "regular":
            gx[:, :, T] = 0.0
            if bd is not None:
                for b in range(B):
                    gx[b, :, bd[b, 3]] = 0.0  # the builder wrote -inf there: nothing flows back
        want = cf.pruned_logits_grad(logits, sym, ranges, 0, gx, gy, -w, rnnt_type, hat=hat)
        grad = Fenced(logits.shape, dtype, np.nan, at)
        args = (p(fl), p(norm), keep(gx.astype(dtype)), keep(gy.astype(dtype)), keep(w.astype(dtype)),
                p(fs), p(fr), p(fb), p(grad), B, S, T, R, C)
        if hat:
            assert lib.k2amd_rnnt_hat_logprobs_pruned_backward(*args, code, dc, None) == 0
        else:
            assert lib.k2amd_rnnt_logprobs_pruned_backward(*args, 0, code, dc, None) == 0
        np.testing.assert_allclose(grad.a, want, **(dict(rtol=1e-8, atol=1e-10) if dtype == np.float64
                                                    else dict(rtol=1e-3, atol=1e-5)))
        for f in (px, py, norm, grad):
            assert f.intact()


# ---- prune ranges, the pruning gather and its gradient ------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_prune_ranges_bit_exact(lib, dtype, modified):
    rt = "modified" if modified else "regular"
    for k, (B, T, S, R) in enumerate(((2, 9, 5, 3), (1, 70, 20, 5), (3, 33, 33, 7), (2, 130, 4, 5), (1, 5, 1, 2))):
        c = cases.rnnt_case(640 + k, B, T, S, 6, dtype=dtype, t_lo=max(S, T - 3), s_lo=max(1, S - 2), modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        want = orn.prune_ranges(gx, gy, c["boundary"], R)
        keep = Inputs()
        r_final = want.shape[2]
        out = Fenced((B, T, r_final), np.int64, fill=-7)
        assert lib.k2amd_rnnt_prune_ranges(keep(gx), keep(gy), keep(c["boundary"]), p(out), B, S, T,
                                           int(modified), r_final, dcode(dtype), None) == 0
        np.testing.assert_array_equal(out.a, want)
        assert out.intact()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("modified", [False, True])
def test_deprecated_prune_ranges_bit_exact(lib, dtype, modified):
    """k2amd_rnnt_prune_ranges_deprecated against the oracle's restatement of
    get_rnnt_prune_ranges_deprecated (rnnt_loss.py:786-910), which the reference's recorded
    ranges pin (tests/test_oracle_rnnt_fixtures.py): prefix sums accumulated in double and rounded
    once, differences in the input type, first maximum."""
    rt = "modified" if modified else "regular"
    for k, (B, T, S, R) in enumerate(((2, 9, 5, 3), (1, 70, 20, 5), (3, 33, 33, 7), (2, 300, 4, 5), (1, 5, 1, 2),
                                      (2, 40, 6, 7), (2, 12, 3, 1 if modified else 2))):
        c = cases.rnnt_case(680 + k, B, T, S, 6, dtype=dtype, t_lo=max(S, T - 3), s_lo=max(1, S - 2), modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        want = orn.prune_ranges_deprecated(gx, gy, c["boundary"], R)
        keep = Inputs()
        r_final = want.shape[2]
        out = Fenced((B, T, r_final), np.int64, fill=-7)
        assert lib.k2amd_rnnt_prune_ranges_deprecated(keep(gx), keep(gy), keep(c["boundary"]), p(out), B, S, T,
                                                      int(modified), r_final, dcode(dtype), None) == 0
        np.testing.assert_array_equal(out.a, want)
        assert out.intact()
    # sums that tie or differ in the last bits: rows of equal occupation
    rng = np.random.default_rng(689)
    B, T, S, R = 2, 50, 12, 3
    T1 = T if modified else T + 1
    gx = rng.integers(0, 3, (B, S, T1)).astype(dtype) * dtype(0.1)
    gy = rng.integers(0, 3, (B, S + 1, T)).astype(dtype) * dtype(0.1)
    bd = np.array([[0, 0, S, T], [0, 0, S - 1, T - 4]], dtype=np.int64)
    want = orn.prune_ranges_deprecated(gx, gy, bd, R)
    keep = Inputs()
    out = Fenced((B, T, R), np.int64, fill=-7)
    assert lib.k2amd_rnnt_prune_ranges_deprecated(keep(gx), keep(gy), keep(bd), p(out), B, S, T, int(modified),
                                                  R, dcode(dtype), None) == 0
    np.testing.assert_array_equal(out.a, want)


@pytest.mark.parametrize("modified", [False, True])
def test_prune_ranges_scans_inside_ranges_give_the_same_integers(lib, modified, monkeypatch):
    """Where two rows of T ints exceed LDS the finishing kernel's scans run in the halves of
    ranges[b][t][0] (prune.hip); K2AMD_PRUNE_SCAN_ROWS=global selects that at any T.  s_range = 1
    is the case in which a frame owns nothing but that one word."""
    monkeypatch.setenv("K2AMD_PRUNE_SCAN_ROWS", "global")
    rt = "modified" if modified else "regular"
    for k, (B, T, S, R) in enumerate(((2, 9, 5, 3), (1, 70, 20, 5), (3, 300, 33, 7), (2, 130, 4, 1), (1, 5, 1, 2), (2, 1, 1, 2))):
        c = cases.rnnt_case(660 + k, B, T, S, 6, dtype=np.float32, t_lo=max(S, T - 3), s_lo=max(1, S - 2), modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        want = orn.prune_ranges(gx, gy, c["boundary"], R)
        keep = Inputs()
        r_final = want.shape[2]
        out = Fenced((B, T, r_final), np.int64, fill=-7)
        assert lib.k2amd_rnnt_prune_ranges(keep(gx), keep(gy), keep(c["boundary"]), p(out), B, S, T,
                                           int(modified), r_final, 0, None) == 0
        np.testing.assert_array_equal(out.a, want)
        assert out.intact()


def test_prune_ranges_with_more_frames_than_lds_rows_hold(lib, monkeypatch):
    """T = 8300 frames (two rows of T ints no longer fit 64 KiB): served, same integers as the
    oracle.  Occupation counts drawn at random stand in for a recursion's gradients: the ranges
    are a function of these two tensors and the boundary alone."""
    monkeypatch.delenv("K2AMD_PRUNE_SCAN_ROWS", raising=False)
    rng = np.random.default_rng(83)
    B, T, S, R = 2, 8300, 6, 3
    gx = rng.random((B, S, T + 1)).astype(np.float32)
    gy = rng.random((B, S + 1, T)).astype(np.float32)
    bd = np.array([[0, 0, S, T], [0, 0, S - 2, T - 11]], dtype=np.int64)
    want = orn.prune_ranges(gx, gy, bd, R)
    keep = Inputs()
    out = Fenced((B, T, R), np.int64, fill=-7)
    assert lib.k2amd_rnnt_prune_ranges(keep(gx), keep(gy), keep(bd), p(out), B, S, T, 0, R, 0, None) == 0
    np.testing.assert_array_equal(out.a, want)
    assert out.intact()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_prune_gather_and_its_gradient(lib, dtype):
    rng = np.random.default_rng(650)
    for B, S1, T, R, D in ((2, 6, 9, 3, 8), (1, 21, 40, 5, 70), (3, 4, 3, 4, 129), (2, 9, 300, 2, 5)):
        lm = rng.standard_normal((B, S1, D)).astype(dtype)
        keep = Inputs()
        ranges = _random_ranges(rng, B, T, S1 - 1, R)
        out = Fenced((B, T, R, D), dtype, fill=np.nan)
        fr = fenced(ranges)
        assert lib.k2amd_rnnt_prune_gather(keep(lm), p(fr), p(out), B, S1, T, R, D, dcode(dtype), None) == 0
        want = lm[np.arange(B)[:, None, None], ranges]
        np.testing.assert_array_equal(out.a, want)
        g = rng.standard_normal((B, T, R, D)).astype(dtype)
        lm_grad = Fenced((B, S1, D), dtype, fill=np.nan)
        assert lib.k2amd_rnnt_prune_gather_backward(keep(g), p(fr), p(lm_grad), B, S1, T, R, D, dcode(dtype),
                                                    None) == 0
        want_g = np.zeros((B, S1, D), np.float64)
        for b in range(B):
            np.add.at(want_g[b], ranges[b].reshape(-1), g[b].reshape(-1, D).astype(np.float64))
        np.testing.assert_allclose(lm_grad.a, want_g, **(dict(rtol=1e-12, atol=1e-12) if dtype == np.float64
                                                         else dict(rtol=1e-5, atol=1e-5)))
        assert out.intact() and lm_grad.intact()


# ---- pruned_ranges_to_lattice -------------------------------------------------------------------

def _lattice(lib, ranges, frames, symbols, logits):
    B, T, R = ranges.shape
    S, C = symbols.shape[1], logits.shape[3]
    keep = Inputs()
    arc_local = Fenced((B, T * R + 1), np.int32, fill=-1)
    seq_arcs = Fenced((max(B, 1),), np.int32, fill=-1)
    state_splits, arc_base = Fenced((B + 1,), np.int32, fill=-1), Fenced((B + 1,), np.int32, fill=-1)
    fr, ff = fenced(ranges), fenced(frames)
    assert lib.k2amd_lattice_count(p(fr), p(ff), p(arc_local), p(seq_arcs), p(state_splits), p(arc_base), B, T, R,
                                   None) == 0
    n_states, n_arcs = int(state_splits.a[B]), int(arc_base.a[B])
    arc_splits = Fenced((n_states + 1,), np.int32, fill=-1)
    arcs, arc_map = Fenced((n_arcs, 4), np.int32, fill=-1), Fenced((n_arcs,), np.int32, fill=-1)
    code = {np.dtype(np.float32): 0, np.dtype(np.float64): 1, np.dtype(np.float16): 2}[logits.dtype]
    strides = (ctypes.c_int64 * 4)(*[s // logits.itemsize for s in logits.strides])
    assert lib.k2amd_lattice_fill(p(fr), p(ff), keep(symbols), keep(logits), ctypes.addressof(strides),
                                  p(state_splits), p(arc_base), p(arc_local), p(arc_splits), p(arcs), p(arc_map),
                                  B, T, R, S, C, code, None) == 0
    for f in (arc_local, seq_arcs, state_splits, arc_base, arc_splits, arcs, arc_map):
        assert f.intact()
    return state_splits.a, arc_splits.a, arcs.a, arc_map.a


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_lattice_golden_vectors_and_random_bands(lib, dtype):
    """The reference test's vectors (pruned_ranges_to_lattice_test.py:45-205) and random bands
    against the oracle, bit for bit."""
    from test_oracle_lattice import golden_case
    g = golden_case(dtype)
    todo = [(g["ranges"], g["frames"], g["symbols"], g["logits"])]
    rng = np.random.default_rng(660)
    for B, T, S, R, C in ((2, 7, 5, 3, 6), (1, 1, 1, 2, 3), (3, 20, 9, 4, 11)):
        ranges = _random_ranges(rng, B, T, S, R).astype(np.int32)
        frames = rng.integers(max(1, T - 3), T + 1, B).astype(np.int32)
        todo.append((ranges, frames, rng.integers(1, C, (B, S)).astype(np.int64),
                     rng.standard_normal((B, T, R, C)).astype(dtype)))
    for k, (ranges, frames, symbols, logits) in enumerate(todo):
        state_splits, arc_splits, arcs, scores, arc_map = olat.pruned_ranges_to_lattice(ranges, frames, symbols, logits)
        got = _lattice(lib, ranges, frames, symbols, logits)
        np.testing.assert_array_equal(got[0], state_splits)
        np.testing.assert_array_equal(got[1], arc_splits)
        np.testing.assert_array_equal(got[2][:, :3], arcs)
        np.testing.assert_array_equal(got[2][:, 3].copy().view(np.float32), scores.astype(np.float32))
        np.testing.assert_array_equal(got[3], arc_map)
        if k == 0:  # the reference's own expectations
            np.testing.assert_array_equal(got[3], g["arc_map"])
            np.testing.assert_array_equal(got[2][:, :3], g["arcs"])


# ---- the split of the joint recursion's score ---------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_joint_products(lib, dtype):
    rng = np.random.default_rng(670)
    for N, B, S, T in ((2, 2, 5, 9), (1, 1, 1, 1), (8, 1, 17, 40)):
        pxs = [np.minimum(rng.standard_normal((B, S, T + 1)) - 2, 0).astype(dtype) for _ in range(N)]
        pys = [np.minimum(rng.standard_normal((B, S + 1, T)) - 2, 0).astype(dtype) for _ in range(N)]
        pxs[0][0, 0, 0] = -np.inf  # clamped at the dtype's lowest value before the product
        gx, gy = rng.uniform(0, 1, (B, S, T + 1)).astype(dtype), rng.uniform(0, 1, (B, S + 1, T)).astype(dtype)
        fx, fy = [fenced(a) for a in pxs], [fenced(a) for a in pys]
        keep = Inputs()
        xs = (ctypes.c_void_p * N)(*[f.a.ctypes.data for f in fx])
        ys = (ctypes.c_void_p * N)(*[f.a.ctypes.data for f in fy])
        prods = Fenced((N, B), dtype, fill=np.nan)
        scratch = Fenced((lib.k2amd_mi_joint_products_scratch_elements(N, B),), dtype, fill=np.nan)
        assert lib.k2amd_mi_joint_products(ctypes.addressof(xs), ctypes.addressof(ys), N, keep(gx), keep(gy),
                                           p(prods), p(scratch), B, S * (T + 1), (S + 1) * T, dcode(dtype), None) == 0
        lowest = np.finfo(dtype).min
        want = np.array([[(np.maximum(pxs[n][b], lowest).astype(np.float64) * gx[b]).sum()
                          + (np.maximum(pys[n][b], lowest).astype(np.float64) * gy[b]).sum() for b in range(B)]
                         for n in range(N)])
        np.testing.assert_allclose(prods.a, want, **(dict(rtol=1e-12) if dtype == np.float64 else dict(rtol=2e-5)))
        assert prods.intact() and scratch.intact()


# ---- get_rnnt_logprobs (rnnt_simple.hip) and the smoothed builder on top of it ------------------

def _simple_forward(lib, c, rnnt_type, bd, at="end"):
    lm, am, sym = c["lm"], c["am"], c["symbols"]
    dt = lm.dtype
    B, T, C = am.shape
    S = lm.shape[1] - 1
    T1 = T + 1 if rnnt_type == "regular" else T
    out = dict(px=Fenced((B, S, T1), dt, np.nan, at), py=Fenced((B, S + 1, T), dt, np.nan, at),
               lm_probs=Fenced(lm.shape, dt, np.nan, at), am_probs=Fenced(am.shape, dt, np.nan, at),
               lm_max=Fenced((B, S + 1), dt, np.nan, at), am_max=Fenced((B, T), dt, np.nan, at),
               denom=Fenced((B, S + 1, T), dt, np.nan, at),
               lm=fenced(lm, at), am=fenced(am, at), sym=fenced(sym, at), bd=fenced(bd, at))
    assert lib.k2amd_rnnt_logprobs_simple_forward(
        p(out["lm"]), p(out["am"]), p(out["sym"]), p(out["bd"]), p(out["px"]), p(out["py"]), p(out["lm_probs"]),
        p(out["am_probs"]), p(out["lm_max"]), p(out["am_max"]), p(out["denom"]), B, S, T, C, 0, CODES[rnnt_type],
        dcode(dt), None) == 0
    for k in ("px", "py", "lm_probs", "am_probs", "lm_max", "am_max", "denom"):
        assert out[k].intact(), k
    return out


def _simple_backward(lib, f, gx, gy, w, rnnt_type, at="end"):
    dt = f["lm"].a.dtype
    B, T, C = f["am"].a.shape
    S = f["lm"].a.shape[1] - 1
    keep = Inputs(at)
    lm_grad, am_grad = Fenced(f["lm"].a.shape, dt, np.nan, at), Fenced(f["am"].a.shape, dt, np.nan, at)
    n = lib.k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, T)
    q = Fenced((n,), dt, np.nan, at)
    args = (keep(gx.astype(dt)), keep(gy.astype(dt)), None if w is None else keep(w.astype(dt)), p(f["sym"]),
            p(f["bd"]), p(f["lm_probs"]), p(f["am_probs"]), p(f["denom"]), p(lm_grad), p(am_grad), p(q))
    dims = (B, S, T, C, 0, CODES[rnnt_type], dcode(dt), None)
    if n > 0:
        assert lib.k2amd_rnnt_logprobs_simple_backward(*args, n - 1, *dims) == 3  # too little scratch: refused
        assert np.isnan(lm_grad.a).all()
    assert lib.k2amd_rnnt_logprobs_simple_backward(*args, n, *dims) == 0
    assert lm_grad.intact() and am_grad.intact() and q.intact()
    return lm_grad, am_grad


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_simple_builder(lib, rnnt_type, dtype):
    """Forward against the oracle, backward against the closed form; fp32 through the emulated
    matrix instruction (the kernel for small products), fp64 on the vector path."""
    at = "start" if rnnt_type == "constrained" else "end"
    for k, (B, T, S, C) in enumerate(((2, 9, 4, 7), (1, 70, 33, 70), (3, 33, 0, 5))):
        c = cases.rnnt_case(700 + k, B, T, S, C, dtype=dtype, t_lo=max(S, T - 3), s_lo=max(0, S - 2),
                            modified=rnnt_type != "regular")
        if S > 1:
            c["symbols"][:, 1] = c["symbols"][:, 0]
        bd = c["boundary"] if k != 1 else None
        f = _simple_forward(lib, c, rnnt_type, bd, at)
        wpx, wpy = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rnnt_type, bd)
        np.testing.assert_allclose(f["px"].a, wpx, **TOL[np.dtype(dtype)])
        np.testing.assert_allclose(f["py"].a, wpy, **TOL[np.dtype(dtype)])
        _, gx, gy = omi.mi(wpx.astype(np.float64), wpy.astype(np.float64), bd)
        w = np.linspace(0.5, 1.5, B)
        want_lm, want_am = cf.simple_grads(c["lm"], c["am"], c["symbols"], 0, gx, gy, -w, rnnt_type)
        lm_grad, am_grad = _simple_backward(lib, f, gx, gy, w, rnnt_type, at)
        tol = dict(rtol=1e-8, atol=1e-10) if dtype == np.float64 else dict(rtol=1e-3, atol=1e-5)
        np.testing.assert_allclose(lm_grad.a, want_lm, **tol)
        np.testing.assert_allclose(am_grad.a, want_am, **tol)


def test_simple_builder_without_frames(lib):
    """T = 0: px is its one -inf column, the lm gradient all zeros; the backward needs no scratch
    and takes a null pointer for it."""
    B, S, C = 2, 3, 5
    c = cases.rnnt_case(710, B, 0, S, C, dtype=np.float32, with_boundary=False)
    f = _simple_forward(lib, c, "regular", None)
    assert np.isneginf(f["px"].a).all()
    lm_grad = Fenced(c["lm"].shape, np.float32, np.nan)
    assert lib.k2amd_rnnt_logprobs_simple_backward_scratch_elements(B, S, 0) == 0
    assert lib.k2amd_rnnt_logprobs_simple_backward(None, None, None, p(f["sym"]), None, p(f["lm_probs"]), None, None,
                                                   p(lm_grad), None, None, 0, B, S, 0, C, 0, 0, 0, None) == 0
    assert (lm_grad.a == 0).all() and lm_grad.intact()


@pytest.mark.skipif(os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1",
                    reason="ten minutes on eight cores: run with K2AMD_SLOW_CPU_TESTS=1")
def test_simple_builder_lds_tiled_products(lib):
    """A shape large enough for the 64 x 64 LDS-tiled product kernel (it takes over at 512 tiles):
    the forward product (both operands contiguous along k) and the am-gradient product (neither).
    Hundreds of workgroups of 256 threads each: slow on the host, so not part of the default run."""
    B, T, S, C = 16, 1000, 127, 130
    c = cases.rnnt_case(720, B, T, S, C, dtype=np.float32, t_lo=900, s_lo=100)
    f = _simple_forward(lib, c, "regular", c["boundary"])
    wpx, wpy = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, "regular", c["boundary"])
    np.testing.assert_allclose(f["px"].a, wpx, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(f["py"].a, wpy, rtol=1e-4, atol=1e-5)
    rng = np.random.default_rng(721)
    gx, gy = rng.uniform(0, 1e-2, wpx.shape), rng.uniform(0, 1e-2, wpy.shape)
    gx[:, :, T] = 0.0
    for b in range(B):
        gx[b, :, c["boundary"][b, 3]] = 0.0
    lm_grad, am_grad = _simple_backward(lib, f, gx, gy, None, "regular")
    for b in (0, B - 1):  # the closed form holds a [S+1][T][C] tensor per sequence: two of them will do
        one = {k: c[k][b:b + 1] for k in ("lm", "am", "symbols")}
        want_lm, want_am = cf.simple_grads(one["lm"], one["am"], one["symbols"], 0, gx[b:b + 1], gy[b:b + 1],
                                           -np.ones(1), "regular")
        np.testing.assert_allclose(lm_grad.a[b:b + 1], want_lm, rtol=1e-3, atol=1e-5)
        np.testing.assert_allclose(am_grad.a[b:b + 1], want_am, rtol=1e-3, atol=1e-5)


@pytest.mark.parametrize("rnnt_type", TYPES)
def test_smoothed_chain_end_to_end(lib, rnnt_type):
    """The two calls per direction that make up get_rnnt_logprobs_smoothed, all in the kernels:
    simple builder without a boundary, mix; simple builder's backward with the scaled weights,
    marginal terms added.  Against the oracle and the closed-form gradients."""
    B, T, S, C = 3, 11, 6, 70
    scales = (0.25, 0.1)
    c = cases.rnnt_case(730, B, T, S, C, dtype=np.float64, t_lo=8, s_lo=3, modified=rnnt_type != "regular")
    bd = c["boundary"]
    f = _simple_forward(lib, c, "regular" if rnnt_type == "regular" else "modified", None)
    T1 = T + 1 if rnnt_type == "regular" else T
    dt = np.float64
    px, py = Fenced((B, S, T1), dt, np.nan), Fenced((B, S + 1, T), dt, np.nan)
    lm_norm, am_norm, unigram = Fenced((B, S + 1), dt, np.nan), Fenced((B, T), dt, np.nan), Fenced((2, C), dt, np.nan)
    n = lib.k2amd_rnnt_smoothed_scratch_elements(B, S, T, C)
    scratch, fbd = Fenced((n,), dt, np.nan), fenced(bd)
    dims = (B, S, T, C, 0, CODES[rnnt_type], 1, None)
    assert lib.k2amd_rnnt_smoothed_forward(
        p(f["lm"]), p(f["am"]), p(f["sym"]), p(fbd), p(f["lm_probs"]), p(f["am_probs"]), p(f["lm_max"]),
        p(f["am_max"]), p(f["px"]), p(f["py"]), p(px), p(py), p(lm_norm), p(am_norm), p(unigram), p(scratch), n,
        *scales, *dims) == 0
    wpx, wpy = orn.logprobs_smoothed(c["lm"], c["am"], c["symbols"], 0, scales[0], scales[1], bd, rnnt_type)
    np.testing.assert_allclose(px.a, wpx, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(py.a, wpy, rtol=1e-10, atol=1e-10)
    _, gx, gy = omi.mi(wpx, wpy, bd)
    w = np.linspace(0.5, 1.5, B)
    f["bd"] = fbd  # the backward of the joint term sees the real boundary and lattice type
    lm_grad, am_grad = _simple_backward(lib, f, gx, gy, w * (1.0 - scales[0] - scales[1]), rnnt_type)
    keep = Inputs()
    assert lib.k2amd_rnnt_smoothed_backward(
        keep(gx), keep(gy), keep(w), p(f["sym"]), p(fbd), p(f["lm_probs"]), p(f["am_probs"]), p(f["lm_max"]),
        p(f["am_max"]), p(lm_norm), p(am_norm), p(unigram), p(lm_grad), p(am_grad), p(scratch), n, *scales,
        *dims) == 0
    want_lm, want_am = cf.smoothed_grads(c["lm"], c["am"], c["symbols"], 0, scales[0], scales[1], gx, gy, -w, rnnt_type)
    np.testing.assert_allclose(lm_grad.a, want_lm, rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(am_grad.a, want_am, rtol=1e-8, atol=1e-10)
