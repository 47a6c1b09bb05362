"""Random small shapes through the host build of the kernels (tests/cpu_kernels.py), fixed seeds:
degenerate lattices (S = 0, T = 1, s_range = S + 1, one to three classes), symbols outside the
vocabulary, boundaries that leave one row or one column, -inf inputs; buffers fenced at either
end.  The same generators ran for ten minutes each with other seeds while this was written (335
row / simple-builder cases, 1421 prune-ranges / lattice cases, 306 recursion cases) without a
failure; what runs by default is a slice of that (K2AMD_SLOW_CPU_TESTS=1 runs five times as
many cases)."""
import os

import numpy as np
import pytest

import cases
import closed_forms as cf
import cpu_kernels as ck
import test_cpu_build_kernels as t
from cpu_kernels import Fenced, fenced, p
from oracle import lattice as olat
from oracle import mi as omi
from oracle import rnnt as orn

CODES = t.CODES
MORE = 5 if os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") == "1" else 1


@pytest.fixture(scope="module")
def lib():
    return ck.lib()


def test_row_builders_and_simple_builder_on_random_small_shapes(lib):
    rng = np.random.default_rng(11)
    for n in range(12 * MORE):
        rnnt_type = ["regular", "modified", "constrained"][rng.integers(3)]
        dtype = [np.float32, np.float64][rng.integers(2)]
        S = int(rng.integers(0, 7)); T = int(rng.integers(max(S, 1), 12)); B = int(rng.integers(1, 4))
        C = int(rng.choice([1, 2, 3, 4, 5, 8, 63, 64, 65, 130, 257, 513]))
        R = int(rng.integers(1, S + 2))
        hat = bool(rng.integers(2)) and C >= 2
        at = ["end", "start"][rng.integers(2)]
        desc = dict(rt=rnnt_type, dt=dtype.__name__, B=B, S=S, T=T, C=C, R=R, hat=hat, at=at)
        c = cases.rnnt_case(int(rng.integers(1 << 30)), B, T, S, max(C, 2), dtype=dtype, t_lo=max(S, 1), s_lo=0, modified=rnnt_type != "regular")
        sym = (c["symbols"] % C).astype(np.int64) if C >= 1 else c["symbols"]
        if rng.integers(4) == 0 and S > 0: sym[0, 0] = C + 3   # outside the vocabulary
        bd = c["boundary"] if rng.integers(3) else None
        if bd is not None and rnnt_type != "regular":
            bd[:, 2] = np.minimum(bd[:, 2], bd[:, 3])
        blank = int(rng.integers(C)) if not hat else 0
        code, dc = CODES[rnnt_type], t.dcode(dtype)
        T1 = T + 1 if rnnt_type == "regular" else T
        # pruned / hat
        logits = (3 * rng.standard_normal((B, T, R, C))).astype(dtype)
        start = np.sort(rng.integers(0, S - R + 2, (B, T)), axis=1); start[:, 0] = 0
        if T >= 2: start[:, -2:] = S - R + 1
        else: start[:, -1:] = 0 if S - R + 1 < 0 else start[:, -1:]
        ranges = (np.maximum.accumulate(start, axis=1)[:, :, None] + np.arange(R)).astype(np.int64)
        keep = t.Inputs(at)
        fl, fs, fr, fb = fenced(logits, at), fenced(sym, at), fenced(ranges, at), fenced(bd, at)
        px, py = Fenced((B, S, T1), dtype, np.nan, at), Fenced((B, S + 1, T), dtype, np.nan, at)
        norm = Fenced((B, T, R), dtype, np.nan, at)
        if hat:
            st = lib.k2amd_rnnt_hat_logprobs_pruned_forward(p(fl), p(fs), p(fr), p(fb), p(px), p(py), p(norm), B, S, T, R, C, code, dc, None)
        else:
            st = lib.k2amd_rnnt_logprobs_pruned_forward(p(fl), p(fs), p(fr), p(fb), p(px), p(py), p(norm), B, S, T, R, C, blank, code, dc, None)
        assert st == 0, st
        valid = (sym >= 0) & (sym < C)
        if valid.all():
            builder = orn.hat_logprobs_pruned if hat else orn.logprobs_pruned
            wpx, wpy = builder(logits, sym, ranges, blank, bd, rnnt_type)
            tol = t.TOL[np.dtype(dtype)]
            np.testing.assert_allclose(px.a, wpx, **tol); np.testing.assert_allclose(py.a, wpy, **tol)
            gx = rng.uniform(0.1, 1.0, wpx.shape); gy = rng.uniform(0.1, 1.0, wpy.shape)
            if rnnt_type == "regular":
                gx[:, :, T] = 0.0
                if bd is not None:
                    for b in range(B): gx[b, :, bd[b, 3]] = 0.0
            w = np.linspace(0.5, 1.5, B)
            want = cf.pruned_logits_grad(logits, sym, ranges, blank, gx, gy, -w, rnnt_type, hat=hat)
            grad = Fenced(logits.shape, dtype, np.nan, at)
            args = (p(fl), p(norm), keep(gx.astype(dtype)), keep(gy.astype(dtype)), keep(w.astype(dtype)), p(fs), p(fr), p(fb), p(grad), B, S, T, R, C)
            st = lib.k2amd_rnnt_hat_logprobs_pruned_backward(*args, code, dc, None) if hat else lib.k2amd_rnnt_logprobs_pruned_backward(*args, blank, code, dc, None)
            assert st == 0
            np.testing.assert_allclose(grad.a, want, **(dict(rtol=1e-8, atol=1e-10) if dtype == np.float64 else dict(rtol=1e-3, atol=1e-5)))
        # simple builder forward + backward
        cc = dict(c); cc["symbols"] = sym
        if C >= 1 and valid.all():
            cc["lm"] = c["lm"][:, :, :C].copy(); cc["am"] = c["am"][:, :, :C].copy()
            f = t._simple_forward(lib, cc, rnnt_type, bd, at)
            wpx, wpy = orn.logprobs_simple(cc["lm"], cc["am"], sym, 0 if hat else blank, rnnt_type, bd) if False else orn.logprobs_simple(cc["lm"], cc["am"], sym, 0, rnnt_type, bd)
            np.testing.assert_allclose(f["px"].a, wpx, **t.TOL[np.dtype(dtype)])
            np.testing.assert_allclose(f["py"].a, wpy, **t.TOL[np.dtype(dtype)])
            gx = rng.uniform(0.1, 1.0, wpx.shape); gy = rng.uniform(0.1, 1.0, wpy.shape)
            if rnnt_type == "regular":
                gx[:, :, T] = 0.0
                if bd is not None:
                    for b in range(B): gx[b, :, bd[b, 3]] = 0.0
            w = np.linspace(0.5, 1.5, B)
            want_lm, want_am = cf.simple_grads(cc["lm"], cc["am"], sym, 0, gx, gy, -w, rnnt_type)
            lm_g, am_g = t._simple_backward(lib, f, gx, gy, w, rnnt_type, at)
            tol = dict(rtol=1e-8, atol=1e-10) if dtype == np.float64 else dict(rtol=1e-3, atol=1e-5)
            np.testing.assert_allclose(lm_g.a, want_lm, **tol); np.testing.assert_allclose(am_g.a, want_am, **tol)


def test_prune_ranges_and_lattice_on_random_small_shapes(lib):
    rng = np.random.default_rng(12)
    for n in range(30 * MORE):
        modified = bool(rng.integers(2)); dtype = [np.float32, np.float64][rng.integers(2)]
        S = int(rng.integers(1, 12)); T = int(rng.integers(max(S, 2), 80)); B = int(rng.integers(1, 4))
        R = int(rng.integers(1 if modified else 2, S + 2))
        rt = "modified" if modified else "regular"
        c = cases.rnnt_case(int(rng.integers(1 << 30)), B, T, S, 5, dtype=dtype, t_lo=max(S, T // 2), s_lo=max(1, S // 2), modified=modified)
        px, py = orn.logprobs_simple(c["lm"], c["am"], c["symbols"], 0, rt, c["boundary"])
        _, gx, gy = omi.mi(px, py, c["boundary"])
        if rng.integers(3) == 0:  # ties: quantised gradients
            gx, gy = (np.round(gx * 4) / 4).astype(dtype), (np.round(gy * 4) / 4).astype(dtype)
        want = orn.prune_ranges(gx, gy, c["boundary"], R)
        r_final = want.shape[2]
        keep = t.Inputs()
        out = Fenced((B, T, r_final), np.int64, fill=-7)
        assert lib.k2amd_rnnt_prune_ranges(keep(gx), keep(gy), keep(c["boundary"]), p(out), B, S, T, int(modified), r_final, t.dcode(dtype), None) == 0
        np.testing.assert_array_equal(out.a, want)
        # lattice on these ranges
        C = 4
        logits = rng.standard_normal((B, T, r_final, C)).astype(np.float32)
        frames = c["boundary"][:, 3].astype(np.int32)
        got = t._lattice(lib, want.astype(np.int32), frames, c["symbols"] % C, logits)
        w = olat.pruned_ranges_to_lattice(want.astype(np.int32), frames, c["symbols"] % C, logits)
        np.testing.assert_array_equal(got[0], w[0]); np.testing.assert_array_equal(got[1], w[1])
        np.testing.assert_array_equal(got[2][:, :3], w[2]); np.testing.assert_array_equal(got[3], w[4])


def test_recursion_kernels_on_random_small_shapes(lib):
    """The exact kernels bit for bit against the CPU loops, the fp64 pipelined kernels to 1e-10,
    the workspace clean after every pair of calls."""
    rng = np.random.default_rng(13)
    ws_bytes = 1 << 20
    ws = Fenced((ws_bytes,), np.uint8)
    assert lib.k2amd_mi_workspace_init(p(ws), ws_bytes, None) == 0
    for n in range(12 * MORE):
        modified = bool(rng.integers(2)); dtype = [np.float32, np.float64][rng.integers(2)]
        B = int(rng.integers(1, 4)); S = int(rng.integers(0, 90)); T = int(rng.integers(0, 40))
        if modified and T < S: T = S + int(rng.integers(0, 5))
        T1 = T if modified else T + 1
        px = rng.standard_normal((B, S, T1)).astype(dtype); py = rng.standard_normal((B, S + 1, T)).astype(dtype)
        kind = int(rng.integers(4))
        if kind == 1: px[rng.random(px.shape) < 0.1] = -np.inf
        if kind == 2: py[rng.random(py.shape) < 0.1] = -np.inf
        bd = None
        if rng.integers(3):
            s0 = rng.integers(0, S + 1, B); s1 = np.array([rng.integers(a, S + 1) for a in s0])
            t0_ = rng.integers(0, T + 1, B); t1 = np.array([rng.integers(a, T + 1) for a in t0_])
            bd = np.stack([s0, t0_, s1, t1], 1).astype(np.int64)
        with np.errstate(all="ignore"):
            want_ans, want_p = omi.mi_forward(px, py, bd)
            want_gx, want_gy = omi.mi_backward(px, py, bd, want_p)
        fpx, fpy, fbd = fenced(px), fenced(py), fenced(bd)
        pp, ans = Fenced((B, S + 1, T + 1), dtype, fill=np.nan), Fenced((B,), dtype, fill=np.nan)
        dc = t.dcode(dtype)
        # exact kernels: no workspace
        assert lib.k2amd_mi_forward(p(fpx), p(fpy), p(fbd), p(pp), p(ans), B, S, T, int(modified), dc, None, 0, None) == 0
        np.testing.assert_array_equal(ans.a, want_ans)
        gx, gy = Fenced(px.shape, dtype, fill=np.nan), Fenced(py.shape, dtype, fill=np.nan)
        g = Fenced((B,), dtype, fill=1.0)
        assert lib.k2amd_mi_backward(p(fpx), p(fpy), p(fbd), p(pp), p(g), p(gx), p(gy), B, S, T, int(modified), dc, 1, None, 0, None) == 0
        np.testing.assert_array_equal(gx.a, want_gx); np.testing.assert_array_equal(gy.a, want_gy)
        if dtype == np.float64 and lib.k2amd_mi_workspace_bytes(B, S, T, int(modified), dc) > 0:
            pp2, ans2 = Fenced((B, S + 1, T + 1), dtype, fill=np.nan), Fenced((B,), dtype, fill=np.nan)
            assert lib.k2amd_mi_forward(p(fpx), p(fpy), p(fbd), p(pp2), p(ans2), B, S, T, int(modified), dc, p(ws), ws_bytes, None) == 0
            np.testing.assert_allclose(ans2.a, want_ans, rtol=1e-10, atol=1e-10)
            gx2, gy2 = Fenced(px.shape, dtype, fill=np.nan), Fenced(py.shape, dtype, fill=np.nan)
            g2 = Fenced((B,), dtype, fill=1.0)
            assert lib.k2amd_mi_backward(p(fpx), p(fpy), p(fbd), p(pp2), p(g2), p(gx2), p(gy2), B, S, T, int(modified), dc, 1, p(ws), ws_bytes, None) == 0
            np.testing.assert_allclose(gx2.a, want_gx, rtol=1e-9, atol=1e-10); np.testing.assert_allclose(gy2.a, want_gy, rtol=1e-9, atol=1e-10)
            words = ws.a.view(np.uint32)
            assert (words[:3] == 0).all() and (words[64:] == 0x7fc5a5a5).all(), "workspace not clean"
