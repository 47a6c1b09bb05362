"""The smoothed builder's HIP kernels (k2_amd/csrc/rnnt_smoothed.hip) compiled with g++ over the
thread stand-in of tests/cpu_build/hip/hip_runtime.h and run on the host: the same kernel source
as the GPU library's, every work-item a thread, barriers and wavefront exchanges real.

What this pins without a GPU: the kernels' indexing (a second build runs under AddressSanitizer
and UBSan), their reductions and their formulas, forward against the oracle's
get_rnnt_logprobs_smoothed (itself pinned by the reference's fixtures) and backward against the
closed-form gradients (pinned by torch autograd in tests/test_closed_forms.py).  What it cannot
pin: anything that differs between the host compiler and hipcc, and the hardware's behaviour."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import cases
import closed_forms as cf
from oracle import mi as omi
from oracle import rnnt as orn

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(ROOT, "k2_amd", "csrc", "rnnt_smoothed.hip")
SHIM = os.path.join(HERE, "cpu_build")
OUT = os.path.join(SHIM, "_build", os.environ.get("PYTEST_XDIST_WORKER", ""))  # as tests/cpu_kernels.py
TYPES = ["regular", "modified", "constrained"]
CODES = {"regular": 0, "modified": 1, "constrained": 2}


def _compile(args, out):
    os.makedirs(OUT, exist_ok=True)
    cmd = ["g++", "-std=c++20", "-O1", "-g", "-pthread", f"-I{SHIM}", f"-I{os.path.join(ROOT, 'k2_amd', 'csrc')}",
           *args, "-o", out]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    return out


@pytest.fixture(scope="module")
def lib():
    import cpu_kernels
    return cpu_kernels.lib()  # the host build of all portable kernels, k2_amd/capi.py's signatures


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


GUARD = 64


class Guarded:
    """An array with a strip of a known pattern on either side: a kernel that writes just outside
    its output is caught when the strips are checked."""

    def __init__(self, shape, dtype, fill=np.nan):
        n = int(np.prod(shape))
        self.raw = np.full(n + 2 * GUARD, 12345.0, dtype=dtype)
        self.a = self.raw[GUARD:GUARD + n].reshape(shape)
        self.a[...] = fill

    def intact(self):
        return bool((self.raw[:GUARD] == 12345.0).all() and (self.raw[-GUARD:] == 12345.0).all())


def _joint_parts(c, rnnt_type):
    """What k2amd_rnnt_logprobs_simple_forward hands over: px / py of the regular or modified
    lattice without a boundary, the max-shifted exponentials and the maxima."""
    lm, am = c["lm"], c["am"]
    px, py = orn.logprobs_simple(lm, am, c["symbols"], 0, "regular" if rnnt_type == "regular" else "modified", None)
    lm_max, am_max = lm.max(axis=2), am.max(axis=2)
    return (np.ascontiguousarray(px), np.ascontiguousarray(py), np.exp(lm - lm_max[..., None]),
            np.exp(am - am_max[..., None]), np.ascontiguousarray(lm_max), np.ascontiguousarray(am_max))


def _run(lib, c, rnnt_type, scales, use_boundary, weights):
    lm, am, sym = c["lm"], c["am"], c["symbols"]
    dt = lm.dtype
    B, T, C = am.shape
    S = lm.shape[1] - 1
    bd = c["boundary"] if use_boundary else None
    code, dcode = CODES[rnnt_type], 0 if dt == np.float32 else 1
    assert lib.k2amd_rnnt_smoothed_supported(B, S, T, C, dcode) == 1
    pxj, pyj, lm_probs, am_probs, lm_max, am_max = _joint_parts(c, rnnt_type)
    T1 = T + 1 if rnnt_type == "regular" else T
    px, py = Guarded((B, S, T1), dt), Guarded((B, S + 1, T), dt)
    lm_norm, am_norm, unigram = Guarded((B, S + 1), dt), Guarded((B, T), dt), Guarded((2, C), dt)
    n = lib.k2amd_rnnt_smoothed_scratch_elements(B, S, T, C)
    scratch = Guarded((n,), dt)
    args = (B, S, T, C, 0, code, dcode, None)
    assert lib.k2amd_rnnt_smoothed_forward(
        _p(lm), _p(am), _p(sym), _p(bd), _p(lm_probs), _p(am_probs), _p(lm_max), _p(am_max), _p(pxj), _p(pyj),
        _p(px.a), _p(py.a), _p(lm_norm.a), _p(am_norm.a), _p(unigram.a), _p(scratch.a), n - 1, *scales, *args) == 3
    assert np.isnan(px.a).all() and np.isnan(py.a).all()  # refused before anything was launched
    assert lib.k2amd_rnnt_smoothed_forward(
        _p(lm), _p(am), _p(sym), _p(bd), _p(lm_probs), _p(am_probs), _p(lm_max), _p(am_max), _p(pxj), _p(pyj),
        _p(px.a), _p(py.a), _p(lm_norm.a), _p(am_norm.a), _p(unigram.a), _p(scratch.a), n, *scales, *args) == 0
    for g in (px, py, lm_norm, am_norm, unigram, scratch):
        assert g.intact()
    want_px, want_py = orn.logprobs_smoothed(lm, am, sym, 0, scales[0], scales[1], bd, rnnt_type)
    tol = dict(rtol=1e-12, atol=1e-12) if dt == np.float64 else dict(rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(px.a, want_px, **tol)
    np.testing.assert_allclose(py.a, want_py, **tol)

    # backward: the occupation probabilities of the mixed lattice as the gradients that reach px / py
    _, gx, gy = omi.mi(want_px.astype(np.float64), want_py.astype(np.float64), bd)
    w = weights
    want_lm, want_am = cf.smoothed_grads(lm, am, sym, 0, scales[0], scales[1], gx, gy,
                                         np.ones(B) if w is None else w, rnnt_type)
    joint_lm, joint_am = cf.simple_grads(lm, am, sym, 0, gx, gy, np.ones(B) if w is None else w, rnnt_type)
    js = 1.0 - scales[0] - scales[1]
    # the gradients of sum_b w[b] score[b] (the closed forms are the loss's: the other sign); the
    # joint term is in the buffers already, as the simple builder's backward leaves it
    lm_grad, am_grad = Guarded(lm.shape, dt), Guarded(am.shape, dt)
    lm_grad.a[...] = -js * joint_lm
    am_grad.a[...] = -js * joint_am
    gxa, gya = np.ascontiguousarray(gx.astype(dt)), np.ascontiguousarray(gy.astype(dt))
    seq = None if w is None else np.ascontiguousarray(w.astype(dt))
    scratch.a[...] = np.nan
    assert lib.k2amd_rnnt_smoothed_backward(
        _p(gxa), _p(gya), _p(seq), _p(sym), _p(bd), _p(lm_probs), _p(am_probs), _p(lm_max), _p(am_max),
        _p(lm_norm.a), _p(am_norm.a), _p(unigram.a), _p(lm_grad.a), _p(am_grad.a), _p(scratch.a), n,
        *scales, *args) == 0
    for g in (lm_grad, am_grad, scratch, lm_norm, am_norm, unigram):
        assert g.intact()
    tol = dict(rtol=1e-9, atol=1e-11) if dt == np.float64 else dict(rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(lm_grad.a, -want_lm, **tol)
    np.testing.assert_allclose(am_grad.a, -want_am, **tol)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("rnnt_type", TYPES)
def test_forward_and_backward_equal_the_oracle_and_the_closed_forms(lib, rnnt_type, dtype):
    # C = 70: a partial second column per lane; B (S+1) = 21 and B T = 33: partial groups of rows;
    # symbols repeat within a sequence (C small against S would do it too: here 6 positions of 69)
    c = cases.rnnt_case(71, 3, 11, 6, 70, dtype=dtype, t_lo=8, s_lo=3, modified=rnnt_type != "regular")
    c["symbols"][:, 1] = c["symbols"][:, 0]  # a repeated symbol: two terms land on one column
    c["symbols"][:, 3] = 0                   # the termination symbol as an ordinary one
    _run(lib, c, rnnt_type, (0.25, 0.1), True, np.linspace(0.5, 1.5, 3))
    _run(lib, c, rnnt_type, (0.0, 0.3), False, None)


def test_column_sums_over_several_chunks_of_rows(lib):
    """Enough rows of lm (164) and of am (180) for three chunks each in the two-step column sums
    (the unigram forward, its gradient backward), a vocabulary that ends inside a block of 64."""
    c = cases.rnnt_case(73, 4, 45, 40, 70, dtype=np.float64, t_lo=42, s_lo=30)
    c["symbols"][:, 5] = c["symbols"][:, 2]
    c["symbols"][:, 9] = c["symbols"][:, 2]  # a chain of three positions
    _run(lib, c, "regular", (0.2, 0.15), True, np.linspace(0.5, 1.5, 4))


def test_shapes_at_the_edges(lib):
    # one row, one frame, one class more than a wavefront's lanes; S = 0
    for B, T, S, C in ((1, 1, 1, 65), (2, 5, 0, 3), (1, 17, 16, 64), (5, 3, 2, 2)):
        c = cases.rnnt_case(72, B, T, S, C, dtype=np.float64, t_lo=T, s_lo=S)
        _run(lib, c, "regular", (0.2, 0.2), False, None)
    # no frames: the regular lattice keeps its one -inf column
    B, S, C = 2, 3, 5
    lm = np.random.default_rng(1).standard_normal((B, S + 1, C))
    lm_max = np.ascontiguousarray(lm.max(axis=2))
    lm_probs = np.exp(lm - lm_max[..., None])
    sym = np.ones((B, S), np.int64)
    px, lm_norm, unigram = Guarded((B, S, 1), np.float64), Guarded((B, S + 1), np.float64), Guarded((2, C), np.float64)
    n = lib.k2amd_rnnt_smoothed_scratch_elements(B, S, 0, C)
    scratch = Guarded((n,), np.float64)
    assert lib.k2amd_rnnt_smoothed_forward(_p(lm), None, _p(sym), None, _p(lm_probs), None, _p(lm_max), None, None,
                                           None, _p(px.a), None, _p(lm_norm.a), None, _p(unigram.a), _p(scratch.a),
                                           n, 0.1, 0.1, B, S, 0, C, 0, 0, 1, None) == 0
    assert np.isneginf(px.a).all() and px.intact() and unigram.intact() and scratch.intact()
    np.testing.assert_allclose(unigram.a[0].sum(), 1.0, rtol=1e-12)


def test_refusals(lib):
    assert lib.k2amd_rnnt_smoothed_supported(2, 10, 20, 100000, 0) == 1    # no vocabulary limit
    assert lib.k2amd_rnnt_smoothed_supported(2, 10, 20, 50, 2) == 0        # float16: not a type of the builders
    none = [None] * 16
    assert lib.k2amd_rnnt_smoothed_forward(*none, 0, 0.1, 0.1, 2, 10, 20, 50, 50, 0, 0, None) == 1   # blank >= C
    assert lib.k2amd_rnnt_smoothed_forward(*none, 0, 0.1, 0.1, 2, 10, 20, 50, 0, 0, 0, None) == 1    # null tensors
    assert lib.k2amd_rnnt_smoothed_forward(*none, 0, 0.1, 0.1, 0, 10, 20, 50, 0, 0, 0, None) == 0    # empty batch
    assert lib.k2amd_rnnt_smoothed_backward(*([None] * 15), 0, 0.1, 0.1, 2, 10, 20, 50, 0, 3, 0, None) == 1


def test_kernels_under_the_address_sanitizer():
    """The same source and stand-in in one executable with exact-size heap buffers, random inputs
    and the shapes above, built with -fsanitize=address,undefined: any access outside a buffer (LDS
    arrays included: the stand-in allocates exactly the bytes a launch asks for) ends it."""
    exe = _compile(["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
                    os.path.join(SHIM, "smoothed_sanitizer_main.cc")], os.path.join(OUT, "smoothed_sanitizer"))
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "all shapes done" in proc.stdout
