"""The pipelined fp32 mutual-information kernels and the single launch (k2_amd/csrc/mi_fast.hip)
on the host build (tests/cpu_kernels.py): the kernels that the library takes by default for fp32,
the single launch among them (the headline measurement's kernel), without a GPU.

Their source is compiled from a copy in which the inline assembly (two DPP arithmetic
instructions, the range-checked buffer loads, coherent loads and stores, wait counts) is replaced
by calls that do what the instructions do; everything else is the GPU library's text: the
specialised wavefronts of a workgroup and what they hand to each other through LDS, blocks, frames
and the gauge, the hand-over between chunks through self-validating words, the cut and the join
of the single launch, its task order, the bounded waits.  Every work-item is a thread and the
workgroups run one after the other, in the order of their tickets.

Checked here: parity with the CPU oracle (oracle/mi.py, fp32 and fp64) to the GPU tests' own bar,
through the C-ABI on buffers that end or begin at an inaccessible page and through the Python
layer with the GPU tests' own routine (tests/test_mi_gpu.py: the pair of launches, the pair with
the log-derivative tensor, with and without p, the single launch, twice, and without a seed); that
the workspace is left as found; that a wait which really expires ends every kernel and is
reported.  Not shown here: anything that needs workgroups running at the same time, the device's
memory model, and timing."""
import os

import numpy as np
import pytest
import torch

import cases
import cpu_kernels as ck
import test_mi_gpu as gpu_tests
from cpu_kernels import Fenced, fenced, p
from oracle import mi as omi
from test_cpu_build_host_layer import host_on_cpu  # noqa: F401  (fixture)

slow = pytest.mark.skipif(os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1",
                          reason="slow on the host: run with K2AMD_SLOW_CPU_TESTS=1")
CPU = torch.device("cpu")
SENTINEL = 0x7FC5A5A5
TIMEOUT = 5  # K2AMD_ERR_TIMEOUT


@pytest.fixture(scope="module")
def lib():
    return ck.lib()


def _workspace(lib, B, S, T, modified, at):
    n = lib.k2amd_mi_workspace_bytes(B, S, T, int(modified), 0)
    assert n > 0 and n % 4 == 0
    ws = Fenced((n // 4,), np.uint32, fill=0, at=at)
    assert lib.k2amd_mi_workspace_init(p(ws), n, None) == 0
    return ws, n


def _clean(ws):
    return bool((ws.a[:3] == 0).all()) and bool((ws.a[64:] == SENTINEL).all())


def _oracles(px, py, bd, ans_grad):
    out = []
    for dt in (np.float32, np.float64):
        x, y = px.astype(dt), py.astype(dt)
        ans, pp = omi.mi_forward(x, y, bd)
        gx, gy = omi.mi_backward(x, y, bd, pp, ans_grad=ans_grad.astype(dt))
        out.append((ans, pp, gx, gy))
    return out


def _compare(name, got, w32, w64):
    tol = gpu_tests.TOL[np.dtype(np.float32)]
    ans, gx, gy = got
    gpu_tests._close(name + " ans", ans, w32[0], w64[0], tol, mode="absolute")
    gpu_tests._close(name + " px_grad", gx, w32[2], w64[2], tol)
    gpu_tests._close(name + " py_grad", gy, w32[3], w64[3], tol)


@pytest.mark.parametrize("modified,at", [(False, "end"), (True, "start"), pytest.param(False, "start", marks=slow),
                                         pytest.param(True, "end", marks=slow)])
def test_every_route_on_fenced_buffers(lib, modified, at):
    """Two chunks of rows, two or three blocks of columns, four sequences with boxes of their own (one of a
    single row, one that starts inside the second block): the pair of launches, the pair with the
    log-derivative tensor and no p, and the single launch, through the C-ABI.  Every tensor, the
    workspace and the single launch's scratch end (or begin) at an inaccessible page."""
    rng = np.random.default_rng(31 + int(modified))
    B, S, T = 4, 70, (75 if modified else 45)  # (a modified lattice needs a frame per symbol)
    T1 = T if modified else T + 1
    px = rng.normal(-1.5, 1.0, (B, S, T1)).astype(np.float32)
    py = rng.normal(-1.5, 1.0, (B, S + 1, T)).astype(np.float32)
    bd = np.array([[0, 0, S, T], [3, 2, 68, T - 4], [5, 7, 5, 30], [1, 33, 9, T]], np.int64)
    seed = np.linspace(0.5, 1.5, B).astype(np.float32)
    w32, w64 = _oracles(px, py, bd, seed)
    fpx, fpy, fbd = fenced(px, at), fenced(py, at), fenced(bd, at)
    ws, n = _workspace(lib, B, S, T, modified, at)
    m = int(modified)

    # the pair of launches
    pp, ans = Fenced((B, S + 1, T + 1), np.float32, fill=np.nan, at=at), Fenced((B,), np.float32, fill=np.nan, at=at)
    assert lib.k2amd_mi_forward(p(fpx), p(fpy), p(fbd), p(pp), p(ans), B, S, T, m, 0, p(ws), n, None) == 0
    assert _clean(ws)
    inside = ~np.isnan(w32[1])
    got_p, p32, p64 = (np.where(inside, a, 0.0) for a in (pp.a, w32[1], w64[1]))
    gpu_tests._close("p", got_p, p32, p64, gpu_tests.TOL[np.dtype(np.float32)], mode="absolute")
    g = fenced(seed, at)
    gx, gy = Fenced(px.shape, np.float32, fill=np.nan, at=at), Fenced(py.shape, np.float32, fill=np.nan, at=at)
    assert lib.k2amd_mi_backward(p(fpx), p(fpy), p(fbd), p(pp), p(g), p(gx), p(gy), B, S, T, m, 0, 1, p(ws), n, None) == 0
    assert _clean(ws)
    _compare("pair", (ans.a, gx.a, gy.a), w32, w64)
    np.testing.assert_allclose(g.a, seed, rtol=1e-3)
    pair = (ans.a.copy(), gx.a.copy(), gy.a.copy(), g.a.copy())

    # the pair with the log-derivatives between them and no p: the same bits
    assert lib.k2amd_mi_keeps_log_deriv(B, S, T, m, 0, 1) == 1
    ld = Fenced((B, S + 1, T + 1), np.float32, fill=np.nan, at=at)
    for f in (ans, gx, gy):
        f.a[...] = np.nan
    g.a[...] = seed
    assert lib.k2amd_mi_forward_keep(p(fpx), p(fpy), p(fbd), None, p(ans), p(ld), B, S, T, m, 0, p(ws), n, None) == 0
    assert lib.k2amd_mi_backward_kept(p(fpx), p(fpy), p(fbd), None, p(ld), p(g), p(gx), p(gy), B, S, T, m, 0, 1,
                                      p(ws), n, None) == 0
    assert _clean(ws)
    for name, a, b in zip(("ans", "px_grad", "py_grad", "ans_grad"), (ans.a, gx.a, gy.a, g.a), pair):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), "kept pair differs in " + name

    # the single launch
    assert lib.k2amd_mi_forward_backward_supported(B, S, T, m, 0, 1) == 1
    nb = lib.k2amd_mi_forward_backward_scratch_bytes(B, S, T, m, 0)
    assert nb > 0 and nb % 4 == 0
    scratch = Fenced((nb // 4,), np.float32, fill=np.nan, at=at)
    for f in (ans, gx, gy):
        f.a[...] = np.nan
    g.a[...] = seed
    assert lib.k2amd_mi_forward_backward(p(fpx), p(fpy), p(fbd), p(ans), p(scratch), nb, p(g), p(gx), p(gy), B, S, T,
                                         m, 0, 1, p(ws), n, None) == 0
    assert _clean(ws)
    _compare("single launch", (ans.a, gx.a, gy.a), w32, w64)
    np.testing.assert_allclose(g.a, seed, rtol=1e-3)
    assert lib.k2amd_mi_workspace_status(p(ws), None) == 0
    for f in (fpx, fpy, fbd, ws, pp, ans, g, gx, gy, ld, scratch):
        assert f.intact()


def _check(name, px, py, bd):
    ans, pp = omi.mi_forward(px, py, bd)
    gx, gy = omi.mi_backward(px, py, bd, pp)
    gpu_tests.check(name, px, py, bd, (ans, pp, gx, gy), CPU)


def test_tiny_lattices_through_the_python_layer(host_on_cpu):
    """A lattice of two by three cells, several to a batch: every 16-byte load then starts in front
    of its sequence's first element.  All routes, with the GPU tests' own routine.  (All sizes
    from one to three cells a side: test_gpu_test_body_sequences_shorter_than_a_quad.)"""
    rng = np.random.default_rng(77)
    for S, T in ((2, 3),):
        B = 3
        px = rng.standard_normal((B, S, T + 1)).astype(np.float32)
        py = rng.standard_normal((B, S + 1, T)).astype(np.float32)
        _check(f"S{S}T{T}", px, py, np.tile(np.array([[0, 0, S, T]], np.int64), (B, 1)))


@pytest.mark.parametrize("modified", [False, pytest.param(True, marks=slow)])
def test_blocked_edges_and_sequences_that_no_path_reaches(host_on_cpu, modified):
    """Edges of log-probability -inf (so many that some end cells are unreachable: those sequences
    take the exact recursion inside the single launch) and of -3000, on two chunks: all routes
    must agree with the CPU code's guards (k2/python/csrc/torch/mutual_information_cpu.cu:195-211)."""
    rng = np.random.default_rng(90 + int(modified))
    B, S, T = 4, 66, 40
    px = rng.normal(-2.0, 1.0, (B, S, T if modified else T + 1)).astype(np.float32)
    py = rng.normal(-2.0, 1.0, (B, S + 1, T)).astype(np.float32)
    for a in (px, py):
        a[rng.random(a.shape) < 0.03] = -np.inf
        a[rng.random(a.shape) < 0.02] = -3000.0
    px[3, 2, :] = -np.inf                                       # nothing gets past row 2 of sequence 3
    bd = np.array([[0, 0, S, T], [2, 3, 60, 38], [0, 10, 3, 14], [0, 0, 9, 30]], dtype=np.int64)
    ans, _ = omi.mi_forward(px, py, bd)
    assert np.isneginf(ans[3]) and np.isfinite(ans).any()
    _check(f"blocked modified={modified}", px, py, bd)


def test_a_wait_that_really_expires_ends_every_kernel_and_is_reported(lib):
    """The ticket counter is handed over one ahead, as if a workgroup had drawn a ticket and died:
    the first chunk of the first sequence never runs, the chunk below it waits for words that never
    come, gives up at the spin limit and raises the flag; every later wait returns at its next look
    at the flag, all workgroups end, ans holds NaN and the status call says so.  (The tensors and
    the workspace are sized for one sequence more than the call names: the last ticket drawn is
    that sequence's.)  The workspace, initialised again, serves the call correctly."""
    rng = np.random.default_rng(5)
    B, S, T = 3, 70, 40
    px = rng.normal(-1.5, 1.0, (B, S, T + 1)).astype(np.float32)
    py = rng.normal(-1.5, 1.0, (B, S + 1, T)).astype(np.float32)
    bd = np.tile(np.array([[0, 0, S, T]], np.int64), (B, 1))
    ws, n = _workspace(lib, B, S, T, False, "end")
    ws.a[0] = 1                                                  # FastHeader::ticket
    pp, ans = np.zeros((B, S + 1, T + 1), np.float32), np.zeros(B, np.float32)
    assert lib.k2amd_mi_forward(p(px), p(py), p(bd), p(pp), p(ans), B - 1, S, T, 0, 0, p(ws), n, None) == 0
    assert np.isnan(ans[:B - 1]).all()
    assert lib.k2amd_mi_workspace_status(p(ws), None) == TIMEOUT
    assert lib.k2amd_mi_workspace_init(p(ws), n, None) == 0
    assert lib.k2amd_mi_forward(p(px), p(py), p(bd), p(pp), p(ans), B - 1, S, T, 0, 0, p(ws), n, None) == 0
    want, _ = omi.mi_forward(px[:B - 1], py[:B - 1], bd[:B - 1])
    np.testing.assert_allclose(ans[:B - 1], want, rtol=1e-4, atol=1e-5)
    assert lib.k2amd_mi_workspace_status(p(ws), None) == 0 and _clean(ws) and ws.intact()


def test_a_raised_flag_turns_every_result_into_nan(host_on_cpu):
    """The error flag set by hand, as the GPU tests do: every wait returns at once, every kernel
    ends, and the forward, the backward and the single launch all say NaN where a caller looks
    first; the status call raises.  (The API's own report, at its next read of a boundary tensor
    from the device, needs a device and is a GPU test.)"""
    capi = host_on_cpu
    rng = np.random.default_rng(9)
    B, S, T = 2, 66, 34
    px = torch.from_numpy(rng.normal(-2, 1, (B, S, T + 1)).astype(np.float32))
    py = torch.from_numpy(rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32))
    pp = torch.empty(B, S + 1, T + 1)
    good = capi.mi_forward(px, py, None, pp).clone()
    assert torch.isfinite(good).all()
    (key,) = capi._workspaces.keys()
    capi._workspaces[key][:16].view(torch.int32)[2] = 1              # FastHeader::error
    assert torch.isnan(capi.mi_forward(px, py, None, pp)).all()
    g = torch.ones(B)
    capi.mi_backward(px, py, None, pp, g, overwrite_ans_grad=True)
    assert torch.isnan(g).all()
    ans, _, _ = capi.mi_forward_backward(px, py, None, torch.ones(B))
    assert torch.isnan(ans).all()
    with pytest.raises(RuntimeError, match="timed out"):
        capi.mi_workspace_status(CPU)
    del capi._workspaces[key]                                        # the next call initialises a new one
    assert torch.equal(capi.mi_forward(px, py, None, pp), good)
    assert capi.mi_workspace_is_clean(CPU)


def test_no_allocation_entry_point_on_the_pipelined_kernels(host_on_cpu):
    """k2amd_mi_forward_noalloc on a shape that the pipelined kernels serve: its scratch is the
    library's static array (looked up by symbol, cleared by the call's own fill kernel), its
    results are k2amd_mi_forward's bits, on two calls in a row, the second smaller."""
    capi = host_on_cpu
    rng = np.random.default_rng(23)
    for B, S, T in ((3, 70, 40), (2, 9, 12)):
        px = torch.from_numpy(rng.normal(-2, 1, (B, S, T + 1)).astype(np.float32))
        py = torch.from_numpy(rng.normal(-2, 1, (B, S + 1, T)).astype(np.float32))
        assert capi.lib().k2amd_mi_workspace_bytes(B, S, T, 0, 0) > 0
        p1, p2 = torch.empty(B, S + 1, T + 1), torch.empty(B, S + 1, T + 1)
        want = capi.mi_forward(px, py, None, p1)
        got = capi.mi_forward_noalloc(px, py, None, p2, torch.empty(B))
        assert torch.equal(got, want) and torch.equal(p1, p2)
        assert capi.lib().k2amd_mi_noalloc_status(None) == 0
        ans, _ = omi.mi_forward(px.numpy(), py.numpy(), None)
        np.testing.assert_allclose(got.numpy(), ans, rtol=1e-4, atol=1e-5)


# ---- the GPU tests' own bodies on the host build (minutes each) ---------------------------------

@slow
@pytest.mark.parametrize("modified", [False, True])
def test_gpu_test_body_sequences_shorter_than_a_quad(host_on_cpu, modified):
    gpu_tests.test_sequences_shorter_than_a_quad(CPU, modified)


@slow
def test_gpu_test_body_reference_fixtures(host_on_cpu):
    gpu_tests.test_reference_fixtures(CPU)


@slow
def test_random_shapes_of_up_to_three_chunks(host_on_cpu):
    """The shapes of the GPU tests' random multi-chunk cases, scaled down to what the host build
    runs in minutes: up to three chunks, up to five blocks, random boundaries, both lattice types."""
    for seed in range(5000, 5012):
        shape = (dict(max_B=3, max_S=150, max_T=60), dict(max_B=5, max_S=80, max_T=100),
                 dict(max_B=2, max_S=70, max_T=170))[seed % 3]
        c = cases.mi_case(seed, dtype=np.float32, **shape)
        _check(f"seed{seed}", c["px"], c["py"], c["boundary"])


@slow
def test_high_magnitude_scores(host_on_cpu):
    """px and py offset by +15 (k2/python/tests/mutual_information_test.py:117-130) on lattices
    of several chunks: what the frames and the gauge of the single launch are for, judged in the
    max norm against the fp64 oracle with the reference's own fp32 code as the yardstick."""
    for seed in (9001, 9002, 9004):
        c = cases.mi_case(seed, dtype=np.float32, max_B=2, max_S=130, max_T=150,
                          force=dict(big_px=seed % 4 in (0, 2, 3), big_py=seed % 4 in (1, 2), random_px=True,
                                     random_py=True))
        px, py, bd = c["px"], c["py"], c["boundary"]
        a32, p32 = omi.mi_forward(px, py, bd)
        gx32, gy32 = omi.mi_backward(px, py, bd, p32)
        a64, p64 = omi.mi_forward(px.astype(np.float64), py.astype(np.float64), bd)
        gx64, gy64 = omi.mi_backward(px.astype(np.float64), py.astype(np.float64), bd, p64)
        ans, _, gx, gy, _, _ = gpu_tests.run_gpu(px, py, bd, CPU)
        assert gpu_tests.run_gpu.single is not None
        for route, a, x, y in (("two launches", ans, gx, gy), ("single launch",) + tuple(gpu_tests.run_gpu.single[:3])):
            fin = np.isfinite(a64)
            assert (np.isfinite(a) == fin).all(), (seed, route)
            np.testing.assert_allclose(a[fin], a64[fin], rtol=1e-4, atol=1e-5, err_msg=f"seed {seed} {route} ans")
            gpu_tests.max_norm_check(f"seed {seed} {route} px_grad", x, gx32, gx64)
            gpu_tests.max_norm_check(f"seed {seed} {route} py_grad", y, gy32, gy64)


def random_case(rng):
    """A random small lattice for the pipelined kernels: one to three chunks, zero to three blocks,
    S = 0 and T = 0 among them, boxes that leave one row or one column or nothing, blocked edges."""
    modified = bool(rng.integers(2))
    B = int(rng.integers(1, 4))
    S = int((0, 1, 3, 62, 63, 64, 65, 127, 130)[rng.integers(9)]) if rng.integers(2) else int(rng.integers(0, 140))
    T = int((0, 1, 2, 3, 31, 32, 33, 64, 65)[rng.integers(9)]) if rng.integers(2) else int(rng.integers(0, 80))
    if modified and T < S and rng.integers(4):
        T = S + int(rng.integers(0, 5))
    T1 = T if modified else T + 1
    px = rng.normal(-1.0, 1.0, (B, S, T1)).astype(np.float32)
    py = rng.normal(-1.0, 1.0, (B, S + 1, T)).astype(np.float32)
    kind = int(rng.integers(5))
    if kind == 1:
        px[rng.random(px.shape) < 0.05] = -np.inf
    if kind == 2:
        py[rng.random(py.shape) < 0.05] = -np.inf
    if kind == 3:
        px += 15.0
    bd = None
    if rng.integers(3):
        s0 = rng.integers(0, S + 1, B)
        s1 = np.array([rng.integers(a, S + 1) for a in s0])
        t0 = rng.integers(0, T + 1, B)
        t1 = np.array([rng.integers(a, T + 1) for a in t0])
        bd = np.stack([s0, t0, s1, t1], 1).astype(np.int64)
    elif not modified and T1 > 0 and rng.integers(2):
        px[:, :, -1] = -np.inf   # as the reference's builders leave it
    return modified, B, S, T, px, py, bd


def run_random_case(lib, rng, ws, ws_bytes):
    modified, B, S, T, px, py, bd = random_case(rng)
    m = int(modified)
    what = f"modified={modified} B={B} S={S} T={T} bd={None if bd is None else bd.tolist()}"
    if lib.k2amd_mi_workspace_bytes(B, S, T, m, 0) == 0:
        return 0
    assert lib.k2amd_mi_workspace_bytes(B, S, T, m, 0) <= ws_bytes
    seed = rng.uniform(0.5, 1.5, B).astype(np.float32)
    with np.errstate(all="ignore"):
        w32, w64 = _oracles(px, py, bd, seed)
    at = ("end", "start")[rng.integers(2)]
    fpx, fpy, fbd = fenced(px, at), fenced(py, at), fenced(bd, at)
    reachable = np.isfinite(w64[0])
    # with px offset by +15 the scores are in the hundreds and thousands: the bar for such inputs
    # is the max norm against fp64 with the reference's fp32 code as the yardstick
    big = bool(np.abs(w64[0][reachable]).max() > 200) if reachable.any() else False

    def judge(route, ans, gx, gy, g):
        if big:
            np.testing.assert_allclose(ans[reachable], w64[0][reachable], rtol=1e-4, atol=1e-5, err_msg=what + route)
            gpu_tests.max_norm_check(what + route + " px_grad", gx, w32[2], w64[2])
            gpu_tests.max_norm_check(what + route + " py_grad", gy, w32[3], w64[3])
        else:
            _compare(what + route, (ans, gx, gy), w32, w64)
        np.testing.assert_allclose(g[reachable], seed[reachable], rtol=1e-3, err_msg=what + route)

    pp, ans = Fenced((B, S + 1, T + 1), np.float32, fill=np.nan, at=at), Fenced((B,), np.float32, fill=np.nan, at=at)
    gx, gy = Fenced(px.shape, np.float32, fill=np.nan, at=at), Fenced(py.shape, np.float32, fill=np.nan, at=at)
    g = fenced(seed, at)
    assert lib.k2amd_mi_forward(p(fpx), p(fpy), p(fbd), p(pp), p(ans), B, S, T, m, 0, p(ws), ws_bytes, None) == 0, what
    assert lib.k2amd_mi_backward(p(fpx), p(fpy), p(fbd), p(pp), p(g), p(gx), p(gy), B, S, T, m, 0, 1, p(ws), ws_bytes,
                                 None) == 0, what
    assert _clean(ws), what
    judge(" pair", ans.a, gx.a, gy.a, g.a)
    launches = 2
    if lib.k2amd_mi_forward_backward_supported(B, S, T, m, 0, 1):
        nb = lib.k2amd_mi_forward_backward_scratch_bytes(B, S, T, m, 0)
        scratch = Fenced((max(nb // 4, 1),), np.float32, fill=np.nan, at=at)
        for f in (ans, gx, gy):
            f.a[...] = np.nan
        g.a[...] = seed
        assert lib.k2amd_mi_forward_backward(p(fpx), p(fpy), p(fbd), p(ans), p(scratch), nb, p(g), p(gx), p(gy), B, S,
                                             T, m, 0, 1, p(ws), ws_bytes, None) == 0, what
        assert _clean(ws), what
        judge(" single launch", ans.a, gx.a, gy.a, g.a)
        assert scratch.intact()
        launches += 1
    assert lib.k2amd_mi_workspace_status(p(ws), None) == 0, what
    for f in (fpx, fpy, fbd, pp, ans, g, gx, gy):
        assert f is None or f.intact(), what
    return launches


def test_random_small_shapes(lib):
    """Fixed seeds; the same generator ran for a quarter of an hour with other seeds while this was
    written.  K2AMD_SLOW_CPU_TESTS=1 runs five times as many cases."""
    rng = np.random.default_rng(4711)
    ws_bytes = 1 << 18
    ws = Fenced((ws_bytes // 4,), np.uint32, fill=0)
    assert lib.k2amd_mi_workspace_init(p(ws), ws_bytes, None) == 0
    launches = 0
    for _ in range(8 * (5 if os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") == "1" else 1)):
        launches += run_random_case(lib, rng, ws, ws_bytes)
    assert launches >= 12 and ws.intact()


# ---- sanitizers -----------------------------------------------------------------------------------

def _program(name, main, compile_flags=(), link_flags=(), kernels=None):
    """A program of its own: tests/cpu_build/<main> with the host copy of mi_fast.hip (or
    `kernels` in its place) and what its entry points need (mi_capi, mi_generic, mi_wave)."""
    import subprocess
    ck.build()  # (writes the host copy)
    flags = [f for f in ck.FLAGS if f != "-fPIC"] + list(compile_flags)
    sources = [kernels or os.path.join(ck.OUT, "mi_fast_host.hip")]
    sources += [os.path.join(ck.CSRC, s + ".hip") for s in ("mi_capi", "mi_generic", "mi_wave")]
    sources.append(os.path.join(ck.SHIM, main))
    jobs = []
    for src in sources:
        obj = os.path.join(ck.OUT, name + "_" + os.path.basename(src).split(".")[0] + ".o")
        jobs.append((obj, subprocess.Popen(["g++", *flags, "-x", "c++", "-c", src, "-o", obj], stdout=subprocess.PIPE,
                                           stderr=subprocess.STDOUT, text=True)))
    for obj, proc in jobs:
        out, _ = proc.communicate()
        assert proc.returncode == 0, out[-3000:]
    exe = os.path.join(ck.OUT, name)
    proc = subprocess.run(["g++", "-pthread", *link_flags, "-o", exe] + [j[0] for j in jobs],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-3000:]
    return exe


def _sanitizer_program(name, sanitizer, extra=()):
    """tests/cpu_build/pipelined_sanitizer_main.cc, everything built with -fsanitize=<sanitizer>."""
    runtime = "-static-libtsan" if sanitizer == "thread" else "-static-libasan"
    return _program(name, "pipelined_sanitizer_main.cc",
                    ["-fsanitize=" + sanitizer, "-fno-sanitize-recover=all", *extra], ["-fsanitize=" + sanitizer, runtime])


def _run_sanitizer_program(exe, *args):
    import subprocess
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 report_signal_unsafe=0 exitcode=0")
    proc = subprocess.run([exe] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=900, env=env)
    if "FATAL: ThreadSanitizer" in proc.stdout:
        pytest.skip("the thread sanitizer does not start here: " + proc.stdout[:200])
    return proc.returncode, proc.stdout


@slow
def test_no_data_race_between_the_wavefronts_of_a_workgroup():
    """The pair, the kept pair and the single launch on two chunks and three blocks, regular and
    modified, under -fsanitize=thread: every work-item is a thread, and what orders two of them is
    what orders two wavefronts on the device (the workgroup's barrier, an atomic) or two lanes of
    one (a wavefront exchange, a fence at wavefront scope, which stands for lockstep here).  No
    report means: no wavefront reads or writes LDS or device memory that another one writes without
    such an ordering between them, on these shapes.  The sanitizer is then shown to see what it
    should: the same program built with wavefront fences that order nothing reports the race in
    the join on the cut (and computes a wrong score)."""
    exe = _sanitizer_program("pipelined_race", "thread")
    scores = {}
    for modified in (0, 1):
        for route in (0, 1, 2):
            code, out = _run_sanitizer_program(exe, 2, 70, 75, modified, route)
            assert code == 0 and "ThreadSanitizer" not in out, out[-4000:]
            scores[modified, route] = float(out.split("score")[1])
        assert scores[modified, 0] == scores[modified, 1]
        assert scores[modified, 2] == pytest.approx(scores[modified, 0], rel=1e-4)
    control = _sanitizer_program("pipelined_race_control", "thread", ["-DHIP_THREADS_FENCES_ARE_NOT_BARRIERS"])
    code, out = _run_sanitizer_program(control, 2, 70, 75, 0, 2)
    assert "WARNING: ThreadSanitizer: data race" in out and "WaveCutJoin" in out, out[-4000:]


@slow
def test_no_access_outside_a_buffer_or_an_lds_array():
    """-fsanitize=address,undefined (with its bounds check of every index into an array of known
    size, the arrays inside a workgroup's LDS structure among them): one to three chunks, one to
    three blocks, chunks and blocks exactly full, lattices of a single cell, both lattice types."""
    exe = _sanitizer_program("pipelined_bounds", "address,undefined")
    for B, S, T, modified in ((2, 70, 75, 0), (2, 70, 75, 1), (3, 130, 33, 0), (3, 1, 1, 0), (1, 64, 64, 1),
                              (2, 63, 31, 0), (2, 127, 32, 0)):
        for route in (0, 1, 2):
            code, out = _run_sanitizer_program(exe, B, S, T, modified, route)
            assert code == 0 and "status 0" in out, (B, S, T, modified, route, out[-4000:])


# ---- workgroups that really overlap ---------------------------------------------------------------

@slow
def test_overlapping_workgroups_give_the_bits_of_workgroups_in_order():
    """tests/cpu_build/pipelined_concurrent_main.cc: every workgroup of a launch in a child process
    of its own, six at a time, so that the chunks of a sequence, the two halves of the single
    launch and its backward tasks really run at the same time and wait for each other's words and
    counters in shared memory.  What a launch computes does not depend on how its workgroups
    interleave, so every output has to have the bits of the run with the workgroups in order; the
    workspace has to be clean and no wait expired.  Random shapes of one to three chunks, the pair
    with the log-derivative tensor, the single launch and the fp64 pair (mi_wave.hip), three
    overlapping runs each.

    That the workgroups do overlap is shown by a control: the same program over a copy of the
    kernels in which the take of a word between chunks does not wait for it.  In order that is
    harmless (every word is there before its reader starts); overlapping, a reader gets ahead of
    its writer: the outputs differ, or a word is left behind in the workspace."""
    import subprocess
    exe = _program("pipelined_concurrent", "pipelined_concurrent_main.cc")
    proc = subprocess.run([exe, "6", "3", "6", "11"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1800)
    assert proc.returncode == 0 and "all rounds done" in proc.stdout, proc.stdout[-3000:]
    text = open(os.path.join(ck.OUT, "mi_fast_host.hip")).read()
    wait = "    if (v != kSentinel) {\n      __hip_atomic_store(Global(word), kSentinel,"
    assert text.count(wait) == 1
    control_source = os.path.join(ck.OUT, "mi_fast_host_no_wait.hip")
    with open(control_source, "w") as f:
        f.write(text.replace(wait, wait.replace("v != kSentinel", "true")))
    control = _program("pipelined_concurrent_control", "pipelined_concurrent_main.cc", kernels=control_source)
    proc = subprocess.run([control, "6", "3", "6", "11"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=1800)
    assert proc.returncode == 1 and ("not the bits of the run in order" in proc.stdout
                                     or "workspace not clean" in proc.stdout), proc.stdout[-3000:]
