#!/usr/bin/env python3
"""Headline benchmark: MI recursion forward + backward on one MI355X.

Workload (BASELINE config 4): fp32, modified lattice, B=32, S=200, T=1000, px/py = min(N(-3,1), 0),
per-sequence boundary with T_b in [600,1000] and S_b in [100,200].  One step = the forward and
the backward recursion through the C-ABI (one launch: k2amd_mi_forward_backward), inputs resident
in HBM and taken in turn from eight copies, so that every step reads them from HBM rather than
from what the step before left in the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` counts ACTIVE lattice cells, sum_b (S_b+1)(T_b+1), per second of
fwd+bwd wall time on the GPU: the steps alone between two synchronisations.  `roofline` prices the
step's kernel (the slower of the two where two launches are asked for) against the HBM peak with
its algorithmic bytes and its average launch duration, which HIP events measure in a second pass
over the same steps (one event per ten launches of the single launch: an event between two
launches costs the GPU 3-4 us, which neither figure should carry); `cache_resident` is
the same measurement with one copy of the inputs; `cpu_baseline` is the reference's CPU loop on
this host.  `secondary`, `other_configs` and `fused_joiner` are further workloads through the Python
API (configs 3, 2, 5, and config 3's shape with the joiner inside the loss), none of them `value`.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# Algorithmic bytes per lattice cell, fp32: forward reads px, py and writes p (12 B); backward
# reads px, p and writes px_grad, py_grad (16 B; the backward never needs py).
FWD_BYTES_PER_CELL = 12
EVENT_GROUP = 10  # launches between two events of the pass that times the kernels
REPEATS = 5       # the timed region (--steps steps between two synchronisations) is run this often
BWD_BYTES_PER_CELL = 16

# HBM bytes per launch on the default workload, from rocprofv3's FETCH_SIZE / WRITE_SIZE counters
# scaled by a 256 MiB device copy (profiles/mi_bidir_kernel_c4_hbm_traffic.md).  Reported only
# for the default shape; any other --B/--S/--T prints null.
MEASURED_TRAFFIC_BYTES = {"mi_forward_backward": 141090000, "mi_forward": 50120000, "mi_backward": 69230000}
MEASURED_TRAFFIC_BYTES_PLAIN_PAIR = {"mi_forward": 50040000, "mi_backward": 85940000}  # --no-keep


def cpu_baseline(c, budget_s=12.0):
    """Times the CPU path on this host, single-threaded like the reference's loops
    (k2/python/csrc/torch/mutual_information_cpu.cu:89,179 have no parallel_for)."""
    from oracle import mi as omi
    kind = "reference" if omi.have_ref() else "port"
    backend = "ref" if kind == "reference" else "port"
    px, py, bd = c["px"], c["py"], c["boundary"]
    cells = int(((bd[:, 2] - bd[:, 0] + 1) * (bd[:, 3] - bd[:, 1] + 1)).sum())
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        ans, p = omi.mi_forward(px, py, bd, backend=backend)
        omi.mi_backward(px, py, bd, p, backend=backend)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {
        "value": cells / med, "unit": "cells/s", "cores": 1, "kind": kind,
        "sample": f"the same B={c['B']} S={c['S']} T={c['T']} workload, {len(times)} full fwd+bwd "
                  f"passes, median {med * 1e3:.1f} ms (host has {os.cpu_count()} logical cpus)",
    }


def _cpu_pruned_loss(logits, symbols, ranges, boundary, blank=0):
    """k2's CPU route for rnnt_loss_pruned, restated with torch CPU ops (the reference is a chain
    of torch ops, k2/python/k2/rnnt_loss.py:1180-1348, around its CPU recursion
    k2/python/csrc/torch/mutual_information_cpu.cu): log-softmax, gathers, dense px / py with -inf
    outside the band, the CPU lattice recursion, autograd back to the logits."""
    import torch
    from oracle import mi as omi
    backend = "ref" if omi.have_ref() else "port"
    B, T, R, C = logits.shape
    S = symbols.shape[1]

    class Lattice(torch.autograd.Function):
        @staticmethod
        def forward(ctx, px, py):
            npx, npy = px.detach().numpy(), py.detach().numpy()
            ans, p = omi.mi_forward(npx, npy, boundary.numpy(), backend=backend)
            gx, gy = omi.mi_backward(npx, npy, boundary.numpy(), p, backend=backend)
            ctx.save_for_backward(torch.from_numpy(gx), torch.from_numpy(gy))
            return torch.from_numpy(ans)

        @staticmethod
        def backward(ctx, g):
            gx, gy = ctx.saved_tensors
            return gx * g.reshape(-1, 1, 1), gy * g.reshape(-1, 1, 1)

    lp = torch.log_softmax(logits, dim=-1)
    s_idx = ranges  # [B,T,R] = s of each kept row
    sym_pad = torch.cat([symbols, torch.full((B, 1), blank, dtype=symbols.dtype)], dim=1)
    sym = torch.gather(sym_pad.unsqueeze(1).expand(B, T, S + 1), 2, s_idx)          # [B,T,R]
    px_band = torch.gather(lp, 3, sym.unsqueeze(-1)).squeeze(-1)                     # [B,T,R]
    py_band = lp[..., blank]                                                         # [B,T,R]
    t_end = boundary[:, 3].reshape(B, 1, 1)
    t_idx = torch.arange(T).reshape(1, T, 1)
    px_band = torch.where((s_idx < S) & (t_idx != t_end), px_band, torch.full_like(px_band, float("-inf")))
    px = torch.full((B, T, S + 1), float("-inf")).scatter(2, s_idx, px_band)[:, :, :S]
    py = torch.full((B, T, S + 1), float("-inf")).scatter(2, s_idx, py_band)
    px = torch.cat([px.permute(0, 2, 1), torch.full((B, S, 1), float("-inf"))], dim=2).contiguous()
    py = py.permute(0, 2, 1).contiguous()
    return -Lattice.apply(px, py).sum()


def pruned_secondary(dev, steps=None, cpu=True):
    """Second figure asked for next to the headline: pruned RNN-T loss forward + backward on
    BASELINE config 3 (B=32, T=500, S=100, V=500, s_range=5, regular lattice) in utterances/s,
    beside the CPU route on a sample of the same utterances."""
    steps = steps or SECONDARY_STEPS["pruned_secondary"]
    import torch
    import cases
    import k2_amd as k2
    B, T, S, C, R = (SHAPES["c3"][k] for k in ("B", "T", "S", "C", "R"))
    c = cases.rnnt_case(3, B, T, S, C, t_lo=SHAPES["c3"]["t_lo"], s_lo=SHAPES["c3"]["s_lo"])
    lm, am = torch.from_numpy(c["lm"]).to(dev), torch.from_numpy(c["am"]).to(dev)
    sym, bd = torch.from_numpy(c["symbols"]).to(dev), torch.from_numpy(c["boundary"]).to(dev)
    logits = torch.from_numpy(np.random.default_rng(33).standard_normal((B, T, R, C)).astype(np.float32)).to(dev)
    logits.requires_grad_(True)
    # Three copies taken in turn (480 MB): a step's logits then come from HBM, not from what the
    # steps before left in the 256 MB Infinity Cache, which holds one copy (160 MB) whole.
    logits_sets = [logits] + [logits.detach().clone().requires_grad_(True) for _ in range(LOGITS_SETS - 1)]
    turn = [0]

    # A training loop brings a new boundary tensor with every batch, and the functions read its
    # values on the host once per tensor (a device-to-host copy that waits for the stream): every
    # timed step gets a fresh clone, so that the figure includes that read.
    def simple_and_ranges():
        b = bd.clone()
        _, (gx, gy) = k2.rnnt_loss_simple(lm, am, sym, 0, b, reduction="sum", return_grad=True)
        return k2.get_rnnt_prune_ranges(gx, gy, b, R)

    def pruned(ranges, n_sets):
        x = logits_sets[turn[0] % n_sets]
        turn[0] += 1
        x.grad = None
        loss = k2.rnnt_loss_pruned(x, sym, ranges, 0, bd.clone(), reduction="sum")
        loss.backward()
        return loss

    ranges = simple_and_ranges()
    for _ in range(2 * LOGITS_SETS):
        pruned(ranges, LOGITS_SETS)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    torch.cuda.synchronize()
    ev[0].record()
    for _ in range(steps):
        ranges = simple_and_ranges()
    ev[1].record()
    for _ in range(steps):
        loss = pruned(ranges, LOGITS_SETS)
    ev[2].record()
    for _ in range(steps):
        pruned(ranges, 1)
    ev[3].record()
    torch.cuda.synchronize()
    t_ranges = ev[0].elapsed_time(ev[1]) / steps * 1e-3
    t_pruned = ev[1].elapsed_time(ev[2]) / steps * 1e-3
    t_cached = ev[2].elapsed_time(ev[3]) / steps * 1e-3
    # one read of the logits forward, one read + one write backward, fp32
    logits_bytes = 3 * logits.numel() * 4
    out = {
        "workload": "rnnt_loss_pruned fwd+bwd, fp32, regular, B=32 T=500 S=100 V=500 s_range=5 "
                    "(BASELINE config 3), ranges from an rnnt_loss_simple pass; a fresh boundary "
                    "tensor in every step (one host read of it per step, as in a training loop)",
        "value": B / t_pruned, "unit": "utterances/s", "ms_per_step": t_pruned * 1e3,
        "logits": f"taken in turn from {LOGITS_SETS} copies, {LOGITS_SETS * logits.numel() * 4 // 1000000} MB in "
                  "all: they come from HBM",
        "logits_GBps": logits_bytes / t_pruned / 1e9,
        "frac_of_hbm_peak": logits_bytes / t_pruned / 1e9 / HBM_PEAK_GBS,
        "roofline": {"bound": "hbm", "achieved": logits_bytes / t_pruned / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": logits_bytes / t_pruned / 1e9 / HBM_PEAK_GBS,
                     "bytes": "the logits read forward, read again and their gradient written backward (480 MB); "
                              "the whole step through the API, host launches included",
                     **PROFILED_KERNELS["c3_pruned"]},
        "cache_resident": {"logits": "the same 160 MB tensor every step, which the Infinity Cache holds",
                           "ms_per_step": t_cached * 1e3, "value": B / t_cached,
                           "logits_GBps": logits_bytes / t_cached / 1e9},
        "simple_pass_plus_prune_ranges_ms": t_ranges * 1e3,
        "loss": float(loss.detach()),
    }
    if cpu:
        n = B  # utterances in the CPU sample: the whole batch
        cl = logits.detach()[:n].cpu().requires_grad_(True)
        cs, cb, cr = sym[:n].cpu(), bd[:n].cpu(), ranges[:n].cpu()
        times = []
        for _ in range(10):
            cl.grad = None
            t0 = time.perf_counter()
            _cpu_pruned_loss(cl, cs, cr, cb).backward()
            times.append(time.perf_counter() - t0)
        med = float(np.median(times))
        out["cpu_baseline"] = {
            "value": n / med, "unit": "utterances/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the same {n} utterances, {len(times)} fwd+bwd passes, median "
                      f"{med * 1e3:.0f} ms (torch CPU ops with {torch.get_num_threads()} threads + "
                      "the single-threaded CPU recursion)"}
    return out


MFMA_PEAK_TFLOPS = {"fp32": 157.3, "bf16": 2500.0}  # MI355X published dense matrix rates
# BASELINE's configurations as the secondary workloads use them: B, T, S, V (, s_range), and the
# smallest T_b / S_b of the random boundaries.  (One place, so that a test can run this file's
# control flow on toy sizes.)
SHAPES = {"c2": dict(B=16, T=250, S=50, C=500, t_lo=150, s_lo=20),
          "c3": dict(B=32, T=500, S=100, C=500, R=5, t_lo=300, s_lo=50),
          "c5": dict(B=8, T=300, S=75, C=500, t_lo=200, s_lo=40),
          "c4": dict(B=32, S=200, T=1000)}
SECONDARY_STEPS = {"pruned_secondary": 50, "other_configs": 50, "fused_joiner": 20, "next_rows": 30}
LOGITS_SETS = 3  # copies of config 3's logits the secondary figures rotate over (see pruned_secondary)
# The dominant kernel of the secondary workloads and its average duration in the committed kernel
# trace of this file's default run (rocprofv3 --kernel-trace --stats; not measured by the run).
PROFILED_KERNELS = {
    "c3_pruned": {"kernel": "RowGradKernel (grid 5120000)", "kernel_avg_us": 52.8,
                  "kernel_source": "profiles/mi_bidir_kernel_c4_kernel_trace.md, the default run's table "
                                   "(recorded when every step read the same 160 MB of logits)"},
    "c5_joint": {"kernel": "RowGradKernel (grid 11673600)", "kernel_avg_us": 113.6,
                 "kernel_source": "profiles/mi_bidir_kernel_c4_kernel_trace.md, the default run's table"},
}


def fused_joiner(dev, steps=None):
    """The pruned loss with the joiner inside it (k2_amd.rnnt_loss_pruned_joiner) on BASELINE config
    3's shape with a joiner of D=512, forward + backward, beside the chain it replaces on the same
    device (do_rnnt_pruning, torch's tanh and linear, rnnt_loss_pruned).  FLOPs counted: the three
    products an implementation cannot avoid (logits, their gradient times the weight, the
    weight's gradient), 2 * B*T*s_range * D * V each; what the fused kernels multiply again when they
    recompute is not counted."""
    steps = steps or SECONDARY_STEPS["fused_joiner"]
    import torch
    import cases
    import k2_amd as k2
    B, T, S, C, R = (SHAPES["c3"][k] for k in ("B", "T", "S", "C", "R"))
    D = 512
    c = cases.rnnt_case(3, B, T, S, C, t_lo=SHAPES["c3"]["t_lo"], s_lo=SHAPES["c3"]["s_lo"])
    lm0, am0 = torch.from_numpy(c["lm"]).to(dev), torch.from_numpy(c["am"]).to(dev)
    sym, bd = torch.from_numpy(c["symbols"]).to(dev), torch.from_numpy(c["boundary"]).to(dev)
    _, (gx, gy) = k2.rnnt_loss_simple(lm0, am0, sym, 0, bd, reduction="sum", return_grad=True)
    ranges = k2.get_rnnt_prune_ranges(gx, gy, bd, R)
    g = torch.Generator(device="cpu").manual_seed(7)
    am = (0.8 * torch.randn(B, T, D, generator=g)).to(dev).requires_grad_(True)
    lm = (0.8 * torch.randn(B, S + 1, D, generator=g)).to(dev).requires_grad_(True)
    weight = (2.0 / D ** 0.5 * torch.randn(C, D, generator=g)).to(dev).requires_grad_(True)
    bias = (0.5 * torch.randn(C, generator=g)).to(dev).requires_grad_(True)

    def fused(precision):
        return k2.rnnt_loss_pruned_joiner(am, lm, ranges, weight, bias, sym, 0, bd, reduction="sum",
                                          precision=precision)

    def chain(autocast):
        am_p, lm_p = k2.do_rnnt_pruning(am, lm, ranges)
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            logits = torch.nn.functional.linear(torch.tanh(am_p + lm_p), weight, bias)
        return k2.rnnt_loss_pruned(logits.float(), sym, ranges, 0, bd, reduction="sum")

    def timed(fn):
        for _ in range(3):
            for t in (am, lm, weight, bias):
                t.grad = None
            loss = fn()
            loss.backward()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        torch.cuda.synchronize()
        ev[0].record()
        for _ in range(steps):
            for t in (am, lm, weight, bias):
                t.grad = None
            loss = fn()
            loss.backward()
        ev[1].record()
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / steps, float(loss.detach())

    flops = 3 * 2.0 * B * T * R * D * C
    out = {"workload": "do_rnnt_pruning -> tanh -> linear(D=512 -> V=500) -> rnnt_loss_pruned fwd+bwd, "
                       "B=32 T=500 S=100 s_range=5 (BASELINE config 3's shape), gradients to am, lm, "
                       "weight, bias; the fused call never stores the [B,T,s_range,V] logits",
           "algorithmic_GFLOP": flops / 1e9}
    for precision in ("fp32", "bf16"):
        ms, loss = timed(lambda: fused(precision))
        ms_chain, loss_chain = timed(lambda: chain(precision == "bf16"))
        out[precision] = {
            "ms_per_step": ms, "value": B / (ms * 1e-3), "unit": "utterances/s", "loss": loss,
            "roofline": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12,
                         "peak": MFMA_PEAK_TFLOPS[precision], "unit": "TFLOP/s",
                         "frac": flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS[precision]},
            "unfused_chain_ms_per_step": ms_chain, "unfused_chain_loss": loss_chain,
            "unfused_chain": "torch ops for the joiner" + (" under autocast(bfloat16)" if precision == "bf16" else "")
                             + " + k2_amd.rnnt_loss_pruned on its fp32 logits"}
    return out


def other_configs(dev, steps=None):
    """The two remaining BASELINE configurations, forward + backward through the k2-style API with
    gradients to the network outputs: config 2 (rnnt_loss_simple, B=16 T=250 S=50 V=500) and
    config 5 (rnnt_loss on the full joiner lattice, B=8 T=300 S=75 V=500)."""
    steps = steps or SECONDARY_STEPS["other_configs"]
    import torch
    import cases
    import k2_amd as k2

    def timed(fn):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e-3

    out = {}
    B, T, S, C = (SHAPES["c2"][k] for k in ("B", "T", "S", "C"))
    c = cases.rnnt_case(2, B, T, S, C, t_lo=SHAPES["c2"]["t_lo"], s_lo=SHAPES["c2"]["s_lo"])
    lm = torch.from_numpy(c["lm"]).to(dev).requires_grad_(True)
    am = torch.from_numpy(c["am"]).to(dev).requires_grad_(True)
    sym, bd = torch.from_numpy(c["symbols"]).to(dev), torch.from_numpy(c["boundary"]).to(dev)

    def simple():
        lm.grad = None
        am.grad = None
        k2.rnnt_loss_simple(lm, am, sym, 0, bd.clone(), reduction="sum").backward()

    t = timed(simple)
    # lm, am read once forward; their gradients written once backward
    nbytes = 2 * 4 * (lm.numel() + am.numel())
    out["c2_rnnt_loss_simple"] = {
        "workload": "rnnt_loss_simple fwd+bwd, fp32, regular, B=16 T=250 S=50 V=500 (BASELINE config 2)",
        "ms_per_step": t * 1e3, "utterances_per_s": B / t, "algorithmic_GBps": nbytes / t / 1e9,
        "frac_of_hbm_peak": nbytes / t / 1e9 / HBM_PEAK_GBS}
    del lm, am

    B, T, S, C = (SHAPES["c5"][k] for k in ("B", "T", "S", "C"))
    c = cases.rnnt_case(5, B, T, S, C, t_lo=SHAPES["c5"]["t_lo"], s_lo=SHAPES["c5"]["s_lo"])
    logits = torch.from_numpy(
        np.random.default_rng(55).standard_normal((B, T, S + 1, C)).astype(np.float32)).to(dev)
    logits.requires_grad_(True)
    sym, bd = torch.from_numpy(c["symbols"]).to(dev), torch.from_numpy(c["boundary"]).to(dev)

    def joint():
        logits.grad = None
        k2.rnnt_loss(logits, sym, 0, bd.clone(), reduction="sum").backward()

    t = timed(joint)
    nbytes = 3 * 4 * logits.numel()  # read forward; read + write backward
    out["c5_rnnt_loss"] = {
        "workload": "rnnt_loss fwd+bwd, fp32, regular, B=8 T=300 S=75 V=500 (BASELINE config 5)",
        "ms_per_step": t * 1e3, "utterances_per_s": B / t, "logits_GBps": nbytes / t / 1e9,
        "frac_of_hbm_peak": nbytes / t / 1e9 / HBM_PEAK_GBS,
        "logits": "one 365 MB tensor, larger than the 256 MB Infinity Cache: read from HBM in every step",
        "roofline": {"bound": "hbm", "achieved": nbytes / t / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": nbytes / t / 1e9 / HBM_PEAK_GBS,
                     "bytes": "the logits read forward, read again and their gradient written backward (1.09 GB); "
                              "the whole step through the API, host launches included",
                     **PROFILED_KERNELS["c5_joint"]}}
    return out


def next_rows(dev, steps=None):
    """The rows either side of the path that the library also serves, each once at a BASELINE shape:
    pruned_ranges_to_lattice and the HAT pruned loss on config 3's shape, the smoothed loss on
    config 2's, joint_mutual_information_recursion (two px / py pairs) on config 4's.  HIP-event
    time per call through the k2-style API (forward + backward for the losses, a fresh boundary
    tensor per step as in the other secondary figures), with the bytes each has to move at least."""
    steps = steps or SECONDARY_STEPS["next_rows"]
    import torch
    import cases
    import k2_amd as k2

    def timed(fn):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e-3

    def entry(workload, t, nbytes, what):
        return {"workload": workload, "ms_per_call": t * 1e3, "algorithmic_bytes": int(nbytes),
                "bytes_counted": what, "GBps": nbytes / t / 1e9, "frac_of_hbm_peak": nbytes / t / 1e9 / HBM_PEAK_GBS}

    out = {}
    B, T, S, C, R = (SHAPES["c3"][k] for k in ("B", "T", "S", "C", "R"))
    c = cases.rnnt_case(3, B, T, S, C, t_lo=SHAPES["c3"]["t_lo"], s_lo=SHAPES["c3"]["s_lo"])
    lm, am = torch.from_numpy(c["lm"]).to(dev), torch.from_numpy(c["am"]).to(dev)
    sym, bd = torch.from_numpy(c["symbols"]).to(dev), torch.from_numpy(c["boundary"]).to(dev)
    _, (gx, gy) = k2.rnnt_loss_simple(lm, am, sym, 0, bd, reduction="sum", return_grad=True)
    ranges = k2.get_rnnt_prune_ranges(gx, gy, bd, R)
    del lm, am, gx, gy
    logits = torch.from_numpy(
        np.random.default_rng(33).standard_normal((B, T, R, C)).astype(np.float32)).to(dev)
    ranges32, frames = ranges.to(torch.int32), bd[:, 3].to(torch.int32).contiguous()
    lattice, arc_map = k2.pruned_ranges_to_lattice(ranges32, frames, sym, logits)
    arcs = int(arc_map.numel())
    t = timed(lambda: k2.pruned_ranges_to_lattice(ranges32, frames, sym, logits))
    out["pruned_ranges_to_lattice"] = entry(
        f"pruned_ranges_to_lattice, fp32 logits, B={B} T={T} S={S} V={C} s_range={R} (config 3's shape): "
        f"{arcs} arcs; one host read of the two counts per call", t,
        arcs * (16 + 4 + 4) + ranges32.numel() * 4,
        "arc records 16 B + arc_map 4 B written and one logit read per arc, ranges read once")

    logits.requires_grad_(True)
    logits_sets = [logits] + [logits.detach().clone().requires_grad_(True) for _ in range(LOGITS_SETS - 1)]
    turn = [0]

    def hat():
        x = logits_sets[turn[0] % LOGITS_SETS]
        turn[0] += 1
        x.grad = None
        k2.rnnt_loss_pruned(x, sym, ranges, 0, bd.clone(), reduction="sum", use_hat_loss=True).backward()

    out["hat_pruned_loss"] = entry(
        f"rnnt_loss_pruned(use_hat_loss=True) fwd+bwd, fp32, regular, B={B} T={T} S={S} V={C} s_range={R}; "
        f"logits taken in turn from {LOGITS_SETS} copies (from HBM)",
        timed(hat), 3 * logits.numel() * 4, "logits read forward, read + gradient written backward")
    del logits, logits_sets

    B, T, S, C = (SHAPES["c2"][k] for k in ("B", "T", "S", "C"))
    c = cases.rnnt_case(2, B, T, S, C, t_lo=SHAPES["c2"]["t_lo"], s_lo=SHAPES["c2"]["s_lo"])
    lm = torch.from_numpy(c["lm"]).to(dev).requires_grad_(True)
    am = torch.from_numpy(c["am"]).to(dev).requires_grad_(True)
    sym, bd = torch.from_numpy(c["symbols"]).to(dev), torch.from_numpy(c["boundary"]).to(dev)

    def smoothed():
        lm.grad = None
        am.grad = None
        k2.rnnt_loss_smoothed(lm, am, sym, 0, lm_only_scale=0.25, am_only_scale=0.1, boundary=bd.clone(),
                              reduction="sum").backward()

    out["smoothed_loss"] = entry(
        f"rnnt_loss_smoothed fwd+bwd, fp32, regular, B={B} T={T} S={S} V={C} (config 2's shape)",
        timed(smoothed), 2 * 4 * (lm.numel() + am.numel()), "lm, am read forward; their gradients written backward")
    del lm, am

    B, S, T = (SHAPES["c4"][k] for k in ("B", "S", "T"))
    c = cases.c4_case(B=B, S=S, T=T)
    px, py, bd = (torch.from_numpy(c[k]).to(dev) for k in ("px", "py", "boundary"))
    pxs, pys = (px * 0.75, px * 0.25), (py * 0.75, py * 0.25)
    t = timed(lambda: k2.joint_mutual_information_recursion(pxs, pys, bd))
    out["joint_mutual_information_recursion"] = entry(
        f"joint_mutual_information_recursion, two px / py pairs, fp32, modified, B={B} S={S} T={T} (config 4's shape)",
        t, 4 * (2 + 1 + 1 + 1 + 3) * (px.numel() + py.numel()),
        "the two pairs read and their sum written, the sum read by the recursion, the occupation "
        "probabilities written, then read once with the two pairs for the split (full box)")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the pruned-loss figure (BASELINE config 3) in the 'secondary' field")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain device copy of 256 MiB before the warmup: the unit "
                         "against which rocprofv3's FETCH_SIZE / WRITE_SIZE readings are scaled")
    ap.add_argument("--two-launches", action="store_true",
                    help="run the forward and the backward as two launches where one would do")
    ap.add_argument("--no-keep", action="store_true",
                    help="run the plain forward/backward pair (no log-derivative tensor between them)")
    ap.add_argument("--input-sets", type=int, default=8,
                    help="rotate over this many copies of px / py in device memory, so that a step's "
                         "inputs are not what the previous steps left in the 256 MB Infinity Cache "
                         "(8 copies at the default shape are 410 MB); 1 = the same inputs every step")
    ap.add_argument("--no-cache-resident", action="store_true",
                    help="skip the second measurement on one copy of the inputs ('cache_resident')")
    ap.add_argument("--device", default="cuda:0",
                    help="where the tensors live; anything but a GPU only makes sense under a test that "
                         "stands in for the library (the library itself refuses host tensors)")
    ap.add_argument("--B", type=int, default=32)
    ap.add_argument("--S", type=int, default=200)
    ap.add_argument("--T", type=int, default=1000)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (sequences are "
              "independent, so the batch axis is what would be sharded); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    import cases
    from k2_amd import capi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device(args.device)
    c = cases.c4_case(B=args.B, S=args.S, T=args.T)
    px = torch.from_numpy(c["px"]).to(dev)
    py = torch.from_numpy(c["py"]).to(dev)
    bd = torch.from_numpy(c["boundary"]).to(dev)
    B, S, T = c["B"], c["S"], c["T"]
    bnp = c["boundary"]
    active = int(((bnp[:, 2] - bnp[:, 0] + 1) * (bnp[:, 3] - bnp[:, 1] + 1)).sum())
    full = B * (S + 1) * (T + 1)
    ones = torch.ones(B, dtype=torch.float32, device=dev)
    # as mutual_information_recursion does: the forward hands the backward the px-edge
    # log-derivatives (one more [B][S+1][T+1] tensor written by the forward, read by the backward)
    # (the forward then writes that tensor in place of p)
    keep = not args.no_keep and capi.mi_keeps_log_deriv(px, py)
    lattice = torch.empty(B, S + 1, T + 1, dtype=torch.float32, device=dev)
    p, log_deriv = (None, lattice) if keep else (lattice, None)

    # ... and both recursions run in ONE launch, again as mutual_information_recursion does
    single = keep and not args.two_launches and capi.mi_forward_backward_supported(px, py)

    def measure(n_sets):
        """Times args.steps steps after args.warmup; px / py taken in turn from n_sets copies."""
        sets = [(px, py)] + [(px.clone(), py.clone()) for _ in range(n_sets - 1)]
        turn = [0]

        def step(ev=None):
            x, y = sets[turn[0] % len(sets)]
            turn[0] += 1
            if single:
                return capi.mi_forward_backward(x, y, bd, ones, overwrite_ans_grad=False)
            if ev is not None:
                ev[0].record()
            capi.mi_forward(x, y, bd, p, log_deriv=log_deriv)
            if ev is not None:
                ev[1].record()
            g = capi.mi_backward(x, y, bd, p, ones, overwrite_ans_grad=False, log_deriv=log_deriv)
            if ev is not None:
                ev[2].record()
            return g

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        # The timed region: exactly args.steps steps between two synchronisations, nothing else on
        # the stream (an event recorded between two launches costs the GPU 3-4 us, 7 % of this
        # step).  The kernels' durations come from a second pass over the same steps.
        # The region is run REPEATS times and the median reported (a region of 20 steps lasts a
        # millisecond: one sample of it says little).
        walls = []
        for _ in range(REPEATS):
            t0 = time.perf_counter()
            for k in range(args.steps):
                step()
            torch.cuda.synchronize()
            walls.append((time.perf_counter() - t0) / args.steps * 1e3)
        m = {"ms_per_step": float(np.median(walls)), "ms_per_step_repeats": walls,
             "input_mb": len(sets) * (px.numel() + py.numel()) * 4 // 1000000}
        events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
        torch.cuda.synchronize()
        if single:
            # one kernel does the step: its algorithmic bytes are the forward's plus the backward's.
            # An event every EVENT_GROUP launches: the average launch (kernel + the gap to the next
            # one) of each group, without an event's own cost inside every launch.
            group = max(1, min(EVENT_GROUP, args.steps))
            marks = []
            for k in range(args.steps):
                if k % group == 0:
                    events[k][0].record()
                    marks.append(k)
                step()
            events[-1][2].record()
            torch.cuda.synchronize()
            ends = [events[k][0] for k in marks[1:]] + [events[-1][2]]
            counts = [b - a for a, b in zip(marks, marks[1:] + [args.steps])]
            both_ms = np.array([events[k][0].elapsed_time(end) / n for k, end, n in zip(marks, ends, counts)])
            m.update(dom="mi_forward_backward", dom_ms=float(both_ms.mean()), dom_bytes=both_bytes,
                     both_avg=float(both_ms.mean()),
                     kernel_times={"mi_forward_backward_avg_us": float(both_ms.mean()) * 1e3,
                                   "mi_forward_backward_min_us": float(both_ms.min()) * 1e3,
                                   "launches_per_event": group})
        else:
            for k in range(args.steps):
                step(events[k])
            torch.cuda.synchronize()
            fwd_ms = np.array([e[0].elapsed_time(e[1]) for e in events])
            bwd_ms = np.array([e[1].elapsed_time(e[2]) for e in events])
            # Roofline of the dominant kernel (the one with the longer average launch).
            fwd_avg, bwd_avg = float(fwd_ms.mean()), float(bwd_ms.mean())
            if bwd_avg >= fwd_avg:
                m.update(dom="mi_backward", dom_ms=bwd_avg, dom_bytes=BWD_BYTES_PER_CELL * active)
            else:
                m.update(dom="mi_forward", dom_ms=fwd_avg, dom_bytes=FWD_BYTES_PER_CELL * active)
            m.update(both_avg=fwd_avg + bwd_avg,
                     kernel_times={"mi_forward_avg_us": fwd_avg * 1e3, "mi_forward_min_us": float(fwd_ms.min()) * 1e3,
                                   "mi_backward_avg_us": bwd_avg * 1e3, "mi_backward_min_us": float(bwd_ms.min()) * 1e3})
        del sets
        return m

    if args.copy_probe:
        src = torch.zeros(64 << 20, dtype=torch.float32, device=dev)  # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    both_bytes = (FWD_BYTES_PER_CELL + BWD_BYTES_PER_CELL) * active
    m = measure(args.input_sets)
    ms_per_step, dom, dom_ms, dom_bytes, both_avg = m["ms_per_step"], m["dom"], m["dom_ms"], m["dom_bytes"], m["both_avg"]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    traffic_table = (MEASURED_TRAFFIC_BYTES if keep else MEASURED_TRAFFIC_BYTES_PLAIN_PAIR)
    out = {
        "metric": "MI recursion fwd+bwd lattice-cells/s (B=32,S=200,T=1000) + % HBM roofline",
        "value": active / (ms_per_step * 1e-3),
        "unit": "cells/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"mutual_information_recursion fwd+bwd, fp32, modified, B={B} "
                               f"S={S} T={T}, random boundary (BASELINE config 4)",
                   "active_cells": active, "full_box_cells": full, "log_deriv_kept": bool(keep),
                   "launches_per_step": 1 if single else 2, "input_sets": args.input_sets,
                   "timed_region": f"{args.steps} steps between two synchronisations, run {REPEATS} times; "
                                   "ms_per_step is the median of the runs",
                   "ms_per_step_of_each_run": m["ms_per_step_repeats"],
                   "inputs": ("the same px / py every step: at this size the Infinity Cache serves them from "
                              "the second step on, as it does after the builder kernels of the loss functions"
                              if args.input_sets == 1 else
                              "px / py taken in turn from %d copies, %d MB in all: they come from HBM"
                              % (args.input_sets, m["input_mb"]))},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic_table.get(dom) if (B, S, T) == (32, 200, 1000) else None,
                     "traffic_source": "rocprofv3 FETCH_SIZE + WRITE_SIZE of this kernel on this workload, from the "
                                       "committed profile (profiles/mi_bidir_kernel_c4_hbm_traffic.md); not "
                                       "measured by this run",
                     "kernel": dom,
                     "kernel_avg_us": dom_ms * 1e3},
        "kernels": dict(m["kernel_times"],
                        fwd_bwd_GBps_active_cells=both_bytes / (both_avg * 1e-3) / 1e9,
                        fwd_bwd_frac_of_hbm_peak=both_bytes / (both_avg * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        full_box_cells_per_s=full / (both_avg * 1e-3)),
    }
    if args.input_sets > 1 and not args.no_cache_resident:
        # the same steps on ONE copy of the inputs, which the Infinity Cache then serves (the
        # situation inside the loss functions, where a builder kernel has just written px / py)
        r = measure(1)
        out["cache_resident"] = {
            "inputs": "the same px / py every step",
            "ms_per_step": r["ms_per_step"], "value": active / (r["ms_per_step"] * 1e-3), "unit": "cells/s",
            "kernel": r["dom"], "kernel_avg_us": r["dom_ms"] * 1e3,
            "frac_of_hbm_peak": r["dom_bytes"] / (r["dom_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(c)
    if not args.no_secondary:
        del px, py, p
        # None of these is `value`: a failure in one of them is reported in its field and does not
        # take the headline's line with it.
        for field, part in (("secondary", lambda: pruned_secondary(dev, cpu=not args.no_cpu)),
                            ("other_configs", lambda: other_configs(dev)),
                            ("fused_joiner", lambda: fused_joiner(dev)),
                            ("next_rows", lambda: next_rows(dev))):
            try:
                out[field] = part()
            except Exception as e:  # noqa: BLE001 - whatever it is, the line below still has to come out
                out[field] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
