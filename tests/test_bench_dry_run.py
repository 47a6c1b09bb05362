"""bench.py's control flow on toy sizes and CPU tensors, over the host build of the kernels: every
section runs, the one JSON line comes out with the fields the contract names, the median of the
repeated timed region is what it says, a section that fails (the fused joiner's, made to: at
D = 512 it takes minutes on threads, and it ran through once this way while this was written) is
reported in its field without taking the line with it.  Figures are meaningless here; the point
is that a mistake in the script shows before a GPU is spent on it."""
import contextlib
import io
import json
import os
import sys
import time
import types

import numpy as np
import pytest
import torch

import cpu_kernels as ck

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

slow = pytest.mark.skipif(os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1",
                          reason="most of a minute on eight cores: run with K2AMD_SLOW_CPU_TESTS=1")


class _Event:
    def __init__(self, enable_timing=False):
        self.at = None

    def record(self, stream=None):
        self.at = time.perf_counter()

    def elapsed_time(self, other):
        return (other.at - self.at) * 1e3

    def synchronize(self):
        pass


@slow
def test_every_section_runs_and_the_line_is_whole(monkeypatch):
    from k2_amd import capi, native
    cpu_lib = ck.lib()
    monkeypatch.setattr(capi, "lib", lambda: cpu_lib)
    monkeypatch.setattr(capi, "_on_device", lambda t: True)
    monkeypatch.setattr(capi, "stream_ptr", lambda device: None)
    monkeypatch.setattr(capi, "_workspaces", {})
    monkeypatch.setattr(native, "_ext", None)
    monkeypatch.setattr(native, "_require_device", lambda t: None)
    monkeypatch.setattr(torch.cuda, "device", lambda device: contextlib.nullcontext())
    monkeypatch.setattr(torch.cuda, "current_stream", lambda device=None: types.SimpleNamespace(cuda_stream=0))
    monkeypatch.setattr(torch.cuda, "current_device", lambda: 0)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda device=None: None)
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "Event", _Event)
    monkeypatch.syspath_prepend(ROOT)
    import bench
    monkeypatch.setattr(bench, "SHAPES", {"c2": dict(B=2, T=9, S=4, C=7, t_lo=7, s_lo=2),
                                           "c3": dict(B=2, T=12, S=5, C=9, R=3, t_lo=9, s_lo=3),
                                           "c5": dict(B=2, T=9, S=4, C=7, t_lo=7, s_lo=2),
                                           "c4": dict(B=2, S=5, T=12)})
    monkeypatch.setattr(bench, "SECONDARY_STEPS", {k: 2 for k in bench.SECONDARY_STEPS})

    def failing_section(dev, steps=None):
        raise RuntimeError("made to fail")
    monkeypatch.setattr(bench, "fused_joiner", failing_section)
    monkeypatch.setattr(sys, "argv", ["bench.py", "--device", "cpu", "--B", "2", "--S", "5", "--T", "12", "--steps", "3",
                                      "--warmup", "1", "--input-sets", "2"])
    out = io.StringIO()
    with contextlib.redirect_stdout(out):
        bench.main()
    lines = [l for l in out.getvalue().splitlines() if l.strip()]
    assert len(lines) == 1, lines
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["steps"] == 3 and line["warmup"] == 1 and line["n_gpus"] == 1 and line["vs_baseline"] is None
    runs = line["config"]["ms_per_step_of_each_run"]
    assert len(runs) == bench.REPEATS and line["ms_per_step"] == pytest.approx(float(np.median(runs)))
    assert set(line["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "kernel_avg_us"}
    assert line["roofline"]["traffic"] is None  # not the default shape: no measured figure to quote
    assert set(line["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    assert "cache_resident" in line
    for section in ("secondary", "other_configs", "next_rows"):
        assert "error" not in line[section], line[section]
    assert set(line["secondary"]["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "kernel", "kernel_avg_us"}
    assert "cache_resident" in line["secondary"] and "cpu_baseline" in line["secondary"]
    assert "roofline" in line["other_configs"]["c5_rnnt_loss"]
    assert set(line["next_rows"]) == {"pruned_ranges_to_lattice", "hat_pruned_loss", "smoothed_loss",
                                      "joint_mutual_information_recursion"}
    assert "made to fail" in line["fused_joiner"]["error"]  # the line stands all the same


def test_more_than_one_gpu_is_declined(monkeypatch, capsys):
    monkeypatch.syspath_prepend(ROOT)
    import bench
    monkeypatch.setattr(sys, "argv", ["bench.py", "--gpus", "2"])
    with pytest.raises(SystemExit) as e:
        bench.main()
    assert e.value.code == 2 and "one GPU" in capsys.readouterr().err
