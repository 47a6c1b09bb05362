"""bench.py's command line: what it must do without a GPU (the measured JSON line is checked on the
GPU box by the bench run itself)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args],
                          capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_defaults_are_the_headline_workload():
    r = _run("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--two-launches", "--no-keep"):
        assert flag in r.stdout
    import re
    src = open(os.path.join(ROOT, "bench.py")).read()
    for name, default in (("B", 32), ("S", 200), ("T", 1000), ("gpus", 1)):
        assert re.search(r'"--%s", type=int, default=%d\)' % (name, default), src), name
