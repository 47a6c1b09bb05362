"""Kernels under host sanitizers (the builders' with K2AMD_SLOW_CPU_TESTS=1 only: minutes each; the
exact recursion and the prune ranges without their LDS rows always): programs of their own, built from the same kernel sources over the thread stand-in
(tests/cpu_build/hip/hip_runtime.h) and a small driver that calls the C-ABI on random inputs in
heap buffers of exactly the documented sizes.

-fsanitize=thread sees every work-item as a thread; what orders two of them is what orders two
wavefronts on the device (the workgroup's barrier, an atomic) or two lanes of one wavefront (an
exchange, a wave barrier).  No report means that no wavefront reads or writes LDS or device memory
that another one writes without such an ordering in between, on the driver's shapes.
-fsanitize=address,undefined ends the program at an access outside a buffer or outside the LDS
that a launch asked for.

The pipelined mutual-information kernels have the same two runs, and a control that shows the
thread sanitizer reporting a race that is really there, in tests/test_cpu_build_pipelined.py; the
smoothed builder's address-sanitizer run is in tests/test_cpu_build_smoothed.py."""
import os
import subprocess

import pytest

import cpu_kernels as ck

slow = pytest.mark.skipif(os.environ.get("K2AMD_SLOW_CPU_TESTS", "0") != "1",
                          reason="minutes on eight cores: run with K2AMD_SLOW_CPU_TESTS=1")


def _program(name, sanitizer, sources):
    ck.build()  # (writes the host copies of the sources that need one)
    runtime = "-static-libtsan" if sanitizer == "thread" else "-static-libasan"
    flags = [f for f in ck.FLAGS if f != "-fPIC"] + ["-fsanitize=" + sanitizer, "-fno-sanitize-recover=all"]
    jobs = []
    for src in sources:
        obj = os.path.join(ck.OUT, name + "_" + os.path.basename(src).split(".")[0] + ".o")
        jobs.append((obj, subprocess.Popen(["g++", *flags, "-x", "c++", "-c", src, "-o", obj], stdout=subprocess.PIPE,
                                           stderr=subprocess.STDOUT, text=True)))
    for obj, proc in jobs:
        out, _ = proc.communicate()
        assert proc.returncode == 0, out[-3000:]
    exe = os.path.join(ck.OUT, name)
    proc = subprocess.run(["g++", "-pthread", "-fsanitize=" + sanitizer, runtime, "-o", exe] + [j[0] for j in jobs],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-3000:]
    return exe


def _run(exe):
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 report_signal_unsafe=0 exitcode=0")
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=3000, env=env)
    if "FATAL: ThreadSanitizer" in proc.stdout:
        pytest.skip("the thread sanitizer does not start here: " + proc.stdout[:200])
    assert proc.returncode == 0 and "all shapes done" in proc.stdout, proc.stdout[-4000:]
    assert "Sanitizer" not in proc.stdout, proc.stdout[-4000:]


BUILDERS = [os.path.join(ck.OUT, "joiner_host.hip"), os.path.join(ck.CSRC, "rnnt_simple.hip"),
            os.path.join(ck.SHIM, "builders_sanitizer_main.cc")]


@slow
@pytest.mark.parametrize("sanitizer", ["thread", "address,undefined"])
def test_simple_builder_and_fused_joiner(sanitizer):
    """get_rnnt_logprobs' kernels (fp32 through the matrix instruction, fp64; S = 0 and T = 0 among
    the shapes) and the fused joiner's (fp32 and bfloat16 operands, with and without HAT, with and
    without a bias, all three lattice types), forward and backward."""
    _run(_program("builders_" + sanitizer.split(",")[0], sanitizer, BUILDERS))


@slow
def test_smoothed_builder_under_the_thread_sanitizer():
    _run(_program("smoothed_thread", "thread", [os.path.join(ck.SHIM, "smoothed_sanitizer_main.cc")]))


ROWLESS = [os.path.join(ck.CSRC, "mi_generic.hip"), os.path.join(ck.CSRC, "prune.hip"),
           os.path.join(ck.SHIM, "rowless_sanitizer_main.cc")]


@pytest.mark.parametrize("sanitizer", ["thread", "address,undefined"])
def test_exact_recursion_and_prune_ranges_without_lds_rows(sanitizer):
    """The forms that read the previous step back from the kernel's own output (mi_generic.hip past
    8190 / 4094 rows, prune.hip past 8192 frames; selected here by their switches) and the kernel
    of get_rnnt_prune_ranges_deprecated."""
    _run(_program("rowless_" + sanitizer.split(",")[0], sanitizer, ROWLESS))
