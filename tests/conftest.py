import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


CPU_SUITE_WORKERS = 4


@pytest.hookimpl(tryfirst=True)
def pytest_cmdline_main(config):
    """The CPU suite (-m "not gpu") spends most of its time in the host build of the kernels, where
    every work-item is a thread and a test mostly waits at barriers: its files run in a few
    processes side by side (pytest-xdist where it is installed, a file to a process, each process
    with a build directory of its own: tests/cpu_kernels.py::OUT).  Everything else, the GPU
    tests above all, runs in ONE process as before; so does the CPU suite with an explicit -n or
    with K2AMD_TEST_WORKERS=0."""
    if hasattr(config, "workerinput") or not config.pluginmanager.hasplugin("xdist"):
        return
    option = config.option
    try:
        workers = int(os.environ.get("K2AMD_TEST_WORKERS", CPU_SUITE_WORKERS))
    except ValueError:
        workers = CPU_SUITE_WORKERS
    if (option.markexpr or "").strip() != "not gpu" or workers < 2:
        return
    if option.numprocesses is not None or option.dist != "no" or option.tx or option.collectonly or option.usepdb:
        return
    option.numprocesses = workers
    option.dist = "loadfile"
    option.tx = ["popen"] * workers


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def _seeded():
    """Every test starts from the same state of torch's default generators (CPU and GPU), so that
    inputs drawn without a generator of their own are the same in every run and a tolerance that
    holds once holds always."""
    import torch
    torch.manual_seed(20240531)
    yield
