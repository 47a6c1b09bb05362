"""CPU-side checks of the drop-in boundary: the shared library loads without a GPU, exports every
symbol include/k2_amd.h declares (and the binding declares the same set), argument validation
returns error codes instead of launching, and the Python layer mirrors the reference's names."""
import inspect
import os
import re

import ctypes

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "k2_amd.h")).read()
    return sorted(set(re.findall(r"K2AMD_API\s+[\w\s\*]*?(k2amd_\w+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from k2_amd import capi
    lib = capi.lib()
    names = _declared()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/k2_amd.h but not exported"
    assert sorted(capi.exported_symbols()) == names
    assert lib.k2amd_version() == 100
    assert capi.lib().k2amd_status_string(0) == b"ok"


def test_invalid_arguments_return_codes_without_a_gpu():
    from k2_amd import capi
    lib = capi.lib()
    # negative sizes / unknown dtype are rejected before any HIP call
    assert lib.k2amd_mi_forward(None, None, None, None, None, -1, 1, 1, 0, 0, None, 0, None) == 1
    assert lib.k2amd_mi_forward(None, None, None, None, None, 1, 1, 1, 0, 7, None, 0, None) == 1
    assert lib.k2amd_mi_backward(None, None, None, None, None, None, None, 1, 1, 1, 0, 0, 0, None, 0, None) == 1
    assert lib.k2amd_mi_forward_keep(None, None, None, None, None, None, -1, 1, 1, 0, 0, None, 0, None) == 1
    assert lib.k2amd_mi_backward_kept(None, None, None, None, None, None, None, None, 1, 1, 1, 0, 9, 0, None, 0, None) == 1
    # p may only be left out where the log-derivative tensor stands in for it (fp32 with a workspace)
    one = ctypes.c_void_p(1)  # never dereferenced: the calls below are rejected on their arguments
    assert lib.k2amd_mi_forward_keep(one, one, None, None, one, None, 1, 1, 1, 0, 0, one, 1 << 20, None) == 1
    assert lib.k2amd_mi_forward_keep(one, one, None, None, one, one, 1, 1, 1, 0, 1, one, 1 << 20, None) == 1
    assert lib.k2amd_mi_forward_keep(one, one, None, None, one, one, 1, 1, 1, 0, 0, None, 0, None) == 1
    big = 1 << 20
    assert lib.k2amd_mi_forward_backward(one, one, None, one, None, big, one, one, one, 1, 1, 1, 0, 0, 1, one, big, None) == 1
    assert lib.k2amd_mi_forward_backward(one, one, None, one, one, big, one, one, one, 1, 1, 1, 0, 1, 1, one, big, None) == 2
    assert lib.k2amd_mi_forward_backward(None, None, None, None, None, 0, None, None, None, 0, 1, 1, 0, 0, 1, None, 0, None) == 0
    # scratch or workspace too small for the shape: refused before anything is launched
    assert lib.k2amd_mi_forward_backward(one, one, None, one, one, 16, one, one, one, 4, 10, 20, 0, 0, 1, one, big, None) == 3
    assert lib.k2amd_mi_forward_backward(one, one, None, one, one, big, one, one, one, 4, 10, 20, 0, 0, 1, one, 16, None) == 3
    assert lib.k2amd_mi_forward_backward_supported(4, 10, 20, 0, 1, 1) == 0
    assert lib.k2amd_mi_forward_backward_supported(4, 10, 20, 0, 0, 0) == 0
    # the single launch needs no particular number of resident workgroups: any batch is served
    assert lib.k2amd_mi_forward_backward_supported(4, 10, 20, 0, 0, 1) == 1
    assert lib.k2amd_mi_forward_backward_supported(2000, 200, 1000, 1, 0, 1) == 1
    assert lib.k2amd_mi_forward_backward_supported(4, 2055, 3000, 1, 0, 1) == 0   # more rows than its join keeps
    # per sequence: two halves x one chunk of 64 rows x one block of 32 positions (the cut of a
    # regular 10 x 20 lattice lies 15 diagonals in), in floats
    assert lib.k2amd_mi_forward_backward_scratch_bytes(4, 10, 20, 0, 0) == 4 * 2 * 64 * 32 * 4
    assert lib.k2amd_mi_forward_backward_scratch_bytes(32, 200, 1000, 1, 0) == 32 * 2 * 4 * 16 * 64 * 32 * 4
    assert lib.k2amd_mi_forward_backward_scratch_bytes(4, 10, 20, 0, 1) == 0
    # the log-derivative tensor is only used by the pipelined fp32 kernels, which need a workspace
    assert lib.k2amd_mi_keeps_log_deriv(4, 10, 20, 0, 0, 1) == 1
    assert lib.k2amd_mi_keeps_log_deriv(4, 10, 20, 0, 0, 0) == 0
    assert lib.k2amd_mi_keeps_log_deriv(4, 10, 20, 0, 1, 1) == 0
    assert lib.k2amd_mi_keeps_log_deriv(0, 10, 20, 0, 0, 1) == 0
    assert lib.k2amd_rnnt_prune_ranges(None, None, None, None, 1, 4, 4, 0, 9, 0, None) == 1
    assert lib.k2amd_rnnt_logprobs_joint_forward(None, None, None, None, None, None, 1, 1, 1, 4, 9, 0, 0, None) == 1
    # the simple builder's backward: scratch smaller than its query function says is refused
    # before anything is launched (B=2 S=5 T=9 C=7: 2 * (6*9 + 1*9 + 2*6*1) = 150 elements)
    # a batch beyond the launches' grid is a valid call that this build does not serve
    assert lib.k2amd_rnnt_logprobs_simple_forward(*([None] * 11), 70000, 5, 9, 7, 0, 0, 0, None) == 2
    need = lib.k2amd_rnnt_logprobs_simple_backward_scratch_elements(2, 5, 9)
    assert need == 150
    args = lambda n: (one, one, None, one, None, one, one, one, one, one, one, n, 2, 5, 9, 7, 0, 0, 0, None)
    assert lib.k2amd_rnnt_logprobs_simple_backward(*args(need - 1)) == 3
    assert lib.k2amd_rnnt_logprobs_simple_backward(one, one, None, one, None, one, one, one, one, one, None, need,
                                                   2, 5, 9, 7, 0, 0, 0, None) == 3
    # an empty batch is a no-op
    assert lib.k2amd_mi_forward(None, None, None, None, None, 0, 3, 3, 0, 0, None, 0, None) == 0
    with pytest.raises(RuntimeError):
        capi.check(2)


def test_python_api_mirrors_reference_signatures():
    import k2_amd as k2
    want = {
        "mutual_information_recursion": ["px", "py", "boundary", "return_grad"],
        "joint_mutual_information_recursion": ["px", "py", "boundary"],
        "get_rnnt_logprobs": ["lm", "am", "symbols", "termination_symbol", "rnnt_type", "boundary"],
        "rnnt_loss_simple": ["lm", "am", "symbols", "termination_symbol", "boundary", "rnnt_type",
                             "delay_penalty", "reduction", "return_grad"],
        "get_rnnt_logprobs_joint": ["logits", "symbols", "termination_symbol", "rnnt_type", "boundary"],
        "rnnt_loss": ["logits", "symbols", "termination_symbol", "boundary", "rnnt_type", "delay_penalty",
                      "reduction"],
        "get_rnnt_prune_ranges": ["px_grad", "py_grad", "boundary", "s_range"],
        "do_rnnt_pruning": ["am", "lm", "ranges"],
        "get_rnnt_logprobs_pruned": ["logits", "symbols", "ranges", "termination_symbol", "boundary",
                                     "rnnt_type"],
        "rnnt_loss_pruned": ["logits", "symbols", "ranges", "termination_symbol", "boundary", "rnnt_type",
                             "delay_penalty", "reduction", "use_hat_loss"],
        "get_hat_logprobs_pruned": ["logits", "symbols", "ranges", "termination_symbol", "boundary",
                                    "rnnt_type"],
        "get_rnnt_logprobs_smoothed": ["lm", "am", "symbols", "termination_symbol", "lm_only_scale",
                                       "am_only_scale", "boundary", "rnnt_type"],
        "rnnt_loss_smoothed": ["lm", "am", "symbols", "termination_symbol", "lm_only_scale",
                               "am_only_scale", "boundary", "rnnt_type", "delay_penalty", "reduction",
                               "return_grad"],
        "get_rnnt_prune_ranges_deprecated": ["px_grad", "py_grad", "boundary", "s_range"],
        "pruned_ranges_to_lattice": ["ranges", "frames", "symbols", "logits"],
    }
    for name, params in want.items():
        assert list(inspect.signature(getattr(k2, name)).parameters) == params, name


def test_cpu_tensors_fail_loudly():
    import torch
    import k2_amd as k2
    px = torch.zeros(1, 2, 4)
    py = torch.zeros(1, 3, 3)
    with pytest.raises(RuntimeError, match="no CPU path"):
        k2.mutual_information_recursion(px, py)
    # the reference's own assertions still come first
    with pytest.raises(AssertionError):
        k2.mutual_information_recursion(px, torch.zeros(1, 3, 7))
    with pytest.raises(AssertionError):
        k2.mutual_information_recursion(px, py, torch.tensor([[0, 0, 5, 3]]))


def test_pybind_host_module_mirrors_k2_native_functions():
    """The C++ host module carries the two functions of the reference's `_k2` for this path with
    the same keyword names (k2/python/csrc/torch/mutual_information.cu:26-67) and is the one the
    Python layer routes through."""
    import torch
    from k2_amd import _k2_amd, native
    assert native._ext is _k2_amd
    assert _k2_amd.version() == 100
    doc = _k2_amd.mutual_information_forward.__doc__
    assert all(k in doc for k in ("px:", "py:", "boundary:", "p:"))
    doc = _k2_amd.mutual_information_backward.__doc__
    assert all(k in doc for k in ("px:", "py:", "boundary:", "p:", "ans_grad:"))
    with pytest.raises(RuntimeError, match="no CPU path"):
        _k2_amd.mutual_information_forward(px=torch.zeros(1, 2, 3), py=torch.zeros(1, 3, 3),
                                           boundary=None, p=torch.zeros(1, 3, 4))
    with pytest.raises(RuntimeError, match="3-dimensional"):
        _k2_amd.mutual_information_forward(px=torch.zeros(2, 9), py=torch.zeros(1, 3, 3),
                                           boundary=None, p=torch.zeros(1, 3, 4))


def test_pybind_host_module_covers_every_builder_of_the_c_abi():
    """Each k2amd_rnnt_* entry point has a C++ host function, the Python layer's `native` module
    has a wrapper of the same name, and a host tensor is refused rather than computed on."""
    import torch
    from k2_amd import _k2_amd, native
    names = ("logprobs_simple_forward", "logprobs_simple_backward", "logprobs_joint_forward",
             "logprobs_joint_backward", "logprobs_pruned_forward", "logprobs_pruned_backward",
             "prune_ranges", "prune_gather", "prune_gather_backward", "pruned_ranges_to_lattice")
    for n in names:
        assert callable(getattr(_k2_amd, n)), n
        assert callable(getattr(native, n)), n
    sym = torch.zeros(1, 2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _k2_amd.logprobs_simple_forward(torch.zeros(1, 3, 5), torch.zeros(1, 4, 5), sym, 0, 0, None)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _k2_amd.logprobs_joint_forward(torch.zeros(1, 4, 3, 5), sym, 0, 0, None)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _k2_amd.prune_gather(torch.zeros(1, 3, 5), torch.zeros(1, 4, 2, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="no CPU path"):
        native.prune_ranges(torch.zeros(1, 2, 5), torch.zeros(1, 3, 4),
                            torch.tensor([[0, 0, 2, 4]]), 2)
    with pytest.raises(RuntimeError, match="no CPU path"):
        native.prune_ranges(torch.zeros(1, 2, 5), torch.zeros(1, 3, 4),
                            torch.tensor([[0, 0, 2, 4]]), 2, deprecated=True)


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """The boundary is a C ABI: include/k2_amd.h compiles as C99 without warnings, and a C program
    built with gcc alone links against libk2amd.so and gets status codes back from calls that
    are refused before anything touches a GPU."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    from k2_amd import capi
    header = os.path.join(ROOT, "include", "k2_amd.h")
    proc = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c", header],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    src = tmp_path / "caller.c"
    src.write_text('''
#include <stdio.h>
#include <string.h>
#include "k2_amd.h"
int main(void) {
  if (k2amd_version() != K2AMD_VERSION) return 1;
  if (strcmp(k2amd_status_string(K2AMD_OK), "ok") != 0) return 2;
  /* negative sizes, an unknown dtype, a window longer than S + 1: refused, nothing launched */
  if (k2amd_mi_forward(NULL, NULL, NULL, NULL, NULL, -1, 1, 1, 0, K2AMD_F32, NULL, 0, NULL) != K2AMD_ERR_INVALID_ARGUMENT) return 3;
  if (k2amd_rnnt_prune_ranges(NULL, NULL, NULL, NULL, 1, 4, 4, 0, 9, K2AMD_F32, NULL) != K2AMD_ERR_INVALID_ARGUMENT) return 4;
  if (k2amd_rnnt_prune_ranges_deprecated(NULL, NULL, NULL, NULL, 1, 4, 4, 0, 9, K2AMD_F32, NULL) != K2AMD_ERR_INVALID_ARGUMENT) return 5;
  if (k2amd_mi_workspace_bytes(32, 200, 1000, 1, K2AMD_F32) == 0) return 6;
  printf("c caller ok\\n");
  return 0;
}
''')
    lib_dir = os.path.dirname(capi._LIB_PATH)
    exe = tmp_path / "caller"
    proc = subprocess.run(["gcc", "-std=c99", "-Wall", f"-I{os.path.join(ROOT, 'include')}", str(src), "-o", str(exe),
                           f"-L{lib_dir}", "-lk2amd", f"-Wl,-rpath,{lib_dir}"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    proc = subprocess.run([str(exe)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and "c caller ok" in proc.stdout, (proc.returncode, proc.stdout)
