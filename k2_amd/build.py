"""Builds the native parts of k2_amd in-tree for gfx950.

  libk2amd.so   - HIP kernels + C-ABI (hipcc, no torch dependency)
  _k2_amd*.so   - pybind11 host module taking torch tensors (links libk2amd.so)

hipcc cross-compiles without a GPU, so this runs on any machine with ROCm installed.
"""
import glob
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libk2amd.so")
ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def pybind_module_path():
    return os.path.join(HERE, "_k2_amd" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_kernels(verbose=False):
    """Compiles every .hip file under csrc/ into libk2amd.so."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = []
    procs = []
    for src in srcs:
        obj = os.path.splitext(src)[0] + ".o"
        objs.append(obj)
        procs.append((src, subprocess.Popen(["hipcc", *HIP_FLAGS, "-c", src, "-o", obj],
                                            stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                                            text=True)))
    for src, proc in procs:
        out, _ = proc.communicate()
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}\n{out}")
        if verbose:
            print("compiled", os.path.basename(src))
    _run(["hipcc", f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


def build_pybind(verbose=False):
    """Compiles csrc/pybind.cpp (torch + pybind11 host layer) against libk2amd.so."""
    src = os.path.join(CSRC, "pybind.cpp")
    if not os.path.exists(src):
        return None
    import pybind11
    import torch
    tdir = os.path.dirname(torch.__file__)
    out = pybind_module_path()
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_k2_amd",
        "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        f"-I{tdir}/include", f"-I{tdir}/include/torch/csrc/api/include",
        f"-I{sysconfig.get_paths()['include']}", f"-I{pybind11.get_include()}",
        "-I/opt/rocm/include", f"-I{os.path.join(HERE, '..', 'include')}",
        src, "-o", out,
        f"-L{HERE}", "-lk2amd", "-Wl,-rpath,$ORIGIN",
        f"-L{tdir}/lib", f"-Wl,-rpath,{tdir}/lib",
        "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python", "-ltorch_hip", "-lc10_hip",
    ]
    _run(cmd)
    if verbose:
        print("built", os.path.basename(out))
    return out


def build_all(verbose=False):
    build_kernels(verbose)
    build_pybind(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    sys.exit(0)
