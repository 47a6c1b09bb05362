"""The library's HIP kernels compiled for the host (tests only): every kernel file.

g++ compiles the SAME sources as the GPU library over the thread stand-in of
tests/cpu_build/hip/hip_runtime.h into one shared library, whose C-ABI entry points then take
numpy buffers (or CPU tensors, through the product's own Python layer).  Most files use nothing
but plain HIP (LDS, barriers, wavefront shuffles, atomics); rnnt_simple.hip and joiner.hip besides
that the two matrix instructions (fp32 and bfloat16 operands), which the stand-in computes from
their documented operand layouts, mi_wave.hip two DPP lane shifts, readlane and agent-scope
atomics.  Two files are compiled from copies in which the lines that the host compiler cannot
parse are replaced, and not a character else (EDITS below): joiner.hip (three spellings) and
mi_fast.hip, the pipelined mutual-information kernels and the single launch, whose inline assembly
(two DPP arithmetic instructions, buffer loads, coherent loads and stores, wait counts) gives way
to calls that do what the instructions do.  The ctypes signatures are k2_amd/capi.py's own table,
so a wrong entry there shows up here as well.

What the host build cannot show: anything that depends on workgroups running at the same time
(they run one after the other here, which the kernels allow: every wait of theirs is for a
workgroup that started earlier), the memory model of the device (coherence between compute units,
wait counts), and timing.

Fenced arrays: a numpy array whose last byte sits directly in front of an inaccessible page (or
whose first byte directly behind one), so that a kernel reading or writing past the end of a
tensor stops the test run with a segmentation fault instead of passing unnoticed.
"""
import ctypes
import mmap
import os
import re
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "k2_amd", "csrc")
SHIM = os.path.join(HERE, "cpu_build")
# (a directory per process where the suite runs in several: tests/conftest.py)
OUT = os.path.join(SHIM, "_build", os.environ.get("PYTEST_XDIST_WORKER", ""))
PORTABLE = ["rnnt_rows", "prune", "lattice", "mi_joint", "mi_generic", "rnnt_smoothed", "rnnt_simple", "mi_capi", "mi_wave"]
# -ffp-contract=off: a * b + c rounds twice, as in the reference's CPU loops (the exact
# mutual-information kernels are compared with them bit for bit)
FLAGS = ["-std=c++20", "-O1", "-g", "-fPIC", "-pthread", "-ffp-contract=off", f"-I{SHIM}", f"-I{CSRC}"]

_lib = None


# Two sources hold lines that the host compiler cannot parse; the host build compiles copies in
# which exactly these are replaced and not a character else.  (old, new, count): a literal that
# must be found `count` times (None: at least once); a compiled pattern replaces every match.
EDITS = {
    "joiner": [
        ("typedef __bf16 Bf8 __attribute__((ext_vector_type(8)));", "typedef hip_threads_bf16x8 Bf8;", 1),
        ("return __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));", "return hip_threads_to_bf16(f);", 1),
        ("extern __shared__ __attribute__((aligned(16))) unsigned char smem[];", "HIP_DYNAMIC_SHARED(unsigned char, smem)", None),
    ],
    "mi_fast": [
        # the first half of a forward chain step (twice: natural and base-2 logarithms)
        ("""  asm volatile(
      "v_add_f32 %[x], %[P], %[fy]\\n\\t"
      "s_nop 0\\n\\t"
      "v_add_f32_dpp %[inc], %[P], %[inc] wave_shr:1 row_mask:0xf bank_mask:0xf\\n\\t"
      "v_max_f32 %[mx], %[inc], %[x]\\n\\t"
      "v_sub_f32 %[d], %[inc], %[x]"
      : [x] "=&v"(x), [inc] "+&v"(inc), [mx] "=&v"(mx), [d] "=&v"(d)
      : [P] "v"(P), [fy] "v"(fy));
""", """  x = P + fy;
  inc = hip_threads_add_from_lane_above(P, inc);
  mx = fmaxf(inc, x);
  d = inc - x;
""", 2),
        # a backward chain step
        ("""        asm volatile(
            "s_nop 1\\n\\t"
            "v_mul_f32_dpp %[t], %[G], %[t] wave_shl:1 row_mask:0xf bank_mask:0xf\\n\\t"
            "v_fmac_f32 %[t], %[O], %[G]"
            : [t] "+&v"(ts[e])
            : [O] "v"(os[e]), [G] "v"(G));
""", """        ts[e] = __builtin_fmaf(os[e], G, hip_threads_mul_from_lane_below(G, ts[e]));
""", 1),
        ('asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(v) : "v"(off), "s"(rs) : "memory");',
         "v = hip_threads_buffer_load4(rs, off);", 1),
        ('asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen sc1" : "=v"(v) : "v"(off), "s"(rs) : "memory");',
         "v = hip_threads_buffer_load4(rs, off);", 1),
        ('asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(ptr), "v"(w) : "memory");', "memcpy(ptr, &w, 16);", 1),
        ('asm volatile("global_load_dword %0, %1, off" : "=v"(gauge_v) : "v"(src) : "memory");', "gauge_v = *src;", 1),
        # waits for loads, and empty statements that only pin registers or keep branches apart
        (re.compile(r'asm volatile\("s_waitcnt[^;]*;'), ";", 4),
        (re.compile(r'asm volatile\(""[^;]*;'), ";", 10),
        # vector types whose elements the kernels name .x to .w
        ("typedef int int4v __attribute__((ext_vector_type(4)));", "typedef hip_threads_int4 int4v;", 1),
        ("typedef float float4v __attribute__((ext_vector_type(4)));", "typedef hip_threads_float4 float4v;", 1),
        ("typedef float QuadU __attribute__((ext_vector_type(4), aligned(4)));", "typedef hip_threads_float4 QuadU;", 1),
        # without address spaces this overload is the one in front of it
        ("__device__ __forceinline__ void StoreQuad(float *ptr, float4 v) { StoreQuad(Global(ptr), v); }\n", "", 1),
    ],
}


def _edited_source(name):
    text = open(os.path.join(CSRC, name + ".hip")).read()
    for old, new, count in EDITS[name]:
        if isinstance(old, str):
            found = text.count(old)
            text = text.replace(old, new)
        else:
            text, found = old.subn(new, text)
        assert found >= 1 and (count is None or found == count), (name, old, found)
    assert "asm" not in re.sub(r"//[^\n]*", "", text).replace("assembly", ""), name
    path = os.path.join(OUT, name + "_host.hip")
    with open(path, "w") as f:
        f.write(text)
    return path


def build():
    """Compiles the portable sources and tests/cpu_build/entry.cc into _build/libk2amd_cpu.so."""
    os.makedirs(OUT, exist_ok=True)
    jobs = []
    for name in PORTABLE + list(EDITS) + ["entry"]:
        src = os.path.join(CSRC, name + ".hip") if name != "entry" else os.path.join(SHIM, "entry.cc")
        if name in EDITS:
            src = _edited_source(name)
        obj = os.path.join(OUT, name + ".o")
        jobs.append((src, obj, subprocess.Popen(["g++", *FLAGS, "-x", "c++", "-c", src, "-o", obj],
                                                stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for src, _, proc in jobs:
        out, _ = proc.communicate()
        assert proc.returncode == 0, f"g++ failed on {src}\n{out}"
    path = os.path.join(OUT, "libk2amd_cpu.so")
    proc = subprocess.run(["g++", "-shared", "-pthread", "-o", path, *[j[1] for j in jobs]],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    return path


# The C++ host layer (k2_amd/csrc/pybind.cpp) for CPU tensors: a copy in which the places that
# touch the device are replaced, and not a character else, linked against the host build of the
# kernels.  What stays is what the GPU box runs of that file: every check, every allocation and
# its shape, the order and count of the C-ABI arguments, what is returned.
HOST_LAYER_PRELUDE = """
namespace { struct HostStream { void *stream() const { return nullptr; } }; }
"""
HOST_LAYER_EDITS = [
    ("#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>\n", "", 1),
    ("#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>\n", "", 1),
    ("#include <ATen/hip/HIPEvent.h>\n", HOST_LAYER_PRELUDE, 1),
    # the device guard: nothing to guard
    (re.compile(r"c10::hip::HIPGuardMasqueradingAsCUDA guard\([^;]*\);"), ";", None),
    # torch's current stream of a device: the null stream of the stand-in
    (re.compile(r"c10::hip::getCurrentHIPStreamMasqueradingAsCUDA\([^;]*?\)\.stream\(\)"), "nullptr", None),
    ("auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(boundary.device().index());", "HostStream stream;", 1),
    # the event behind the boundary copy: launches and copies are synchronous here
    ("    event_.record(stream);\n", "", 1),
    ("      event_.synchronize();\n", "", 1),
    ("  at::cuda::CUDAEvent event_;\n", "", 1),
    (".pinned_memory(true)", "", 2),
    # "is on the device" becomes "is a tensor"
    (".is_cuda()", ".defined()", None),
    ("->is_cuda()", "->defined()", None),
    ("PYBIND11_MODULE(_k2_amd, m)", "PYBIND11_MODULE(_k2_amd_host, m)", 1),
    # (the process has usually loaded the GPU build of this module too, with a class of this name)
    ('pybind11::class_<BoundaryRead>(m, "BoundaryRead")', 'pybind11::class_<BoundaryRead>(m, "BoundaryRead", pybind11::module_local())', 1),
]

_host_layer = None


def host_layer():
    """The module built from the edited copy of pybind.cpp (tests/cpu_build/_build/_k2_amd_host*.so)."""
    global _host_layer
    if _host_layer is not None:
        return _host_layer
    import importlib.util
    import sysconfig
    import pybind11
    import torch
    lib()  # the kernels it links against
    text = open(os.path.join(CSRC, "pybind.cpp")).read()
    for old, new, count in HOST_LAYER_EDITS:
        if isinstance(old, str):
            found = text.count(old)
            text = text.replace(old, new)
        else:
            text, found = old.subn(new, text)
        assert found >= 1 and (count is None or found == count), (old, found)
    assert "hip" not in re.sub(r"//[^\n]*", "", text).lower().replace("hipstream", ""), "a device call is left"
    src = os.path.join(OUT, "pybind_host.cpp")
    with open(src, "w") as f:
        f.write(text)
    tdir = os.path.dirname(torch.__file__)
    out = os.path.join(OUT, "_k2_amd_host" + sysconfig.get_config_var("EXT_SUFFIX"))
    cmd = ["g++", "-O0", "-std=c++17", "-fPIC", "-shared", "-DTORCH_EXTENSION_NAME=_k2_amd_host",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           f"-I{tdir}/include", f"-I{tdir}/include/torch/csrc/api/include", f"-I{sysconfig.get_paths()['include']}",
           f"-I{pybind11.get_include()}", f"-I{os.path.join(ROOT, 'include')}", "-fvisibility=hidden", src, "-o", out,
           f"-L{OUT}", "-lk2amd_cpu", "-Wl,-rpath,$ORIGIN", f"-L{tdir}/lib", f"-Wl,-rpath,{tdir}/lib",
           "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-4000:]
    spec = importlib.util.spec_from_file_location("_k2_amd_host", out)
    _host_layer = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(_host_layer)
    return _host_layer


def lib():
    global _lib
    if _lib is None:
        from k2_amd import capi
        _lib = ctypes.CDLL(build())
        for name, (argtypes, restype) in capi._SIGNATURES.items():
            if hasattr(_lib, name):
                fn = getattr(_lib, name)
                fn.argtypes, fn.restype = argtypes, restype
        vp, ci = ctypes.c_void_p, ctypes.c_int
        _lib.cpu_mi_forward_generic.argtypes = [vp] * 5 + [ci] * 5
        _lib.cpu_mi_backward_generic.argtypes = [vp] * 6 + [ci] * 6
    return _lib


_PAGE = mmap.PAGESIZE
_libc = ctypes.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]


class Fenced:
    """``.a``: an array of the given shape and dtype next to a page that may not be touched:
    behind its last element (at="end", the default) or in front of its first (at="start").  The
    other side, up to the page boundary, carries a pattern that ``intact()`` checks."""

    PATTERN = 0xA5

    def __init__(self, shape, dtype, fill=None, at="end"):
        dtype = np.dtype(dtype)
        n = int(np.prod(shape, dtype=np.int64))
        nbytes = n * dtype.itemsize
        pages = max(1, -(-nbytes // _PAGE))
        self.map = mmap.mmap(-1, (pages + 1) * _PAGE)
        self.buf = np.frombuffer(self.map, dtype=np.uint8)
        base = self.buf.ctypes.data
        assert base % _PAGE == 0
        if at == "end":
            guard, start = base + pages * _PAGE, pages * _PAGE - nbytes
            self.slack = slice(0, start)
        else:
            guard, start = base, _PAGE
            self.slack = slice(_PAGE + nbytes, (pages + 1) * _PAGE)
        self.buf[self.slack] = self.PATTERN
        if _libc.mprotect(guard, _PAGE, 0) != 0:
            raise OSError(ctypes.get_errno(), "mprotect")
        self.a = self.buf[start:start + nbytes].view(dtype).reshape(shape)
        if fill is not None:
            self.a[...] = fill

    def intact(self):
        return bool((self.buf[self.slack] == self.PATTERN).all())


def fenced(array, at="end"):
    """A fenced copy of ``array`` (None stays None)."""
    if array is None:
        return None
    f = Fenced(array.shape, array.dtype, at=at)
    f.a[...] = array
    return f


def p(x):
    """The pointer ctypes passes for a Fenced, a numpy array or None."""
    if x is None:
        return None
    a = x.a if isinstance(x, Fenced) else x
    return ctypes.c_void_p(a.ctypes.data)
