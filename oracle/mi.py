"""TEST INFRASTRUCTURE ONLY: numpy front-end of the CPU checkers for the
mutual-information recursion.

Two back-ends with the same call signature:

* ``backend="port"``  -> ``oracle/libk2oracle.so`` built from ``mi_oracle.c`` (this repo's own
  restatement of k2/python/csrc/torch/mutual_information_cpu.cu:50-255);
* ``backend="ref"``   -> ``oracle/_ref/libk2ref.so``, the reference's own CPU sources compiled in
  place (only where that library has been built).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PORT_PATH = os.path.join(_HERE, "libk2oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libk2ref.so")
_port = None
_ref = None

_vp = ctypes.c_void_p
_ci = ctypes.c_int


def build_port():
    """Compile mi_oracle.c (a second or two with gcc)."""
    subprocess.check_call(["make", "-C", _HERE, "oracle"], stdout=subprocess.DEVNULL)


def build_ref(reference="/root/reference"):
    """Compile the reference's CPU sources in place; needs the reference tree."""
    subprocess.check_call(["make", "-C", _HERE, "ref", f"REFERENCE={reference}"],
                          stdout=subprocess.DEVNULL)


def port_lib():
    global _port
    if _port is None:
        if not os.path.exists(_PORT_PATH):
            build_port()
        _port = ctypes.CDLL(_PORT_PATH)
        for sfx in ("f32", "f64"):
            f = getattr(_port, f"k2o_mi_forward_{sfx}")
            f.argtypes = [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci]
            f.restype = None
            g = getattr(_port, f"k2o_mi_backward_{sfx}")
            g.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci]
            g.restype = _ci
        _port.k2o_log_add_f32.argtypes = [ctypes.c_float, ctypes.c_float]
        _port.k2o_log_add_f32.restype = ctypes.c_float
        _port.k2o_log_add_f64.argtypes = [ctypes.c_double, ctypes.c_double]
        _port.k2o_log_add_f64.restype = ctypes.c_double
    return _port


def have_ref():
    return os.path.exists(_REF_PATH)


def ref_lib():
    global _ref
    if _ref is None:
        import torch  # noqa: F401  (libk2ref.so links against libtorch)
        _ref = ctypes.CDLL(_REF_PATH)
        _ref.k2ref_mi_forward.argtypes = [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci]
        _ref.k2ref_mi_forward.restype = _ci
        _ref.k2ref_mi_backward.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                           _ci, _ci, _ci, _ci, _ci]
        _ref.k2ref_mi_backward.restype = _ci
    return _ref


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _shapes(px, py):
    B, S, T1 = px.shape
    T = py.shape[2]
    assert py.shape == (B, S + 1, T), (px.shape, py.shape)
    assert T1 in (T, T + 1)
    return B, S, T, int(T1 == T)


def _prep(px, py, boundary):
    assert px.dtype == py.dtype and px.dtype in (np.float32, np.float64)
    px = np.ascontiguousarray(px)
    py = np.ascontiguousarray(py)
    if boundary is not None:
        boundary = np.ascontiguousarray(boundary, dtype=np.int64)
        assert boundary.shape == (px.shape[0], 4)
    return px, py, boundary


def mi_forward(px, py, boundary=None, p=None, backend="port"):
    """Returns (ans[B], p[B,S+1,T+1]).  Cells of ``p`` outside the boundary box keep whatever
    the passed-in ``p`` held (NaN-filled when ``p`` is None), as in the reference, which
    leaves them uninitialised."""
    px, py, boundary = _prep(px, py, boundary)
    B, S, T, modified = _shapes(px, py)
    if p is None:
        p = np.full((B, S + 1, T + 1), np.nan, dtype=px.dtype)
    ans = np.empty((B,), dtype=px.dtype)
    f64 = px.dtype == np.float64
    if backend == "port":
        fn = getattr(port_lib(), "k2o_mi_forward_f64" if f64 else "k2o_mi_forward_f32")
        fn(_ptr(px), _ptr(py), _ptr(boundary), _ptr(p), _ptr(ans), B, S, T, modified)
    else:
        rc = ref_lib().k2ref_mi_forward(_ptr(px), _ptr(py), _ptr(boundary), _ptr(p), _ptr(ans),
                                        B, S, T, modified, int(f64))
        assert rc == 0
    return ans, p


def mi_backward(px, py, boundary, p, ans_grad=None, backend="port"):
    """Returns (px_grad, py_grad).  With ``boundary`` given, elements outside the box are 0
    (k2/python/csrc/torch/mutual_information_cpu.cu:160-166)."""
    px, py, boundary = _prep(px, py, boundary)
    B, S, T, modified = _shapes(px, py)
    T1 = px.shape[2]
    p = np.ascontiguousarray(p, dtype=px.dtype)
    if ans_grad is None:
        ans_grad = np.ones((B,), dtype=px.dtype)
    ans_grad = np.ascontiguousarray(ans_grad, dtype=px.dtype)
    px_grad = np.zeros((B, S, T1), dtype=px.dtype)
    py_grad = np.zeros((B, S + 1, T), dtype=px.dtype)
    f64 = px.dtype == np.float64
    if backend == "port":
        p_grad = np.empty((B, S + 1, T + 1), dtype=px.dtype)
        fn = getattr(port_lib(), "k2o_mi_backward_f64" if f64 else "k2o_mi_backward_f32")
        fn(_ptr(px), _ptr(py), _ptr(boundary), _ptr(p), _ptr(ans_grad), _ptr(p_grad),
           _ptr(px_grad), _ptr(py_grad), B, S, T, modified)
    else:
        rc = ref_lib().k2ref_mi_backward(_ptr(px), _ptr(py), _ptr(boundary), _ptr(p),
                                         _ptr(ans_grad), _ptr(px_grad), _ptr(py_grad),
                                         B, S, T, modified, int(f64))
        assert rc == 0
    return px_grad, py_grad


def mi(px, py, boundary=None, backend="port"):
    """Forward + backward with ans_grad = 1: (ans, px_grad, py_grad), the triple that
    k2.mutual_information_recursion(..., return_grad=True) returns
    (k2/python/k2/mutual_information.py:157-169)."""
    ans, p = mi_forward(px, py, boundary, backend=backend)
    gx, gy = mi_backward(px, py, boundary, p, backend=backend)
    return ans, gx, gy


def joint_mi(pxs, pys, boundary=None, backend="port"):
    """k2.joint_mutual_information_recursion (k2/python/k2/mutual_information.py:314-423): the
    recursion on the sums of the N px and N py, and the split of its score over the inputs,
    prods[n][b] = <occupation of the px edges, px_n> + <occupation of the py edges, py_n> with
    -inf inputs clamped to the dtype's most negative finite number, the rest of the score added to
    prods[0].  Returns (prods[N][B], px_occupation, py_occupation): the gradient of
    sum(w * prods) to px_n is w[n][b] times the occupation wherever px_n is above that clamp, the
    score itself carrying no gradient in the reference (it is computed outside autograd)."""
    N = len(pxs)
    assert len(pys) == N and N > 0
    dtype = np.asarray(pxs[0]).dtype
    px_tot = np.zeros_like(np.asarray(pxs[0]))
    py_tot = np.zeros_like(np.asarray(pys[0]))
    for n in range(N):  # torch.stack(...).sum(dim=0) adds the inputs in their order
        px_tot = px_tot + np.asarray(pxs[n], dtype=dtype)
        py_tot = py_tot + np.asarray(pys[n], dtype=dtype)
    tot, gx, gy = mi(px_tot, py_tot, boundary, backend=backend)
    lo = np.finfo(dtype).min
    B = px_tot.shape[0]
    prods = np.zeros((N, B), dtype=dtype)
    for n in range(N):
        cx = np.maximum(np.asarray(pxs[n], dtype=dtype), lo).reshape(B, -1)
        cy = np.maximum(np.asarray(pys[n], dtype=dtype), lo).reshape(B, -1)
        prods[n] = (np.einsum("bk,bk->b", gx.reshape(B, -1).astype(np.float64), cx.astype(np.float64)) +
                    np.einsum("bk,bk->b", gy.reshape(B, -1).astype(np.float64), cy.astype(np.float64))).astype(dtype)
    prods[0] += tot - prods.sum(axis=0)
    return prods, gx, gy


def log_add(x, y, dtype=np.float32):
    lib = port_lib()
    if dtype == np.float32:
        return np.float32(lib.k2o_log_add_f32(float(x), float(y)))
    return np.float64(lib.k2o_log_add_f64(float(x), float(y)))
