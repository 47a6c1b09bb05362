"""Writes tests/golden/mi_ref_fixtures.npz from the reference's own CPU code.

Run in a container that has the reference tree: it builds oracle/_ref/libk2ref.so (the
reference's k2/python/csrc/torch/mutual_information_cpu.cu + k2/csrc/log.cu compiled in place,
see oracle/Makefile) and records its outputs on small seeded inputs.  The fixture holds data
only: inputs, the outputs p / ans / px_grad / py_grad, and the case descriptors.

    python tests/golden/make_mi_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import mi  # noqa: E402
import cases  # noqa: E402


def main():
    mi.build_ref()
    out = {}
    names = []
    specs = []
    for seed in range(24):
        for dtype in (np.float32, np.float64):
            specs.append((f"rand{seed}_{np.dtype(dtype).name}",
                          cases.mi_case(seed, dtype=dtype, max_B=3, max_S=8, max_T=40)))
    # BASELINE config 1: B=2, S=10, T=20, regular, N(0,1), no boundary
    rng = np.random.default_rng(1)
    specs.append(("config1_float32", dict(
        px=rng.standard_normal((2, 10, 21)).astype(np.float32),
        py=rng.standard_normal((2, 11, 20)).astype(np.float32), boundary=None)))
    # -inf corner cases: unreachable end cell (modified with S_b > T_b is rejected upstream, but
    # -inf px everywhere reaches the same branch), and a regular lattice whose last px column
    # is -inf as get_rnnt_logprobs produces it.
    rng = np.random.default_rng(2)
    px = rng.standard_normal((2, 4, 7)).astype(np.float32)
    px[:, :, -1] = -np.inf
    specs.append(("neginf_lastcol_float32", dict(px=px, py=rng.standard_normal((2, 5, 6)).astype(np.float32),
                                                  boundary=None)))
    px = np.full((1, 3, 5), -np.inf, dtype=np.float32)
    specs.append(("neginf_all_px_float32", dict(px=px, py=rng.standard_normal((1, 4, 5)).astype(np.float32),
                                                 boundary=None)))
    for name, c in specs:
        px, py, bd = c["px"], c["py"], c["boundary"]
        ans, p = mi.mi_forward(px, py, bd, backend="ref")
        gx, gy = mi.mi_backward(px, py, bd, p, backend="ref")
        names.append(name)
        out[name + "/px"] = px
        out[name + "/py"] = py
        out[name + "/has_boundary"] = np.array(bd is not None)
        out[name + "/boundary"] = bd if bd is not None else np.zeros((0, 4), np.int64)
        out[name + "/p"] = p
        out[name + "/ans"] = ans
        out[name + "/px_grad"] = gx
        out[name + "/py_grad"] = gy
    out["names"] = np.array(names)
    path = os.path.join(HERE, "mi_ref_fixtures.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(names), "cases")


if __name__ == "__main__":
    main()
