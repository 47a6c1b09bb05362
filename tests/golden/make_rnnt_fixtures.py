"""Writes tests/golden/rnnt_ref_fixtures.npz from the reference's own Python chain.

Run in a container that has the reference tree.  The reference's two pure-torch files
(k2/python/k2/rnnt_loss.py and k2/python/k2/mutual_information.py) are loaded by path under a
private package name, so the package's ``__init__`` (which needs the full compiled ``_k2``) is
never executed; the one native module they import, ``_k2``, is a stand-in defined below whose two
functions forward to oracle/_ref/libk2ref.so, i.e. to the reference's own
mutual_information_cpu.cu compiled in place (oracle/Makefile).  Everything recorded is therefore
what k2 itself computes on the CPU with the torch of this container.

The fixture holds data only (inputs, outputs, case descriptors); nothing of the reference's text.

    python tests/golden/make_rnnt_fixtures.py
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import mi as omi  # noqa: E402

REFERENCE = os.environ.get("K2_REFERENCE", "/root/reference")
PKG = "k2_reference_files"


def _load_reference():
    """(rnnt_loss module, mutual_information module) of the reference, loaded by path."""
    shim = types.ModuleType("_k2")

    def mutual_information_forward(px, py, boundary, p):
        bd = None if boundary is None else boundary.numpy()
        ans, p_np = omi.mi_forward(px.detach().numpy(), py.detach().numpy(), bd, backend="ref")
        p.copy_(torch.from_numpy(p_np))
        return torch.from_numpy(ans)

    def mutual_information_backward(px, py, boundary, p, ans_grad):
        bd = None if boundary is None else boundary.numpy()
        gx, gy = omi.mi_backward(px.detach().numpy(), py.detach().numpy(), bd, p.numpy(),
                                 ans_grad.numpy(), backend="ref")
        return [torch.from_numpy(gx), torch.from_numpy(gy)]

    shim.mutual_information_forward = mutual_information_forward
    shim.mutual_information_backward = mutual_information_backward
    sys.modules["_k2"] = shim

    pkg = types.ModuleType(PKG)
    pkg.__path__ = [os.path.join(REFERENCE, "k2", "python", "k2")]
    sys.modules[PKG] = pkg
    mods = []
    for name in ("mutual_information", "rnnt_loss"):
        spec = importlib.util.spec_from_file_location(
            f"{PKG}.{name}", os.path.join(pkg.__path__[0], name + ".py"))
        mod = importlib.util.module_from_spec(spec)
        sys.modules[spec.name] = mod
        spec.loader.exec_module(mod)
        mods.append(mod)
    return mods[1], mods[0]


def _inputs(rng, B, T, S, C, dtype, with_boundary, modified, t_lo, s_lo, scale=1.0):
    am = torch.from_numpy((rng.standard_normal((B, T, C)) * scale).astype(dtype))
    lm = torch.from_numpy((rng.standard_normal((B, S + 1, C)) * scale).astype(dtype))
    symbols = torch.from_numpy(rng.integers(1, C, size=(B, S)).astype(np.int64))
    boundary = None
    if with_boundary:
        Tb = rng.integers(t_lo, T + 1, size=B)
        Sb = rng.integers(s_lo, S + 1, size=B)
        if modified:
            Sb = np.minimum(Sb, Tb)
        boundary = torch.from_numpy(np.stack(
            [np.zeros(B, np.int64), np.zeros(B, np.int64), Sb, Tb], axis=1).astype(np.int64))
    return am, lm, symbols, boundary


class Recorder:
    def __init__(self):
        self.out = {}
        self.names = []

    def add(self, name, **arrays):
        assert name not in self.names
        self.names.append(name)
        for k, v in arrays.items():
            if v is None:
                continue
            if isinstance(v, torch.Tensor):
                v = v.detach().numpy()
            self.out[f"{name}/{k}"] = np.asarray(v)


def main():
    omi.build_ref()
    rl, mi = _load_reference()
    rec = Recorder()
    torch.manual_seed(0)
    torch.set_num_threads(1)

    # ---- the whole chain: simple loss with occupation gradients -> ranges -> pruned loss -------
    chain = [
        # name,      B, T,  S,  C, rnnt_type,    boundary, t_lo, s_lo, R, delay
        ("chain0", 2, 24, 7, 9, "regular", True, 15, 4, 3, 0.0),
        ("chain1", 3, 40, 12, 11, "regular", True, 25, 5, 5, 0.1),
        ("chain2", 2, 33, 9, 8, "modified", True, 20, 5, 4, 0.05),
        ("chain3", 2, 21, 6, 7, "constrained", True, 14, 3, 3, 0.2),
        ("chain4", 2, 18, 5, 6, "regular", False, 18, 5, 2, 0.3),
        ("chain5", 2, 70, 20, 10, "regular", True, 50, 12, 9, 0.0),
        ("chain6", 2, 19, 5, 6, "modified", False, 19, 5, 6, 0.15),   # R = S + 1: no pruning
        ("chain7", 1, 6, 14, 5, "regular", True, 5, 13, 2, 0.0),      # R bumped: S_b > T_b
    ]
    for seed, (name, B, T, S, C, rt, wb, t_lo, s_lo, R, delay) in enumerate(chain):
        rng = np.random.default_rng(100 + seed)
        am, lm, symbols, boundary = _inputs(rng, B, T, S, C, np.float32, wb, rt != "regular",
                                            t_lo, s_lo)
        am_g = am.clone().requires_grad_(True)
        lm_g = lm.clone().requires_grad_(True)
        loss_vec, (gx, gy) = rl.rnnt_loss_simple(
            lm=lm_g, am=am_g, symbols=symbols, termination_symbol=0, boundary=boundary,
            rnnt_type=rt, delay_penalty=delay, reduction="none", return_grad=True)
        w = torch.from_numpy(rng.uniform(0.5, 1.5, B).astype(np.float32))
        (loss_vec * w).sum().backward()
        bd_for_ranges = boundary
        if bd_for_ranges is None:
            bd_for_ranges = torch.tensor([[0, 0, S, T]] * B, dtype=torch.int64)
        ranges = rl.get_rnnt_prune_ranges(px_grad=gx, py_grad=gy, boundary=bd_for_ranges, s_range=R)
        ranges_old = rl.get_rnnt_prune_ranges_deprecated(px_grad=gx, py_grad=gy,
                                                         boundary=bd_for_ranges, s_range=R)
        Reff = ranges.shape[2]
        am_p, lm_p = rl.do_rnnt_pruning(am=am, lm=lm, ranges=ranges)
        logits = (am_p + lm_p).clone().requires_grad_(True)
        pruned = rl.rnnt_loss_pruned(logits=logits, symbols=symbols, ranges=ranges,
                                     termination_symbol=0, boundary=boundary, rnnt_type=rt,
                                     delay_penalty=delay, reduction="none")
        (pruned * w).sum().backward()
        hat = rl.rnnt_loss_pruned(logits=logits.detach(), symbols=symbols, ranges=ranges,
                                  termination_symbol=0, boundary=boundary, rnnt_type=rt,
                                  delay_penalty=delay, reduction="none", use_hat_loss=True)
        full_logits = (am.unsqueeze(2) + lm.unsqueeze(1)).clone().requires_grad_(True)
        full = rl.rnnt_loss(logits=full_logits, symbols=symbols, termination_symbol=0,
                            boundary=boundary, rnnt_type=rt, delay_penalty=delay, reduction="none")
        (full * w).sum().backward()
        smoothed = rl.rnnt_loss_smoothed(lm=lm, am=am, symbols=symbols, termination_symbol=0,
                                         lm_only_scale=0.2, am_only_scale=0.1, boundary=boundary,
                                         rnnt_type=rt, delay_penalty=delay, reduction="none")
        rec.add(name, am=am, lm=lm, symbols=symbols, boundary=boundary,
                rnnt_type=np.array(rt), delay_penalty=np.array(delay, np.float64),
                s_range=np.array(R), weights=w,
                simple_loss=loss_vec, px_grad=gx, py_grad=gy, am_grad=am_g.grad, lm_grad=lm_g.grad,
                ranges=ranges, ranges_deprecated=ranges_old, s_range_effective=np.array(Reff),
                pruned_loss=pruned, pruned_logits_grad=logits.grad, hat_loss=hat,
                full_loss=full, full_logits_grad=full_logits.grad, smoothed_loss=smoothed)

    # ---- get_rnnt_prune_ranges on gradients with exact ties and with near ties ------------------
    ties = [
        # name,     B, S,  T, modified, R
        ("ties0", 2, 8, 13, False, 2),
        ("ties1", 2, 9, 17, False, 3),
        ("ties2", 2, 10, 40, True, 4),
        ("ties3", 3, 12, 37, False, 5),
        ("ties4", 2, 12, 33, True, 6),
        ("ties5", 2, 14, 64, False, 7),
        ("ties6", 2, 14, 45, True, 8),
        ("ties7", 2, 15, 70, False, 9),
        ("ties8", 2, 6, 20, False, 7),    # R = S + 1
        ("ties9", 2, 11, 96, False, 5),
    ]
    for seed, (name, B, S, T, modified, R) in enumerate(ties):
        rng = np.random.default_rng(200 + seed)
        T1 = T if modified else T + 1
        if seed % 2 == 0:
            # multiples of 1/8: window sums are exact, so equal sums are true ties and the first
            # maximum must win
            gx = rng.integers(0, 5, (B, S, T1)).astype(np.float32) / 8
            gy = rng.integers(0, 5, (B, S + 1, T)).astype(np.float32) / 8
        else:
            # one value repeated with last-bit noise: sums that differ by an ulp or two, where the
            # order of the additions decides the arg-max
            base = np.float32(1.0) / np.float32(3.0)
            gx = (base * (1 + rng.integers(-2, 3, (B, S, T1)) * np.float32(2.0 ** -23))).astype(np.float32)
            gy = (base * (1 + rng.integers(-2, 3, (B, S + 1, T)) * np.float32(2.0 ** -23))).astype(np.float32)
        Tb = rng.integers(max(T // 2, S if modified else 1), T + 1, size=B)
        Sb = rng.integers(S // 2, S + 1, size=B)
        if modified:
            Sb = np.minimum(Sb, Tb)
        bd = np.stack([np.zeros(B, np.int64), np.zeros(B, np.int64), Sb, Tb], axis=1).astype(np.int64)
        ranges = rl.get_rnnt_prune_ranges(px_grad=torch.from_numpy(gx), py_grad=torch.from_numpy(gy),
                                          boundary=torch.from_numpy(bd), s_range=R)
        ranges_old = rl.get_rnnt_prune_ranges_deprecated(
            px_grad=torch.from_numpy(gx), py_grad=torch.from_numpy(gy),
            boundary=torch.from_numpy(bd), s_range=R)
        rec.add(name, px_grad=gx, py_grad=gy, boundary=bd, s_range=np.array(R), ranges=ranges,
                ranges_deprecated=ranges_old)

    # ---- get_rnnt_logprobs where the max-shifted exponentials underflow (the `+ tiny` floor) ----
    for seed, (name, rt, scale) in enumerate([("floor0", "regular", 40.0), ("floor1", "modified", 60.0),
                                              ("floor2", "constrained", 25.0)]):
        rng = np.random.default_rng(300 + seed)
        B, T, S, C = 2, 11, 4, 6
        am, lm, symbols, boundary = _inputs(rng, B, T, S, C, np.float32, True, rt != "regular",
                                            8, 3, scale=scale)
        px, py = rl.get_rnnt_logprobs(lm=lm, am=am, symbols=symbols, termination_symbol=0,
                                      rnnt_type=rt, boundary=boundary)
        rec.add(name, am=am, lm=lm, symbols=symbols, boundary=boundary, rnnt_type=np.array(rt),
                px=px, py=py)

    # ---- joint_mutual_information_recursion: the split over the inputs and its gradients --------
    joint = [
        # name,     N, B, S,  T, modified, boundary
        ("joint0", 1, 2, 5, 9, False, False),
        ("joint1", 2, 3, 7, 12, False, True),
        ("joint2", 3, 2, 6, 15, True, True),
        ("joint3", 2, 2, 70, 90, True, True),     # two chunks of rows
        ("joint4", 3, 2, 9, 40, False, False),
        ("joint5", 2, 3, 4, 4, True, False),
    ]
    for seed, (name, N, B, S, T, modified, wb) in enumerate(joint):
        rng = np.random.default_rng(400 + seed)
        T1 = T if modified else T + 1
        pxs = [torch.from_numpy(rng.normal(-1.0, 1.0, (B, S, T1)).astype(np.float32)).requires_grad_(True)
               for _ in range(N)]
        pys = [torch.from_numpy(rng.normal(-1.0, 1.0, (B, S + 1, T)).astype(np.float32)).requires_grad_(True)
               for _ in range(N)]
        if not modified and not wb:
            with torch.no_grad():
                pxs[0][:, :, -1] = -np.inf   # the reference's convention for the last column
        boundary = None
        if wb:
            rows = []
            for _ in range(B):
                s_len = int(rng.integers(S // 2, S + 1))
                t_len = int(rng.integers(max(T // 2, s_len), T + 1))
                s0 = int(rng.integers(0, S - s_len + 1))
                t0 = int(rng.integers(0, T - t_len + 1))
                rows.append([s0, t0, s0 + s_len, t0 + t_len])
            boundary = torch.tensor(rows, dtype=torch.int64)
        prods = mi.joint_mutual_information_recursion(px=pxs, py=pys, boundary=boundary)
        w = torch.from_numpy(rng.uniform(0.5, 1.5, (N, B)).astype(np.float32))
        (prods * w).sum().backward()
        arrays = dict(boundary=boundary, modified=np.array(modified), weights=w, prods=prods,
                      n=np.array(N))
        for i in range(N):
            arrays[f"px{i}"] = pxs[i]
            arrays[f"py{i}"] = pys[i]
            arrays[f"px{i}_grad"] = pxs[i].grad
            arrays[f"py{i}_grad"] = pys[i].grad
        rec.add(name, **arrays)

    # ---- gradients of the smoothed and of the HAT pruned loss to the network outputs -------------
    variants = [
        # name,    B, T,  S, C, rnnt_type,     R, lm_only, am_only
        ("grad0", 2, 17, 5, 7, "regular", 3, 0.25, 0.0),
        ("grad1", 2, 23, 6, 9, "modified", 4, 0.0, 0.3),
        ("grad2", 3, 30, 8, 8, "regular", 5, 0.2, 0.1),
        ("grad3", 2, 20, 6, 6, "constrained", 3, 0.15, 0.25),
    ]
    for seed, (name, B, T, S, C, rt, R, lm_only, am_only) in enumerate(variants):
        rng = np.random.default_rng(500 + seed)
        am, lm, symbols, boundary = _inputs(rng, B, T, S, C, np.float32, True, rt != "regular",
                                            max(T // 2, S), S // 2)
        w = torch.from_numpy(rng.uniform(0.5, 1.5, B).astype(np.float32))
        am_g = am.clone().requires_grad_(True)
        lm_g = lm.clone().requires_grad_(True)
        smoothed = rl.rnnt_loss_smoothed(lm=lm_g, am=am_g, symbols=symbols, termination_symbol=0,
                                         lm_only_scale=lm_only, am_only_scale=am_only,
                                         boundary=boundary, rnnt_type=rt, reduction="none")
        (smoothed * w).sum().backward()
        _, (gx, gy) = rl.rnnt_loss_simple(lm=lm, am=am, symbols=symbols, termination_symbol=0,
                                          boundary=boundary, rnnt_type=rt, reduction="none",
                                          return_grad=True)
        ranges = rl.get_rnnt_prune_ranges(px_grad=gx, py_grad=gy, boundary=boundary, s_range=R)
        am_p, lm_p = rl.do_rnnt_pruning(am=am, lm=lm, ranges=ranges)
        logits = (am_p + lm_p).clone().requires_grad_(True)
        hat = rl.rnnt_loss_pruned(logits=logits, symbols=symbols, ranges=ranges, termination_symbol=0,
                                  boundary=boundary, rnnt_type=rt, reduction="none", use_hat_loss=True)
        (hat * w).sum().backward()
        rec.add(name, am=am, lm=lm, symbols=symbols, boundary=boundary, rnnt_type=np.array(rt),
                weights=w, lm_only_scale=np.array(lm_only), am_only_scale=np.array(am_only),
                smoothed_loss=smoothed, smoothed_am_grad=am_g.grad, smoothed_lm_grad=lm_g.grad,
                ranges=ranges, hat_logits=logits.detach(), hat_loss=hat, hat_logits_grad=logits.grad)

    rec.out["names"] = np.array(rec.names)
    rec.out["torch_version"] = np.array(torch.__version__)
    path = os.path.join(HERE, "rnnt_ref_fixtures.npz")
    np.savez_compressed(path, **rec.out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(rec.names), "cases")


if __name__ == "__main__":
    main()
