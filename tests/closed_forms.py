"""Closed-form gradients of the RNN-T losses with respect to the network outputs, in numpy fp64.

With the occupation probabilities gx = d score / d px [B][S][T1] and gy = d score / d py
[B][S+1][T] of the lattice recursion, the gradient of  sum_b scale[b] * loss[b]  (loss = -score)
with respect to a row of logits that feeds one px entry (with weight GX) and one py entry (with
weight GY) through a log-softmax over the vocabulary is

    scale * ( softmax(row) * (GX + GY)  -  GX * onehot(symbol)  -  GY * onehot(blank) ).

These forms are independent of the kernels and of autograd; tests/test_closed_forms.py pins them
against torch autograd over the plain-torch definitions at small sizes, and the GPU tests use them
at the full BASELINE sizes, where materialising an autograd graph is not practical.
"""
import numpy as np


def _softmax(x):
    x = x.astype(np.float64)
    m = x.max(axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(x - m)
    return e / e.sum(axis=-1, keepdims=True)


def _edge_weights(gx, gy, rnnt_type):
    """(GX [B][S+1][T], GY [B][S+1][T]): weight of the symbol term and of the blank term of the
    log-softmax row at lattice position (s, t); row S has no symbol.  "constrained" adds
    py[s+1][t] to px[s][t] (k2/python/k2/rnnt_loss.py:220-223), so the blank term of row s+1 also
    collects gx[s][t]."""
    B, S, T1 = gx.shape
    T = gy.shape[2]
    GX = np.zeros((B, S + 1, T), np.float64)
    GX[:, :S, :] = gx[:, :, :T]
    GY = gy.astype(np.float64).copy()
    if rnnt_type == "constrained":
        GY[:, 1:, :] += gx[:, :, :T]
    return GX, GY


def _alternatives(fn, gx, gy):
    """gx, gy may be tuples of alternative occupation gradients (say the fp32 and the fp64
    oracle's): the softmax of each row is then formed once for all of them."""
    if isinstance(gx, (tuple, list)):
        return fn(list(gx), list(gy))
    return fn([gx], [gy])[0]


def simple_grads(lm, am, symbols, blank, gx, gy, scale, rnnt_type="regular"):
    """(lm_grad, am_grad) of sum_b scale[b] * rnnt_loss_simple(...)[b]."""
    return _alternatives(lambda a, b: [_simple_grads(lm, am, symbols, blank, x, y, scale, rnnt_type, None)
                                       for x, y in zip(a, b)], gx, gy)


def _simple_grads(lm, am, symbols, blank, gx, gy, scale, rnnt_type, _unused):
    B, T, C = am.shape
    S = lm.shape[1] - 1
    GX, GY = _edge_weights(gx, gy, rnnt_type)
    lm_grad = np.zeros(lm.shape, np.float64)
    am_grad = np.zeros(am.shape, np.float64)
    for b in range(B):
        P = _softmax(lm[b][:, None, :].astype(np.float64) + am[b][None, :, :])  # [S+1][T][C]
        W = GX[b] + GY[b]
        lg = np.einsum("st,stc->sc", W, P)
        ag = np.einsum("st,stc->tc", W, P)
        lg[:, blank] -= GY[b].sum(axis=1)
        ag[:, blank] -= GY[b].sum(axis=0)
        if S > 0:
            np.subtract.at(lg, (np.arange(S), symbols[b]), GX[b, :S].sum(axis=1))
            np.subtract.at(ag, (np.arange(T)[None, :].repeat(S, 0), symbols[b][:, None].repeat(T, 1)),
                           GX[b, :S])
        lm_grad[b] = scale[b] * lg
        am_grad[b] = scale[b] * ag
    return lm_grad, am_grad


def joint_logits_grad(logits, symbols, blank, gx, gy, scale, rnnt_type="regular"):
    """Gradient of sum_b scale[b] * rnnt_loss(...)[b] w.r.t. logits [B][T][S+1][C]."""
    return _alternatives(lambda a, b: _joint_logits_grad(logits, symbols, blank, a, b, scale, rnnt_type),
                         gx, gy)


def _joint_logits_grad(logits, symbols, blank, gxs, gys, scale, rnnt_type):
    B, T, S1, C = logits.shape
    S = S1 - 1
    W = [_edge_weights(gx, gy, rnnt_type) for gx, gy in zip(gxs, gys)]
    outs = [np.empty(logits.shape, np.float64) for _ in W]
    for b in range(B):
        P = _softmax(logits[b])
        for (GX, GY), out in zip(W, outs):
            gxb, gyb = GX[b].T, GY[b].T                  # [T][S+1]
            g = P * (gxb + gyb)[..., None]
            g[..., blank] -= gyb
            if S > 0:
                idx = np.broadcast_to(symbols[b][None, :, None], (T, S, 1))
                np.put_along_axis(g[:, :S, :], idx,
                                  np.take_along_axis(g[:, :S, :], idx, axis=2) - gxb[:, :S, None], axis=2)
            out[b] = scale[b] * g
    return outs


def pruned_logits_grad(logits, symbols, ranges, blank, gx, gy, scale, rnnt_type="regular", hat=False):
    """Gradient of sum_b scale[b] * rnnt_loss_pruned(...)[b] w.r.t. logits [B][T][R][C]; row k of
    frame t is lattice position s = ranges[b][t][k] (k2/python/k2/rnnt_loss.py:1180-1348).
    hat: blank probability sigmoid(l0), the others (1 - sigmoid(l0)) softmax(l[1:])
    (k2/python/k2/rnnt_loss.py:992-1177)."""
    return _alternatives(lambda a, b: _pruned_logits_grad(logits, symbols, ranges, blank, a, b, scale,
                                                          rnnt_type, hat), gx, gy)


def _pruned_logits_grad(logits, symbols, ranges, blank, gxs, gys, scale, rnnt_type, hat):
    B, T, R, C = logits.shape
    S = symbols.shape[1]
    W = [_edge_weights(gx, gy, rnnt_type) for gx, gy in zip(gxs, gys)]
    outs = [np.empty(logits.shape, np.float64) for _ in W]
    sym_ext = np.concatenate([symbols, np.full((B, 1), blank, np.int64)], axis=1)
    for b in range(B):
        s = ranges[b]                                     # [T][R]
        t = np.arange(T)[:, None]
        sym = sym_ext[b][s]
        if not hat:
            P = _softmax(logits[b])
        else:
            assert blank == 0
            P = _softmax(logits[b][..., 1:])
            sig = 1.0 / (1.0 + np.exp(-logits[b][..., 0].astype(np.float64)))
        for (GX, GY), out in zip(W, outs):
            gxb = np.where(s < S, GX[b][np.minimum(s, S), t], 0.0)
            gyb = GY[b][s, t]
            if not hat:
                g = P * (gxb + gyb)[..., None]
                g[..., blank] -= gyb
            else:
                # log px = l[sym] - logsumexp(l[1:]) + log(1 - sig);  log py = log sig
                g = np.zeros(logits[b].shape, np.float64)
                g[..., 1:] = P * gxb[..., None]
                g[..., 0] = gxb * sig - gyb * (1.0 - sig)
            # (after column 0 is in place: a label equal to 0 takes its -gx there as anywhere else)
            np.put_along_axis(g, sym[..., None],
                              np.take_along_axis(g, sym[..., None], axis=2) - gxb[..., None], axis=2)
            out[b] = scale[b] * g
    return outs


def smoothed_grads(lm, am, symbols, blank, lm_only_scale, am_only_scale, gx, gy, scale, rnnt_type="regular"):
    """(lm_grad, am_grad) of sum_b scale[b] * rnnt_loss_smoothed(...)[b]
    (k2/python/k2/rnnt_loss.py:1471-1704).  Every lattice edge carries
        joint_scale * log softmax(lm_s + am_t) + lm_only_scale * log softmax(lm_s)
                                               + am_only_scale * log softmax(am_t + log unigram),
    unigram = mean over all B (S+1) rows of softmax(lm) + tiny.  The joint term is the simple
    loss's gradient times joint_scale.  With Wx, Wy the symbol / blank weights of a row summed over
    its frames, the lm-only term gives row (b, s) of lm
        lm_only_scale * (softmax(lm_s) (Wx + Wy) - Wx onehot(symbol_s) - Wy onehot(blank));
    the am-only term gives row (b, t) of am the same shape of expression, dz, with the weights summed
    over s and the symbol one-hots weighted one by one, and through the unigram it reaches every
    row of lm:  softmax(lm_s) (dU - <softmax(lm_s), dU>) / (B (S+1)),  dU = sum_{b,t} dz / unigram."""
    def one(gx, gy):
        B, T, C = am.shape
        S = lm.shape[1] - 1
        joint_scale = 1.0 - lm_only_scale - am_only_scale
        ls = lm_only_scale or 1.0e-20
        as_ = am_only_scale or 1.0e-20
        lm_g, am_g = _simple_grads(lm, am, symbols, blank, gx, gy, scale, rnnt_type, None)
        lm_g *= joint_scale
        am_g *= joint_scale
        GX, GY = _edge_weights(gx, gy, rnnt_type)
        w = np.asarray(scale, np.float64)
        pl = _softmax(lm)                                              # [B][S+1][C]
        unigram = pl.mean(axis=(0, 1)) + np.finfo(lm.dtype).tiny
        pa = _softmax(am.astype(np.float64) + np.log(unigram))         # [B][T][C]
        # lm only
        wx, wy = GX.sum(axis=2), GY.sum(axis=2)                        # [B][S+1]
        g = pl * (wx + wy)[..., None]
        g[..., blank] -= wy
        for b in range(B):
            if S > 0:
                np.subtract.at(g[b], (np.arange(S), symbols[b]), wx[b, :S])
        lm_g += ls * w[:, None, None] * g
        # am only
        vx, vy = GX.sum(axis=1), GY.sum(axis=1)                        # [B][T]
        dz = pa * (vx + vy)[..., None]
        dz[..., blank] -= vy
        for b in range(B):
            if S > 0:
                np.subtract.at(dz[b], (np.arange(T)[None, :].repeat(S, 0), symbols[b][:, None].repeat(T, 1)),
                               GX[b, :S])
        dz *= as_ * w[:, None, None]
        am_g += dz
        du = dz.sum(axis=(0, 1)) / unigram / (B * (S + 1))             # d loss / d softmax(lm)[b][s][c], any b, s
        lm_g += pl * (du - (pl * du).sum(axis=-1, keepdims=True))
        return lm_g, am_g
    return _alternatives(lambda a, b: [one(x, y) for x, y in zip(a, b)], gx, gy)
