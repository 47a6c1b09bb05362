"""Plain-PyTorch (CPU) definitions of the RNN-T quantities, written from the textbook formulas
(log-softmax over the vocabulary, log-add-exp lattice recursion), differentiable by autograd.
They are the float reference for the gradients of the fused HIP kernels; sizes must stay small
(the simple-joiner version materialises the full [B,T,S+1,C] lattice)."""
import torch


def logprobs_from_logits(logits, symbols, blank, rnnt_type="regular", boundary=None):
    """logits [B,T,S+1,C] -> (px [B,S,T1], py [B,S+1,T])."""
    return _from_logprobs(torch.log_softmax(logits, dim=-1), symbols, blank, rnnt_type, boundary)


def logprobs_smoothed(lm, am, symbols, blank, lm_only_scale, am_only_scale, rnnt_type="regular",
                      boundary=None):
    """Log-linear mix of three normalised distributions over the vocabulary: softmax(am + lm),
    softmax(lm), and softmax(am + log unigram) with the unigram the batch mean of softmax(lm)."""
    joint = torch.log_softmax(am.unsqueeze(2) + lm.unsqueeze(1), dim=-1)       # [B,T,S+1,C]
    lm_only = torch.log_softmax(lm, dim=-1).unsqueeze(1)                        # [B,1,S+1,C]
    unigram = torch.softmax(lm, dim=-1).mean(dim=(0, 1)) + torch.finfo(lm.dtype).tiny
    am_only = torch.log_softmax(am + unigram.log(), dim=-1).unsqueeze(2)        # [B,T,1,C]
    joint_scale = 1.0 - lm_only_scale - am_only_scale
    lm_only_scale = lm_only_scale or 1.0e-20
    am_only_scale = am_only_scale or 1.0e-20
    mix = joint * joint_scale + lm_only * lm_only_scale + am_only * am_only_scale
    return _from_logprobs(mix, symbols, blank, rnnt_type, boundary)


def _from_logprobs(lp, symbols, blank, rnnt_type, boundary):
    B, T, S1, C = lp.shape
    S = S1 - 1
    idx = symbols.reshape(B, 1, S, 1).expand(B, T, S, 1)
    px = lp[:, :, :S, :].gather(3, idx).squeeze(-1).permute(0, 2, 1)  # [B,S,T]
    py = lp[..., blank].permute(0, 2, 1)  # [B,S+1,T]
    if rnnt_type == "regular":
        px = torch.cat([px, torch.full((B, S, 1), float("-inf"), dtype=px.dtype)], dim=2)
        if boundary is not None:
            mask = torch.zeros(B, 1, T + 1, dtype=torch.bool)
            mask[torch.arange(B), 0, boundary[:, 3]] = True
            px = px.masked_fill(mask, float("-inf"))
    elif rnnt_type == "constrained":
        px = px + py[:, 1:, :]
    return px, py


def logprobs_simple(lm, am, symbols, blank, rnnt_type="regular", boundary=None):
    return logprobs_from_logits(am.unsqueeze(2) + lm.unsqueeze(1), symbols, blank, rnnt_type, boundary)


def logprobs_pruned(logits, symbols, ranges, blank, boundary, rnnt_type="regular", hat=False):
    """logits [B,T,R,C]; dense px/py with -inf outside the band.  ``hat``: the blank (column 0)
    has probability sigmoid(l0) and the others (1 - sigmoid(l0)) softmax(l[1:])."""
    B, T, R, C = logits.shape
    S = symbols.shape[1]
    if hat:
        assert blank == 0
        p_blank = torch.sigmoid(logits[..., :1])
        lp = torch.cat([p_blank.log(),
                        (1 - p_blank).log() + torch.log_softmax(logits[..., 1:], dim=-1)], dim=-1)
    else:
        lp = torch.log_softmax(logits, dim=-1)
    T1 = T + 1 if rnnt_type == "regular" else T
    px = torch.full((B, S, T1), float("-inf"), dtype=logits.dtype)
    py = torch.full((B, S + 1, T), float("-inf"), dtype=logits.dtype)
    pxs, pys = [], []
    px_rows = {}
    # assemble with index_put on a flat view so autograd flows
    bi, si, ti, vals = [], [], [], []
    bj, sj, tj, valy = [], [], [], []
    for b in range(B):
        for t in range(T):
            s0 = int(ranges[b, t, 0])
            for k in range(R):
                s = s0 + k
                if s < S and not (rnnt_type == "regular" and boundary is not None and int(boundary[b, 3]) == t):
                    bi.append(b); si.append(s); ti.append(t); vals.append(lp[b, t, k, int(symbols[b, s])])
                if s <= S:
                    bj.append(b); sj.append(s); tj.append(t); valy.append(lp[b, t, k, blank])
    if vals:
        px = px.index_put((torch.tensor(bi), torch.tensor(si), torch.tensor(ti)), torch.stack(vals))
    if valy:
        py = py.index_put((torch.tensor(bj), torch.tensor(sj), torch.tensor(tj)), torch.stack(valy))
    if rnnt_type == "constrained":
        px = px + py[:, 1:, :]
    return px, py


def mi_scores(px, py, boundary=None):
    """The lattice recursion with torch.logaddexp, differentiable; small sizes only."""
    B, S, T1 = px.shape
    T = py.shape[2]
    modified = T1 == T
    off = -1 if modified else 0
    out = []
    ninf = torch.tensor(float("-inf"), dtype=px.dtype)
    for b in range(B):
        s0, t0, s1, t1 = (0, 0, S, T) if boundary is None else [int(v) for v in boundary[b]]
        p = {}
        for s in range(s0, s1 + 1):
            for t in range(t0, t1 + 1):
                if s == s0 and t == t0:
                    p[(s, t)] = torch.zeros((), dtype=px.dtype)
                    continue
                terms = []
                if s > s0 and t + off >= t0:
                    terms.append(p[(s - 1, t + off)] + px[b, s - 1, t + off])
                if t > t0:
                    terms.append(p[(s, t - 1)] + py[b, s, t - 1])
                # drop -inf terms so autograd never differentiates logaddexp(-inf, -inf)
                terms = [x for x in terms if torch.isfinite(x)]
                if not terms:
                    p[(s, t)] = ninf
                elif len(terms) == 1:
                    p[(s, t)] = terms[0]
                else:
                    p[(s, t)] = torch.logaddexp(terms[0], terms[1])
        out.append(p[(s1, t1)])
    return torch.stack(out)
