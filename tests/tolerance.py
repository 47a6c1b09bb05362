"""How the fp32 results of the GPU path are compared with the CPU oracle.

The stated bar is |got - want| <= 1e-5 + 1e-4 |want| against the reference's CPU result.  The
reference's CPU path exists in fp32 and in fp64 (mutual_information_cpu.cu:81,168 dispatches on
the dtype), and an element meets the bar PLAINLY if it is that close to either of them: to the
fp32 result (the kernels that repeat the reference's additions land on its bits almost
everywhere), or to the fp64 result of the same inputs (the exact answer, which a kernel that
sums in another order is often closer to than the reference's own fp32 code is).

Where |p| reaches the hundreds or thousands, one fp32 ulp of p is 3e-5 .. 2.4e-4, every gradient
is a sum over paths of products of exp() of differences of such values, the rounding errors add
up along the S_b + T_b steps of a path like a random walk, and the reference's OWN fp32 gradients
then differ from an fp64 run by several 1e-4 relative: two correct fp32 implementations cannot
agree to 1e-4 there, nor can either agree with fp64.  The elements that meet the bar against
neither result are ARBITRATED by the fp64 oracle, element by element:

    |got - f64| <= 1e-5 + 1e-4 |f64| + 2 max(|cpu32 - f64|, Q_b |f64|)

where Q_b is the 99.9th percentile, over the elements of the same sequence b, of the relative
error |cpu32 - f64| / |f64| of the reference's fp32 code against fp64 (elements with |f64| >= 1e-4;
mode "absolute": the percentile of |cpu32 - f64| itself, for quantities that are signed sums).
So the GPU may be as far from the truth as twice what the reference's fp32 code is at that
element, or, relative to the element's own size, twice what the reference's fp32 code is at the
worst thousandth of the same sequence's elements; a tiny element is never granted a large
element's noise.  A percentile is not a maximum: of tens of millions of elements a few lie in
the far tail of either implementation's error, so up to TAIL_FRACTION of the elements (one in a
hundred thousand) may exceed that budget, by no more than TAIL_FACTOR times.  The share of
elements that needed the arbitration is returned and bounded by the caller (max_arbitrated: the
rule is for a thin tail, not a second tolerance), and so is the share that missed the bar against
the fp32 result alone.
"""
import numpy as np

RTOL, ATOL = 1e-4, 1e-5
QUANTILE = 0.999
MIN_MAGNITUDE = 1e-4
TAIL_FRACTION = 1e-5
TAIL_FACTOR = 4.0

# name -> dict of the figures of the last comparison under that name (read by tests that report)
last_stats = {}


def _per_sequence_quantile(err, mag, mode):
    """[B] -> broadcastable [B,1,..]: the percentile of the reference's own error per sequence."""
    B = err.shape[0] if err.ndim > 0 else 1
    e = err.reshape(B, -1)
    m = mag.reshape(B, -1)
    q = np.zeros(B)
    for b in range(B):
        if mode == "relative":
            sel = np.isfinite(e[b]) & np.isfinite(m[b]) & (m[b] >= MIN_MAGNITUDE)
            vals = e[b][sel] / m[b][sel]
        else:
            sel = np.isfinite(e[b])
            vals = e[b][sel]
        if vals.size:
            q[b] = np.quantile(vals, QUANTILE)
    return q.reshape((B,) + (1,) * (err.ndim - 1)) if err.ndim > 0 else q[0]


def close_f32(name, got, want32, want64, max_arbitrated=1.0, mode="relative"):
    """Asserts the comparison described above; the leading axis of the arrays is the sequence.
    Returns the statistics dict."""
    got = np.asarray(got, dtype=np.float64)
    w32 = np.asarray(want32, dtype=np.float64)
    with np.errstate(invalid="ignore"):
        same = (got == w32) | (np.isnan(got) & np.isnan(w32))
        plain = same | (np.abs(got - w32) <= ATOL + RTOL * np.abs(w32))
        stats = dict(n=int(got.size), arbitrated=0, arbitrated_frac=0.0, beyond_fp32_bar=int((~plain).sum()),
                     max_gpu_vs_cpu32=float(np.max(np.abs(got - w32), where=~same & np.isfinite(got - w32),
                                                   initial=0.0)))
    if want64 is not None:
        w64 = np.asarray(want64, dtype=np.float64)
        with np.errstate(invalid="ignore"):
            fin = np.isfinite(w64) & np.isfinite(got) & np.isfinite(w32)
            stats["max_gpu_vs_fp64"] = float(np.max(np.abs(got - w64), where=fin, initial=0.0))
            stats["max_cpu32_vs_fp64"] = float(np.max(np.abs(w32 - w64), where=fin, initial=0.0))
    if not plain.all():
        assert want64 is not None, (name, int((~plain).sum()), got[~plain][:5], w32[~plain][:5])
        with np.errstate(invalid="ignore"):
            # the same bar against the reference's fp64 result
            plain = plain | (got == w64) | (np.abs(got - w64) <= ATOL + RTOL * np.abs(w64))
            ref_err = np.abs(w32 - w64)
            q = _per_sequence_quantile(ref_err, np.abs(w64), mode)
            floor = q * np.abs(w64) if mode == "relative" else q
            noise = 2.0 * np.maximum(ref_err, floor)
            err = np.abs(got - w64)
            ok = plain | (got == w64) | (err <= ATOL + RTOL * np.abs(w64) + noise)
            ok_tail = ok | (err <= ATOL + RTOL * np.abs(w64) + TAIL_FACTOR * noise)
        stats["reference_error_quantile_max"] = float(np.max(q))
        stats["tail"] = int((~ok).sum())
        assert ok_tail.all(), (name, int((~ok_tail).sum()), got[~ok_tail][:5], w32[~ok_tail][:5],
                               w64[~ok_tail][:5], stats)
        assert stats["tail"] <= TAIL_FRACTION * got.size, (name, stats["tail"], got[~ok][:5], w32[~ok][:5],
                                                            w64[~ok][:5], stats)
        stats["arbitrated"] = int((~plain).sum())
        stats["arbitrated_frac"] = stats["arbitrated"] / max(got.size, 1)
    assert stats["arbitrated_frac"] <= max_arbitrated, (name, stats)
    last_stats[name] = stats
    return stats
