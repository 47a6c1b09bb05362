"""How the fp32 results of the GPU path are compared with the CPU oracle.

The stated bar is |got - want| <= 1e-5 + 1e-4 |want| against the reference's fp32 result.  Where
|p| reaches the thousands, one fp32 ulp of p is 1.2e-4 .. 2.4e-4, every gradient is exp() of a
difference of such values, and the reference's OWN fp32 gradients then differ from an fp64 run by
several 1e-4 relative: two correct fp32 implementations cannot agree to 1e-4 there.  For the
elements that miss the plain bar the fp64 oracle arbitrates, element by element:

    |got - f64| <= 1e-5 + 1e-4 |f64| + max(2 |cpu32 - f64|, 4 ulp(p_scale) |f64|)

i.e. the GPU may be as far from the truth as twice what the reference's fp32 code is AT THAT
ELEMENT, with a floor of four ulps of the largest |p| of the element's sequence (an element where
the reference's rounding errors happen to cancel does not set the bar for everybody else's).
The share of elements that needed the arbitration is returned and bounded by the caller.
"""
import numpy as np

RTOL, ATOL = 1e-4, 1e-5
FLOOR_ULPS = 4.0

# name -> dict of the figures of the last comparison under that name (read by tests that report)
last_stats = {}


def p_scale_of(p64):
    """Largest finite |p| of each sequence of an fp64 p [B][S+1][T+1] (NaN / inf ignored), at least 1."""
    mag = np.where(np.isfinite(p64), np.abs(p64), 0.0)
    return np.maximum(mag.reshape(mag.shape[0], -1).max(axis=1), 1.0)


def close_f32(name, got, want32, want64, p_scale=None, max_arbitrated=1.0, relative_floor=True):
    """Asserts the comparison described above.  p_scale: [B] (broadcast over the trailing axes of
    got) or None for no floor.  relative_floor=False makes the floor absolute (4 ulps of p_scale:
    for p itself rather than for a gradient).  Returns the statistics dict."""
    got = np.asarray(got, dtype=np.float64)
    w32 = np.asarray(want32, dtype=np.float64)
    with np.errstate(invalid="ignore"):
        same = (got == w32) | (np.isnan(got) & np.isnan(w32))
        plain = same | (np.abs(got - w32) <= ATOL + RTOL * np.abs(w32))
    stats = dict(n=int(got.size), arbitrated=0, arbitrated_frac=0.0,
                 max_gpu_vs_cpu32=float(np.nanmax(np.where(same, 0.0, np.abs(got - w32)), initial=0.0)))
    if want64 is not None:
        w64 = np.asarray(want64, dtype=np.float64)
        with np.errstate(invalid="ignore"):
            fin = np.isfinite(w64) & np.isfinite(got) & np.isfinite(w32)
            stats["max_gpu_vs_fp64"] = float(np.max(np.abs(got - w64), where=fin, initial=0.0))
            stats["max_cpu32_vs_fp64"] = float(np.max(np.abs(w32 - w64), where=fin, initial=0.0))
    if not plain.all():
        assert want64 is not None, (name, int((~plain).sum()), got[~plain][:5], w32[~plain][:5])
        with np.errstate(invalid="ignore"):
            floor = 0.0
            if p_scale is not None:
                ps = np.asarray(p_scale, dtype=np.float32).reshape((-1,) + (1,) * (got.ndim - 1))
                floor = FLOOR_ULPS * np.spacing(ps).astype(np.float64)
                if relative_floor:
                    floor = floor * np.abs(w64)
            budget = ATOL + RTOL * np.abs(w64) + np.maximum(2.0 * np.abs(w32 - w64), floor)
            ok = plain | (got == w64) | (np.abs(got - w64) <= budget)
        assert ok.all(), (name, int((~ok).sum()), got[~ok][:5], w32[~ok][:5], w64[~ok][:5])
        stats["arbitrated"] = int((~plain).sum())
        stats["arbitrated_frac"] = stats["arbitrated"] / max(got.size, 1)
    assert stats["arbitrated_frac"] <= max_arbitrated, (name, stats)
    last_stats[name] = stats
    return stats
