"""TEST INFRASTRUCTURE: element-wise comparison of a gradient with the float64 oracle's.

The normwise bound (largest error against the largest entry of the sentence) says nothing about posteriors a few decades
below that maximum; this check holds every entry to a relative bound that depends on how large it is against its
sentence's maximum:  1e-4 relative for every entry of at least 1e-6 of it (reported in two bands, from 1e-3 and from 1e-6
of the maximum up; measured worst cases: 4e-5 in either band);  below: 1e-9 of the maximum, absolute (such entries do not
move a parameter update).  Returns the worst relative error of each band for the tests' printouts."""
import numpy as np

BANDS = ((1e-3, 1e-4), (1e-6, 1e-4))  # (share of the sentence maximum, relative bound)
FLOOR_ABS = 1e-9                     # absolute bound, as a share of the maximum, below the last band


def elementwise_errors(got, want):
    """got, want: arrays of one sentence.  Returns [(band floor, worst relative error, index of it)] and the worst
    absolute error below the bands as a share of the maximum."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    mx = np.abs(want).max()
    out = []
    if mx == 0:
        return [(f, 0.0, None) for f, _ in BANDS], float(np.abs(got).max())
    mag = np.abs(want)
    upper = np.inf
    for floor, _ in BANDS:
        sel = (mag >= floor * mx) & (mag < upper * mx if np.isfinite(upper) else True)
        if sel.any():
            rel = np.abs(got - want)[sel] / mag[sel]
            k = int(rel.argmax())
            out.append((floor, float(rel[k]), tuple(int(i) for i in np.argwhere(sel)[k])))
        else:
            out.append((floor, 0.0, None))
        upper = floor
    rest = mag < BANDS[-1][0] * mx
    below = float((np.abs(got - want)[rest]).max() / mx) if rest.any() else 0.0
    return out, below


def assert_elementwise(got, want, what):
    """Asserts the bounds of the module docstring for one sentence; returns the per-band worst relative errors."""
    bands, below = elementwise_errors(got, want)
    for (floor, bound), (_, err, where) in zip(BANDS, bands):
        assert err <= bound, "%s: entry %s (>= %.0e of the sentence maximum) is off by %.2e relative (bound %.0e)" % (
            what, where, floor, err, bound)
    assert below <= FLOOR_ABS, "%s: an entry below %.0e of the sentence maximum is off by %.2e of the maximum" % (
        what, BANDS[-1][0], below)
    return [e for _, e, _ in bands]
