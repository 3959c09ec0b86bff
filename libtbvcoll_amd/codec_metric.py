"""Accuracy figures of the int8 payload codec (TBV_CODEC=1): how far the coded all-reduce's result lies from
the exact sum of its two operands.

The reference asks for the codec to sit behind a threshold because it changes the numerics
(reports/12_references.md:140-142) and has no code or metric for it; the figures here are this build's.
The codec's step is (max - min) / 255 per group of 128 consecutive elements, so ONE large element stretches
the step of the whole group: the error is small against the tensor's norm (which the outliers dominate) and
large against the typical element.  Both views are reported.
"""
import numpy as np

GROUP = 128


def _rel_l2(err, ref):
    d = float(np.sqrt(np.sum(ref * ref)))
    return float(np.sqrt(np.sum(err * err))) / d if d > 0 else 0.0


def _snr_db(rel):
    return float("inf") if rel == 0 else float(-20.0 * np.log10(rel))


def accuracy(out, a, b, outlier_cut=None, exact_type_out=None):
    """`out`: the coded all-reduce's result; `a`, `b`: its operands (all as float arrays of the values as stored).
    The reference is the exact sum float64(a) + float64(b).

    rel_l2 / snr_db                 whole tensor: ||out - exact|| / ||exact||
    With `outlier_cut` (an element is an outlier when |x| >= cut in either operand):
    outlier_element_frac            fraction of elements that are outliers
    stretched_group_frac            fraction of groups of 128 (of either operand) that hold an outlier
    rel_l2_typical / snr_db_typical the same ratio over the non-outlier elements only
    rel_l2_typical_in_stretched / _in_clean   ... split by whether the element's group holds an outlier
    With `exact_type_out` (the uncoded all-reduce's result in the storage type): rel_l2_uncoded[_typical],
    what rounding the exact sum to the storage type costs, for scale."""
    a = np.asarray(a, dtype=np.float64).reshape(-1); b = np.asarray(b, dtype=np.float64).reshape(-1)
    out = np.asarray(out, dtype=np.float64).reshape(-1)
    exact = a + b
    err = out - exact
    r = {"elements": int(a.size), "rel_l2": _rel_l2(err, exact)}
    r["snr_db"] = _snr_db(r["rel_l2"])
    r["max_abs_err"] = float(np.max(np.abs(err))) if a.size else 0.0
    unc = None
    if exact_type_out is not None:
        unc = np.asarray(exact_type_out, dtype=np.float64).reshape(-1) - exact
        r["rel_l2_uncoded"] = _rel_l2(unc, exact)
    if outlier_cut is not None and a.size:
        is_out = (np.abs(a) >= outlier_cut) | (np.abs(b) >= outlier_cut)
        n = a.size
        pad = (-n) % GROUP
        grp = np.pad(is_out, (0, pad)).reshape(-1, GROUP).any(axis=1)          # a group of either operand is stretched
        in_stretched = np.repeat(grp, GROUP)[:n]
        typ = ~is_out
        r["outlier_element_frac"] = float(is_out.mean())
        r["stretched_group_frac"] = float(grp.mean())
        r["rel_l2_typical"] = _rel_l2(err[typ], exact[typ])
        r["snr_db_typical"] = _snr_db(r["rel_l2_typical"])
        ts, tc = typ & in_stretched, typ & ~in_stretched
        r["rel_l2_typical_in_stretched"] = _rel_l2(err[ts], exact[ts]) if ts.any() else 0.0
        r["rel_l2_typical_in_clean"] = _rel_l2(err[tc], exact[tc]) if tc.any() else 0.0
        if unc is not None:
            r["rel_l2_uncoded_typical"] = _rel_l2(unc[typ], exact[typ])
    return {k: (round(v, 6) if isinstance(v, float) and np.isfinite(v) else v) for k, v in r.items()}


# The four distributions the figures are quoted on: (name, generator of one operand from (synth, seed, n), outlier cut)
def distributions(synth):
    return [
        ("prefill_N(0,0.02^2)+0.1%_outliers_at_8", lambda seed, n: synth.prefill_activations(seed, n), 1.0),
        ("prefill_N(0,0.02^2)_no_outliers", lambda seed, n: synth.normal(seed, n, std=0.02), 1.0),
        ("N(0,1)", lambda seed, n: synth.normal(seed, n), 6.0),
        ("U[-4,4]", lambda seed, n: synth.uniform(seed, n), 6.0),
    ]
