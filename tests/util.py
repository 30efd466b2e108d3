"""Shared comparison helpers for the parity tests."""
import numpy as np


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def assert_bit_exact(got, want, what=""):
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    if got.dtype == np.float32:
        bad = np.flatnonzero(bits(got).ravel() != bits(want).ravel())
    else:
        bad = np.flatnonzero(got.ravel() != want.ravel())
    assert bad.size == 0, (f"{what}: {bad.size} of {got.size} elements differ; first at {bad[0]}: "
                           f"{got.ravel()[bad[0]]!r} vs {want.ravel()[bad[0]]!r}")


def ulp_distance(got, want):
    """distance in units of last place between two finite fp32 arrays"""
    def key(a):
        u = bits(a).astype(np.int64)
        return np.where(u & 0x80000000, 0x80000000 - u, u)
    return np.abs(key(got) - key(want))


def rel_err(got, want, floor_frac=1e-3):
    """max over elements of |g-w| / max(|w|, floor_frac*max|w|): relative error
    with the denominator floored at a fraction of the tensor's largest
    magnitude, so that cancellation to ~0 in a sum of O(1) terms is judged on
    the scale of the data rather than of the cancelled result."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = np.max(np.abs(want)) if want.size else 0.0
    den = np.maximum(np.abs(want), floor_frac * scale)
    den = np.where(den == 0, 1.0, den)
    return float(np.max(np.abs(got - want) / den)) if want.size else 0.0


def strict_rel_err(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    den = np.where(want == 0, 1.0, np.abs(want))
    return float(np.max(np.abs(got - want) / den)) if want.size else 0.0


def scaled_err(got, want, scale):
    """max |g-w| / scale, element-wise, for contractions: `scale` is the sum of
    the magnitudes of the accumulated terms, sum_k |a_ik||b_kj| (+|bias|).  Two
    fp32 evaluations of one dot product in different orders differ by up to
    ~k*eps of THAT quantity whatever the size of the (possibly cancelled)
    result, so it is the denominator a relative tolerance on a contraction can
    be held to; for sums without cancellation it equals the plain relative
    error."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = np.asarray(scale, np.float64)
    scale = np.where(scale == 0, 1.0, scale)
    return float(np.max(np.abs(got - want) / scale)) if want.size else 0.0
