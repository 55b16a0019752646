"""Shared test helpers: seeded inputs, view builders that apply the same slicing
to a numpy array (for the oracle) and to a device array, and comparisons at the
bars the parity contract states."""
import math

import numpy as np


def _ordered(a):
    """Maps floats onto an integer line in which neighbours differ by 1 (both zeros map to 0)."""
    if a.dtype == np.float32:
        i = a.view(np.int32).astype(np.int64)
        return np.where(i < 0, -(i & 0x7FFFFFFF), i)
    i = a.view(np.int64)
    mag = i & np.int64(0x7FFFFFFFFFFFFFFF)
    return np.where(i < 0, -mag, mag)


def ulp_diff(a, b):
    """Distance in units in the last place between two float arrays of one dtype
    (NaN matches NaN; signed zeros count as equal values but are reported by
    `same_bits`)."""
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape, (a.dtype, b.dtype, a.shape, b.shape)
    ai, bi = _ordered(a), _ordered(b)
    big = np.iinfo(np.int64).max
    with np.errstate(over="ignore"):
        d = ai - bi
    wrapped = ((ai >= 0) != (bi >= 0)) & ((d >= 0) != (ai >= 0))
    d = np.where(wrapped | (d == np.iinfo(np.int64).min), big, np.abs(d))
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    d = np.where(both_nan, 0, d)
    d = np.where(one_nan, np.iinfo(np.int64).max, d)
    return d


def assert_ulp(got, want, max_ulp, what=""):
    d = ulp_diff(got, want)
    if d.size and d.max() > max_ulp:
        i = np.unravel_index(np.argmax(d), d.shape)
        raise AssertionError("%s: %d ulp at %r: got %r want %r" % (what, d.max(), i, np.asarray(got)[i], np.asarray(want)[i]))


def assert_bits_equal(got, want, what=""):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert got.dtype == want.dtype, (what, got.dtype, want.dtype)
    if got.dtype.kind == "f":
        g = got.view(np.uint32 if got.dtype == np.float32 else np.uint64)
        w = want.view(np.uint32 if want.dtype == np.float32 else np.uint64)
        nan = np.isnan(got) & np.isnan(want)
        bad = (g != w) & ~nan
    else:
        bad = got != want
    if bad.any():
        i = np.unravel_index(np.argmax(bad), bad.shape)
        raise AssertionError("%s: differs at %r: got %r want %r (%d of %d differ)" % (what, i, got[i], want[i], bad.sum(), bad.size))


def reduction_tol(dtype, n):
    """rel 1e-5*log2(n) for SFloat, 1e-12*log2(n) for DFloat (n = elements folded)."""
    base = 1e-5 if np.dtype(dtype) == np.float32 else 1e-12
    return base * max(1.0, math.log2(max(2, n)))


def assert_reduction_close(got, want, n, scale=None, what=""):
    """Float reductions: |got - want| <= tol * scale, where scale defaults to
    |want| and callers of cancelling sums pass sum(|x|)."""
    got = np.asarray(got, dtype=np.float64)
    want64 = np.asarray(want, dtype=np.float64)
    tol = reduction_tol(np.asarray(want).dtype if np.asarray(want).dtype.kind == "f" else np.float64, n)
    sc = np.abs(want64) if scale is None else np.asarray(scale, dtype=np.float64)
    nan = np.isnan(want64)
    assert (np.isnan(got) == nan).all(), "%s: NaN pattern differs" % what
    inf = np.isinf(want64)
    assert ((got == want64) | ~inf).all(), "%s: inf differs" % what
    ok = nan | inf | (np.abs(got - want64) <= tol * sc + 1e-300)
    if not ok.all():
        i = np.unravel_index(np.argmax(~ok), ok.shape) if ok.shape else ()
        raise AssertionError("%s: got %r want %r tol %g scale %r" % (what, got[i], want64[i], tol, sc[i] if np.ndim(sc) else sc))


VIEW_KINDS = ["contig", "colslice", "rowslice", "transpose", "reverse", "stepneg", "bcast_row"]


def make_view(kind, arr):
    """Applies the same view to a numpy array or a cumo_amd array (both take
    __getitem__ with slices and .transpose())."""
    if kind == "contig":
        return arr
    if kind == "colslice":
        return arr[..., 1::2]
    if kind == "rowslice":
        return arr[::3]
    if kind == "transpose":
        return arr.transpose()
    if kind == "reverse":
        return arr[::-1]
    if kind == "stepneg":
        return arr[..., ::-2]
    raise ValueError(kind)
