"""Every SFloat NMath function over a sweep of the float bit patterns (every 64th pattern:
2^26 arguments covering every binade, both signs, subnormals, infinities and NaNs) against
the DFloat function of the same argument rounded to float once. The DFloat functions are
held to correctly rounded vectors elsewhere; this holds the SFloat algorithms, which are
evaluated in double to 2^-40 or better with the device's reciprocal estimates inside, to
the path's bar of one ulp at every argument, and counts how rarely they use it."""
import numpy as np
import pytest

from helpers import ulp_diff

pytestmark = pytest.mark.gpu

ONE = ("sqrt cbrt log log2 log10 exp exp2 exp10 sin cos tan asin acos atan sinh cosh tanh "
       "asinh acosh atanh sinc erf erfc log1p expm1").split()
STRIDE = 64


@pytest.fixture(scope="module")
def patterns():
    import cumo_amd
    bits = np.arange(0, 1 << 32, STRIDE, dtype=np.uint64).astype(np.uint32)
    # the sweep starts at +0 and, with this stride, meets -0, both infinities and 1.0 exactly
    assert 0x80000000 % STRIDE == 0 and 0x7f800000 % STRIDE == 0 and 0x3f800000 % STRIDE == 0
    x = bits.view(np.float32)
    xs = cumo_amd.SFloat.cast(x)
    xd = cumo_amd.DFloat.cast(xs)
    return x, xs, xd


def compare(name, x, got, want):
    """Results whose bits differ (the sign of a zero and the kind of a NaN included) are few:
    only those go through the ulp distance. Returns how many differ in value."""
    at = np.flatnonzero(got.view(np.uint32) != want.view(np.uint32))
    g, w, xa = got[at], want[at], x[at]
    both_nan = np.isnan(g) & np.isnan(w)
    g, w, xa = g[~both_nan], w[~both_nan], xa[~both_nan]
    if g.size == 0:
        return 0
    zeros = (g == 0) & (w == 0)
    assert not zeros.any(), "%s: the sign of a zero result differs at x=%r: SFloat %r, DFloat rounded %r" % (
        name, xa[zeros][0], g[zeros][0], w[zeros][0])
    d = ulp_diff(g, w)
    i = int(np.argmax(d))
    assert d[i] <= 1, "%s: %d ulp at x=%r (bits %08x): SFloat %r, DFloat rounded %r" % (
        name, d[i], xa[i], xa.view(np.uint32)[i], g[i], w[i])
    return int(g.size)


@pytest.mark.parametrize("name", ONE)
def test_sfloat_function_against_dfloat_function_rounded_once(patterns, name):
    import cumo_amd
    x, xs, xd = patterns
    f = getattr(cumo_amd.NMath, name)
    got = f(xs).to_numpy()
    want = cumo_amd.SFloat.cast(f(xd)).to_numpy()
    differ = compare(name, x, got, want)
    # nowhere near every argument may use the ulp: these are double evaluations rounded once
    assert differ <= x.size >> 12, (name, differ)


@pytest.mark.parametrize("y", [2.5, -0.75, 0.5, 3.0, -2.0, 10.25, 1.0 / 3.0])
def test_sfloat_power_against_dfloat_power_rounded_once(patterns, y):
    import cumo_amd
    x, xs, xd = patterns
    y = float(np.float32(y))
    got = (xs ** y).to_numpy()
    want = cumo_amd.SFloat.cast(xd ** y).to_numpy()
    differ = compare("pow %r" % y, x, got, want)
    assert differ <= x.size >> 10, (y, differ)


def test_sfloat_power_with_an_array_of_exponents(patterns):
    import cumo_amd
    x, xs, xd = patterns
    rng = np.random.default_rng(11)
    y = rng.uniform(-40, 40, x.size).astype(np.float32)
    y[::7] = np.round(y[::7])            # integers: the sign rules for a negative base
    y[::1013] = rng.choice(np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0], dtype=np.float32), y[::1013].size)
    got = (xs ** cumo_amd.SFloat.cast(y)).to_numpy()
    want = cumo_amd.SFloat.cast(xd ** cumo_amd.DFloat.cast(y.astype(np.float64))).to_numpy()
    differ = compare("pow", x, got, want)
    assert differ <= x.size >> 10, differ
