"""Reduction parity: the HIP reduction engine through the C-ABI against the CPU
oracle. Integer results, min/max values and every index are bit-exact; float sums
and moments are within rel 1e-5*log2(n) (SFloat) / 1e-12*log2(n) (DFloat) of the
oracle's sequential answer, scaled by sum(|x|) because a sum of signed values has
no scale of its own."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import numo_oracle as oracle  # noqa: E402

from helpers import assert_bits_equal, assert_reduction_close  # noqa: E402

pytestmark = pytest.mark.gpu

FLOATS = [("sfloat", np.float32), ("dfloat", np.float64)]


def cls_of(name):
    import cumo_amd
    return {"sfloat": cumo_amd.SFloat, "dfloat": cumo_amd.DFloat, "int32": cumo_amd.Int32}[name]


def host_value(r):
    """A reduction's answer as a numpy array (a full reduction answers a number or an array of no dimensions)."""
    return np.asarray(r.to_numpy() if hasattr(r, "to_numpy") else r)


def red_n(shape, axis):
    if axis is None:
        return int(np.prod(shape))
    ax = (axis,) if isinstance(axis, int) else axis
    return int(np.prod([shape[a] for a in ax]))


def abs_sum(h, axis, keepdims=False):
    return np.abs(h.astype(np.float64)).sum(axis=axis, keepdims=keepdims)


def exact_reduce(name, h, axis):
    """The reduction in extended precision (x87 long double: 64-bit mantissa)."""
    x = h.astype(np.longdouble)
    if name == "sum":
        r = x.sum(axis=axis)
    elif name == "mean":
        r = x.mean(axis=axis)
    elif name == "var":
        r = x.var(axis=axis, ddof=1)
    elif name == "stddev":
        r = np.sqrt(x.var(axis=axis, ddof=1))
    elif name == "rms":
        r = np.sqrt((x * x).mean(axis=axis))
    else:
        raise ValueError(name)
    return np.asarray(r, dtype=np.float64)


VIEWS = {
    "contig": lambda a: a,
    "colslice": lambda a: a[..., 1::2],
    "rowslice": lambda a: a[::2],
    "transpose": lambda a: a.transpose(),
    "reverse": lambda a: a[::-1],
    "middle": lambda a: a[:, 1:-1] if a.ndim > 1 else a[1:-1],
}


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("view", list(VIEWS))
def test_float_reductions_every_axis(tname, dt, view):
    # the pattern of test/narray_test.rb:3449-3486,4329-4363: every reduction over every
    # axis of several kinds of view
    rng = np.random.default_rng(200)
    cls = cls_of(tname)
    h = (rng.integers(-64, 64, size=(12, 20, 36)) / 16.0).astype(dt)  # multiples of 1/16: many ties
    d = cls.cast(h)
    hv, dv = VIEWS[view](h), VIEWS[view](d)
    for axis in [None, 0, 1, 2, -1, (0, 1), (1, 2), (0, 2)]:
        n = red_n(hv.shape, axis if axis != -1 else 2)
        for name in ("min", "max", "ptp"):
            assert_bits_equal(getattr(dv, name)(axis=axis).to_numpy(), oracle.reduce(name, hv, axis=axis), "%s %s %r" % (name, view, axis))
        for name in ("argmin", "argmax"):
            assert_bits_equal(getattr(dv, name)(axis=axis).to_numpy(), oracle.reduce(name, hv, axis=axis), "%s %s %r" % (name, view, axis))
        # sums of multiples of 1/16 this small are exact in any order
        assert_bits_equal(dv.sum(axis=axis).to_numpy(), oracle.reduce("sum", hv, axis=axis), "sum %s %r" % (view, axis))
        assert_reduction_close(dv.mean(axis=axis).to_numpy(), oracle.reduce("mean", hv, axis=axis), n, abs_sum(hv, axis) / n, "mean")
        for name in ("var", "stddev", "rms"):
            want = oracle.reduce(name, hv, axis=axis)
            assert_reduction_close(getattr(dv, name)(axis=axis).to_numpy(), want, n, np.abs(want) + 1e-30, "%s %s %r" % (name, view, axis))
        lo, hi = dv.minmax(axis=axis)
        assert_bits_equal(lo.to_numpy(), oracle.reduce("min", hv, axis=axis))
        assert_bits_equal(hi.to_numpy(), oracle.reduce("max", hv, axis=axis))
    # keepdims
    assert dv.sum(axis=1, keepdims=True).shape == tuple(1 if k == 1 else s for k, s in enumerate(hv.shape))
    assert_bits_equal(dv.max(axis=(0, 2), keepdims=True).to_numpy(), oracle.reduce("max", hv, axis=(0, 2), keepdims=True))
    # max_index / min_index answer positions in the view's own flattening
    assert_bits_equal(dv.max_index(axis=1).to_numpy(), oracle.reduce("max_index", np.ascontiguousarray(hv), axis=1))
    assert_bits_equal(dv.min_index().to_numpy(), oracle.reduce("min_index", np.ascontiguousarray(hv)))


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_reductions_along_an_axis_that_strides_through_memory(tname, dt):
    """Full and partial reductions of transposed and permuted views of 65536 elements or more, where the reduce
    axis' lanes would stride through memory: the view is copied into its own order first. Ties, both zeros and
    positions answer in the view's order."""
    rng = np.random.default_rng(207)
    cls = cls_of(tname)
    if dt == np.int32:
        h2 = rng.integers(-50, 50, size=(300, 260)).astype(dt)
        h3 = rng.integers(-50, 50, size=(40, 50, 64)).astype(dt)
    else:
        h2 = (rng.integers(-8, 8, size=(300, 260)) / 4.0).astype(dt)
        h3 = (rng.integers(-8, 8, size=(40, 50, 64)) / 4.0).astype(dt)
        h2[h2 == 0] = np.where(rng.random(int((h2 == 0).sum())) < 0.5, dt(-0.0), dt(0.0))
        h2 = np.minimum(h2, dt(0.0))       # the maximum is a zero: which one depends on the view's order
    d2, d3 = cls.cast(h2), cls.cast(h3)
    cases = [(d2.transpose(), h2.T, None), (d2.transpose(), h2.T, 1), (d2.transpose()[::2, 3:], h2.T[::2, 3:], None),
             (d3.transpose(2, 1, 0), h3.transpose(2, 1, 0), None), (d3.transpose(2, 1, 0), h3.transpose(2, 1, 0), (1, 2)),
             (d3.transpose(1, 2, 0), h3.transpose(1, 2, 0), (0, 2)), (d3.transpose(0, 2, 1), h3.transpose(0, 2, 1), 2)]
    for dv, hv, axis in cases:
        hv = np.ascontiguousarray(hv)
        what = "%r axis %r" % (hv.shape, axis)
        for name in ("min", "max", "sum", "argmin", "argmax", "ptp"):
            got = getattr(dv, name)(axis=axis)
            got = np.asarray(got.to_numpy() if hasattr(got, "to_numpy") else got)
            want = np.asarray(oracle.reduce(name, hv, axis=axis))
            assert_bits_equal(got.astype(want.dtype), want, "%s %s" % (name, what))
        lo, hi = (np.asarray(v.to_numpy() if hasattr(v, "to_numpy") else v, dtype=dt) for v in dv.minmax(axis=axis))
        assert_bits_equal(lo, np.asarray(oracle.reduce("min", hv, axis=axis), dtype=dt), "minmax lo " + what)
        assert_bits_equal(hi, np.asarray(oracle.reduce("max", hv, axis=axis), dtype=dt), "minmax hi " + what)
        if dt != np.int32:
            n = red_n(hv.shape, axis)
            want = oracle.reduce("var", hv, axis=axis)
            got = dv.var(axis=axis)
            got = np.asarray(got.to_numpy() if hasattr(got, "to_numpy") else got)
            assert_reduction_close(got, want, n, np.abs(want) + 1e-30, "var " + what)
        got = dv.max_index(axis=axis)
        got = np.asarray(got.to_numpy() if hasattr(got, "to_numpy") else got)
        assert_bits_equal(got, np.asarray(oracle.reduce("max_index", hv, axis=axis)).astype(got.dtype), "max_index " + what)


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_one_result_over_views_whose_rows_do_not_follow_one_another(tname, dt):
    """x[true, 1..-1].sum and its like: a full reduction over a view of 65536 elements or more whose innermost dimension
    runs along memory while the outer ones do not merge with it goes rows first, then over the rows' results. Sums
    within the reduction tolerance; min / max exactly, the zero that comes first in the view's order included."""
    rng = np.random.default_rng(209)
    cls = cls_of(tname)
    if dt == np.int32:
        h2 = rng.integers(-50, 50, size=(300, 260)).astype(dt)
        h3 = rng.integers(-50, 50, size=(12, 50, 131)).astype(dt)
    else:
        h2 = (rng.integers(-8, 8, size=(300, 260)) / 4.0).astype(dt)
        h3 = (rng.integers(-8, 8, size=(12, 50, 131)) / 4.0).astype(dt)
    d2, d3 = cls.cast(h2), cls.cast(h3)
    views = [(d2[:, 1:], h2[:, 1:]), (d2[::-1, :-3], h2[::-1, :-3]), (d3[:, :, 1:], h3[:, :, 1:]), (d3[::2, 1:, 2:-1], h3[::2, 1:, 2:-1]),
             (d3.transpose(1, 0, 2)[:, :, 3:], h3.transpose(1, 0, 2)[:, :, 3:])]
    for dv, hv in views:
        hv = np.ascontiguousarray(hv)
        what = "%r" % (hv.shape,)
        n = hv.size
        for name in ("min", "max"):
            got = host_value(getattr(dv, name)())
            assert_bits_equal(got.astype(dt), np.asarray(oracle.reduce(name, hv, axis=None), dtype=dt), "%s %s" % (name, what))
        if dt != np.int32:
            for name in ("sum", "mean"):
                want = exact_reduce(name, hv, None)
                got = host_value(getattr(dv, name)()).astype(np.float64)
                scale = abs_sum(hv, None) / (n if name == "mean" else 1)
                assert_reduction_close(got.astype(dt), want.astype(dt), n, scale, "%s %s" % (name, what))
    if dt != np.int32:
        # the zero that comes first: a matrix of zeros of both signs, seen through the slice
        z = np.where(rng.random((300, 260)) < 0.5, dt(0.0), dt(-0.0)).astype(dt)
        dz = cls.cast(z)
        for dv, hv in ((dz[:, 1:], z[:, 1:]), (dz[::-1, 2:], z[::-1, 2:]), (dz[5:, :-1], z[5:, :-1])):
            hv = np.ascontiguousarray(hv)
            for name in ("min", "max"):
                got = host_value(getattr(dv, name)()).astype(dt)
                assert_bits_equal(got, np.asarray(oracle.reduce(name, hv, axis=None), dtype=dt), "%s of zeros %r" % (name, hv.shape))
        hp = (1.0 + rng.uniform(-1, 1, size=(300, 260)) * 1e-4).astype(dt)
        want = np.prod(hp[:, 1:].astype(np.longdouble))
        got = host_value(cls.cast(hp)[:, 1:].prod()).astype(np.float64)
        # (every multiplication rounds: n / 2 units in the last place at worst)
        assert abs(float(got) / float(want) - 1.0) <= hp[:, 1:].size * np.finfo(dt).eps / 2, ("prod", float(got), float(want))


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("shape", [(4096, 1023), (4096, 1022), (2048, 1021), (4098, 1023), (4097, 1023), (1024, 4095)])
def test_column_sums_of_rows_that_are_not_whole_vectors(tname, dt, shape):
    """sum / mean / prod (and the nan forms of the first two) down the columns of a contiguous matrix whose rows are not
    whole 16-byte vectors, a few thousand columns wide: the axis is cut across blocks and a second launch folds the parts."""
    rng = np.random.default_rng(208)
    cls = cls_of(tname)
    h = rng.uniform(-1, 1, size=shape).astype(dt)
    h[rng.random(shape) < 0.001] = np.nan
    hn = np.where(np.isnan(h), dt(0.25), h)
    n = shape[0]
    for src, names in ((hn, ("sum", "mean")), (h, ("sum", "mean"))):
        d = cls.cast(src)
        for name in names:
            nan = src is h
            want = exact_reduce(name, hn if not nan else np.where(np.isnan(h), 0, h), 0)
            if nan and name == "mean":
                want = want * n / np.maximum((~np.isnan(h)).sum(axis=0), 1)
            got = getattr(d, name)(axis=0, nan=True).to_numpy() if nan else getattr(d, name)(axis=0).to_numpy()
            scale = abs_sum(hn, 0) / (n if name == "mean" else 1)
            assert_reduction_close(got, want.astype(dt), n, scale, "%s nan=%r %r" % (name, nan, shape))
        if src is h:
            # without nan: true a NaN anywhere in the column is the answer
            got = d.sum(axis=0).to_numpy()
            assert (np.isnan(got) == np.isnan(h).any(axis=0)).all()
    # products of numbers next to 1, so that 4096 of them stay in range
    hp = (1.0 + rng.uniform(-1, 1, size=shape) * 1e-3).astype(dt)
    want = np.prod(hp.astype(np.longdouble), axis=0)
    got = cls.cast(hp).prod(axis=0).to_numpy()
    assert_reduction_close(got, want.astype(dt), n, np.abs(want).astype(np.float64), "prod %r" % (shape,))


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("shape,axis", [((1000003,), None), ((7, 100000), 1), ((100000, 7), 0), ((3, 40000, 5), 1),
                                        ((64, 64, 64), (0, 2)), ((2, 3), None), ((1,), None), ((70000, 3), 1),
                                        ((5, 8192), 1), ((4096, 33), 0), ((33, 4096), 0), ((3, 2000003), 1), ((130, 40000), 1), ((260, 30000), 1)])
def test_random_float_sums(tname, dt, shape, axis):
    rng = np.random.default_rng(201)
    cls = cls_of(tname)
    h = rng.uniform(-1, 1, size=shape).astype(dt)
    d = cls.cast(h)
    n = red_n(shape, axis)
    # Numo folds a float32 axis sequentially, so over 10^6 elements its own answer
    # carries up to n*eps/2 of rounding (var of 10^6 uniform values is 3.7e-4 off
    # the exact value). The device is held to the stated tolerance against the
    # EXACT value (extended precision), and the oracle is shown to sit within its
    # a-priori sequential bound of the same value: the two agree to that.
    names = ["sum", "mean", "rms"] + (["var", "stddev"] if n > 1 else [])
    for name in names:
        want = exact_reduce(name, h, axis)
        scale = {"sum": abs_sum(h, axis), "mean": abs_sum(h, axis) / n}.get(name, np.abs(want))
        got = getattr(d, name)(axis=axis).to_numpy()
        assert_reduction_close(got, want.astype(dt), n, scale, name)
        ora = oracle.reduce(name, h, axis=axis).astype(np.float64)
        eps = np.finfo(dt).eps
        assert (np.abs(ora - want) <= (2 * n * eps) * np.asarray(scale, dtype=np.float64) + 1e-300).all(), "oracle %s" % name
    assert_bits_equal(d.max(axis=axis).to_numpy(), oracle.reduce("max", h, axis=axis))
    assert_bits_equal(d.min(axis=axis).to_numpy(), oracle.reduce("min", h, axis=axis))
    assert_bits_equal(d.argmax(axis=axis).to_numpy(), oracle.reduce("argmax", h, axis=axis))
    assert_bits_equal(d.argmin(axis=axis).to_numpy(), oracle.reduce("argmin", h, axis=axis))
    p = oracle.reduce("prod", (h[..., :20] if h.ndim > 1 else h[:20]) * 1.5, axis=-1)
    dp = cls.cast(np.ascontiguousarray((h[..., :20] if h.ndim > 1 else h[:20]) * dt(1.5)))
    assert_reduction_close(dp.prod(axis=-1).to_numpy(), p, 20, np.abs(p), "prod")


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_nan_rules(tname, dt):
    rng = np.random.default_rng(202)
    cls = cls_of(tname)
    h = rng.standard_normal((9, 3000)).astype(dt)
    h[0, 5] = np.nan          # one NaN
    h[1, :] = np.nan          # a whole row
    h[2, 0] = np.nan          # leading
    h[3, -1] = np.nan         # trailing
    h[4, ::2] = np.nan        # half
    h[5, 100] = np.inf
    h[6, 200] = -np.inf
    d = cls.cast(h)
    for nan in (False, True):
        for name in ("min", "max", "ptp", "argmin", "argmax"):
            assert_bits_equal(getattr(d, name)(axis=1, nan=nan).to_numpy(), oracle.reduce(name, h, axis=1, nan=nan), "%s nan=%s" % (name, nan))
            assert_bits_equal(getattr(d, name)(axis=0, nan=nan).to_numpy(), oracle.reduce(name, h, axis=0, nan=nan), "%s nan=%s axis0" % (name, nan))
        for name in ("sum", "mean", "rms"):
            want = oracle.reduce(name, h, axis=1, nan=nan)
            got = getattr(d, name)(axis=1, nan=nan).to_numpy()
            fin = np.isfinite(want)
            assert (np.isnan(got) == np.isnan(want)).all(), name
            assert_reduction_close(got[fin], want[fin], 3000, np.nansum(np.abs(h[fin].astype(np.float64)), axis=1) if name == "sum" else np.abs(want[fin]) + 1e-3, name)
        for name in ("var", "stddev"):
            want = oracle.reduce(name, h[:5], axis=1, nan=nan)
            got = getattr(d[:5], name)(axis=1, nan=nan).to_numpy()
            assert (np.isnan(got) == np.isnan(want)).all(), name
            fin = np.isfinite(want)
            assert_reduction_close(got[fin], want[fin], 3000, np.abs(want[fin]), name)
    lo, hi = d.minmax(axis=1, nan=True)
    assert_bits_equal(lo.to_numpy(), oracle.reduce("min", h, axis=1, nan=True))
    assert_bits_equal(hi.to_numpy(), oracle.reduce("max", h, axis=1, nan=True))
    # signed zeros: the earlier of two equal elements (test/narray_test.rb:667-672), also across lanes
    z = np.zeros(5000, dtype=dt)
    z[1::2] = -0.0
    for arr in (z, -z, z[::-1].copy()):
        dz = cls.cast(arr)
        assert_bits_equal(dz.min().to_numpy(), oracle.reduce("min", arr))
        assert_bits_equal(dz.max().to_numpy(), oracle.reduce("max", arr))


def test_int32_reductions():
    rng = np.random.default_rng(203)
    cls = cls_of("int32")
    h = rng.integers(-2**30, 2**30, size=(17, 33, 20), dtype=np.int32)
    d = cls.cast(h)
    for view in VIEWS:
        hv, dv = VIEWS[view](h), VIEWS[view](d)
        for axis in [None, 0, 1, 2, (0, 2)]:
            for name in ("sum", "min", "max", "ptp", "argmin", "argmax"):
                assert_bits_equal(getattr(dv, name)(axis=axis).to_numpy(), oracle.reduce(name, hv, axis=axis), "%s %s %r" % (name, view, axis))
    small = rng.integers(-3, 4, size=(6, 12), dtype=np.int32)
    assert_bits_equal(cls.cast(small).prod(axis=1).to_numpy(), oracle.reduce("prod", small, axis=1))
    lo, hi = d.minmax(axis=1)
    assert_bits_equal(lo.to_numpy(), h.min(axis=1))
    assert_bits_equal(hi.to_numpy(), h.max(axis=1))
    big = rng.integers(-2**31, 2**31 - 1, size=3000001, dtype=np.int32)
    assert int(cls.cast(big).sum()) == int(big.astype(np.int64).sum())
    assert cls.cast(big).sum().to_numpy().dtype == np.int64


def test_empty_and_degenerate():
    import cumo_amd
    # reference: narray/narray.c:1704-1716 -- "cannot reduce empty NArray", whatever the axis
    for empty in (cumo_amd.SFloat.zeros(0, 5), cumo_amd.SFloat.zeros(4, 0), cumo_amd.SFloat.zeros(0)):
        for op in ("sum", "max", "argmax", "mean"):
            with pytest.raises(cumo_amd.ShapeError):
                getattr(empty, op)(axis=0)
    with pytest.raises(ValueError):
        cumo_amd.SFloat.zeros(3, 4).sum(axis=2)   # DimensionError: dimension is out of range
    one0 = cumo_amd.DFloat.cast(np.array(2.5))    # a 0-dimensional array reduces to itself
    assert float(one0.sum()) == 2.5 and int(one0.argmax()) == 0
    one = cumo_amd.DFloat.cast(np.array([[3.5]]))
    assert float(one.sum()) == 3.5 and float(one.max(axis=0).to_numpy()[0]) == 3.5
    assert int(one.argmax()) == 0


def test_dfloat_kahan_sum():
    import cumo_amd
    h = np.array([1e16, 1.0, -1e16, 1.0] * 1000)
    assert float(cumo_amd.DFloat.cast(h).kahan_sum()) == 2000.0


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("shape,axis", [((300, 77), 1), ((300, 77), 0), ((5, 20000), 1), ((20000, 5), 0), ((3000001,), None),
                                        ((64, 33, 40), (0, 2)), ((6, 70000), 1), ((2, 3, 4096), 2), ((3000, 1000), 0), ((70000, 64), 0),
                                        ((8192, 260), 0), ((4, 512, 256), 1), ((3, 130, 64), 1)])
def test_min_max_keep_the_zero_that_came_first(tname, dt, shape, axis):
    # Numo's sequential loop only replaces on a strict comparison (real_accum.h:217-278), so of
    # +0 and -0 the earlier one is the answer. Every output here ends on a zero, with both signs
    # present at seeded positions, through the row, column, block-wide and split kernels.
    rng = np.random.default_rng(411)
    cls = cls_of(tname)
    sign = rng.integers(0, 2, size=shape).astype(bool)
    zero = rng.random(shape) < 0.05
    mag = rng.random(shape).astype(dt) + dt(0.5)
    for name, away in (("max", -1.0), ("min", 1.0)):
        h = (mag * dt(away)).astype(dt)
        h[zero] = 0.0
        h[zero & sign] = -0.0
        d = cls.cast(h)
        want = oracle.reduce(name, h, axis=axis)
        got = getattr(d, name)(axis=axis).to_numpy()
        assert_bits_equal(got, want, "%s %r axis %r" % (name, shape, axis))
        if want.size >= 100:
            zeros = want[want == 0]
            assert np.signbit(zeros).any() and not np.signbit(zeros).all(), "the inputs are meant to produce both signs"
        # minmax answers the same zero at that end, and the other end as min / max alone do
        if not isinstance(axis, tuple):
            lo, hi = (np.asarray(v.to_numpy() if hasattr(v, "to_numpy") else v, dtype=dt) for v in d.minmax(axis=axis))
            assert_bits_equal(lo, np.asarray(oracle.reduce("min", h, axis=axis), dtype=dt), "minmax lo %r axis %r" % (shape, axis))
            assert_bits_equal(hi, np.asarray(oracle.reduce("max", h, axis=axis), dtype=dt), "minmax hi %r axis %r" % (shape, axis))
    # both ends zero: every element a zero of either sign
    hz = np.where(sign, dt(-0.0), dt(0.0)).astype(dt)
    dz = cls.cast(hz)
    if not isinstance(axis, tuple):
        lo, hi = (np.asarray(v.to_numpy() if hasattr(v, "to_numpy") else v, dtype=dt) for v in dz.minmax(axis=axis))
        assert_bits_equal(lo, np.asarray(oracle.reduce("min", hz, axis=axis), dtype=dt), "minmax of zeros, lo")
        assert_bits_equal(hi, np.asarray(oracle.reduce("max", hz, axis=axis), dtype=dt), "minmax of zeros, hi")
        spread = dz.ptp(axis=axis)
        spread = np.asarray(spread.to_numpy() if hasattr(spread, "to_numpy") else spread, dtype=dt)
        assert (spread == 0).all() and not np.signbit(spread).any()
    # NaN in the mix: skipped unless the output holds nothing else
    h = (mag * dt(-1.0)).astype(dt)
    h[zero] = np.nan
    h[..., 0] = np.nan
    d = cls.cast(h)
    assert_bits_equal(d.max(axis=axis).to_numpy(), oracle.reduce("max", h, axis=axis), "max with NaN")
    alln = np.full(shape, np.nan, dtype=dt)
    assert np.isnan(cls.cast(alln).max(axis=axis).to_numpy()).all()


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("shape,axis", [((700, 24), 0), ((3, 700, 24), 1), ((40000, 8), 0), ((2, 5000, 3), 1), ((130, 1024), 0),
                                        ((3000, 1000), 0), ((4096, 520), 0), ((2, 2100, 516), 1), ((3000, 1001), 0), ((700, 4095), 0),
                                        ((40, 70001), 0), ((5000, 259), 0), ((70000, 64), 0), ((8192, 1028), 0),
                                        ((3, 700, 67), 1), ((5, 64, 1023), 1), ((2, 2100, 517), 1), ((9, 130, 259), 1), ((64, 40, 131), 1),
                                        ((300, 20, 33), 1)])
def test_few_outputs_across_memory_share_the_axis_inside_a_block(tname, dt, shape, axis):
    """The column kernel with the reduce axis cut inside the block (and, for the long ones, across
    blocks as well): ties resolve to the lowest index across the parts, NaN rules, both results of
    minmax, moments, every value exact where the arithmetic allows."""
    import cumo_amd
    rng = np.random.default_rng(77)
    cls = cls_of(tname)
    h = (rng.integers(-8, 8, size=shape) / 4.0).astype(dt)          # few distinct values: ties everywhere
    d = cls.cast(h)
    n = shape[axis]
    for name in ("min", "max", "ptp", "argmin", "argmax", "sum"):
        assert_bits_equal(getattr(d, name)(axis=axis).to_numpy(), oracle.reduce(name, h, axis=axis), name)
    lo, hi = d.minmax(axis=axis)
    assert_bits_equal(lo.to_numpy(), oracle.reduce("min", h, axis=axis))
    assert_bits_equal(hi.to_numpy(), oracle.reduce("max", h, axis=axis))
    assert_bits_equal(d.max_index(axis=axis).to_numpy(), oracle.reduce("max_index", h, axis=axis))
    for name in ("mean", "var", "stddev", "rms"):
        want = oracle.reduce(name, h, axis=axis)
        assert_reduction_close(getattr(d, name)(axis=axis).to_numpy(), want, n, np.abs(want) + 1e-30, name)
    # NaN: skipped by default, winning with nan: true, the first one for the arg forms
    hn = h.copy()
    hn[rng.random(shape) < 0.01] = np.nan
    hn[(slice(None),) * axis + (slice(n // 2, None),) + (slice(None),) * (len(shape) - axis - 1)][..., 0] = np.nan
    dn = cls.cast(hn)
    for name in ("min", "max", "argmin", "argmax", "sum"):
        for nan in (False, True):
            got = getattr(dn, name)(axis=axis, nan=nan).to_numpy()
            want = oracle.reduce(name, hn, axis=axis, nan=nan)
            if name == "sum":
                assert (np.isnan(got) == np.isnan(want)).all() and (got[~np.isnan(want)] == want[~np.isnan(want)]).all(), (name, nan)
            else:
                assert_bits_equal(got, want, "%s nan=%s" % (name, nan))
    hi32 = rng.integers(-1000, 1000, size=shape).astype(np.int32)
    di = cumo_amd.Int32.cast(hi32)
    for name in ("sum", "min", "max", "argmax", "argmin"):
        assert (getattr(di, name)(axis=axis).to_numpy() == oracle.reduce(name, hi32, axis=axis)).all(), name


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("shape,axis", [((7, 1027), 1), ((1, 4099), 1), ((2051,), None), ((3, 5, 1030), 2), ((300001,), None), ((40, 20011), 1),
                                        ((64, 1023), 1), ((9, 5, 131), 2), ((33, 67), 1), ((5, 33), 1)])
def test_runs_that_end_in_part_of_a_vector(tname, dt, shape, axis):
    """A contiguous reduce axis of 16 vectors or more that is not a whole number of vectors: the
    lean row kernels take its whole vectors and one lane folds the last one to three elements.
    What decides the answer is put into those last elements: the extreme, a tie with an earlier
    element (the earlier index wins), the zero of the other sign (the one that came first wins),
    a NaN (skipped, or winning with nan: true), a large addend; the ordinary case beside them."""
    import cumo_amd
    rng = np.random.default_rng(91)
    cls = cls_of(tname)
    n = shape[-1]
    base = (rng.integers(-8, 8, size=shape) / 4.0).astype(dt)
    cases = {"plain": base}
    h = base.copy(); h[..., -1] = 50.0; h[..., -2] = -50.0
    cases["extremes at the end"] = h
    h = base.copy(); h[..., 5] = 9.0; h[..., -1] = 9.0; h[..., 7] = -9.0; h[..., -1 - (n % 2)] = -9.0 if n % 2 else h[..., -1]
    cases["ties with the end"] = h
    h = np.abs(base) + 1.0; h[..., 3] = -0.0; h[..., -1] = 0.0
    cases["zeros: minus first, plus in the last element"] = h
    h = -np.abs(base) - 1.0; h[..., -1] = -0.0; h[..., 11] = 0.0
    cases["zeros: plus first, minus in the last element"] = h
    h = base.copy(); h[..., -1] = np.nan
    cases["NaN in the last element"] = h
    h = base.copy(); h[..., -1] = 2.0 ** 20
    cases["a large last addend"] = h
    for what, h in cases.items():
        d = cls.cast(h)
        has_nan = bool(np.isnan(h).any())
        for name in ("min", "max", "argmin", "argmax", "sum", "ptp"):
            for nan in ((False, True) if has_nan and name != "ptp" else (False,)):
                kw = {"nan": True} if nan else {}
                got = getattr(d, name)(axis=axis, **kw).to_numpy()
                want = oracle.reduce(name, h, axis=axis, **kw)
                assert_bits_equal(got, want, "%s: %s nan=%s" % (what, name, nan))
        lo, hi = d.minmax(axis=axis)
        assert_bits_equal(lo.to_numpy(), oracle.reduce("min", h, axis=axis), what)
        assert_bits_equal(hi.to_numpy(), oracle.reduce("max", h, axis=axis), what)
        if not has_nan:
            # against the value in extended precision (a float32 oracle that adds 300001 squares in turn is
            # itself further from it than the bar)
            for name in ("mean", "var", "stddev", "rms"):
                want = exact_reduce(name, h, axis)
                scale = abs_sum(h, axis) / n if name == "mean" else np.abs(want) + 1e-30
                assert_reduction_close(getattr(d, name)(axis=axis).to_numpy(), want.astype(dt), n, scale, "%s: %s" % (what, name))
            hp = np.where(rng.random(shape) < 0.01, 2.0, 1.0).astype(dt) * np.where(rng.random(shape) < 0.5, 1.0, -1.0).astype(dt)
            hp[..., -1] = -2.0
            assert_bits_equal(cls.cast(hp).prod(axis=axis).to_numpy(), np.asarray(oracle.reduce("prod", hp, axis=axis)), what + ": prod")
    hi32 = rng.integers(-1000, 1000, size=shape).astype(np.int32)
    hi32[..., -1] = 5000
    di = cumo_amd.Int32.cast(hi32)
    for name in ("sum", "min", "max", "argmax", "argmin"):
        assert (getattr(di, name)(axis=axis).to_numpy() == oracle.reduce(name, hi32, axis=axis)).all(), name


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_reductions_of_slices_that_start_off_a_16_byte_boundary(tname, dt):
    """Inner slices beginning at an odd column, with lengths that are whole 128-bit accesses: the
    kernels read them with wide loads on element boundaries; along the rows, down the columns, all."""
    rng = np.random.default_rng(808)
    cls = cls_of(tname)
    h = (rng.integers(-64, 64, size=(9, 70, 1040)) / 16.0).astype(dt)
    d = cls.cast(h)
    for lo, n in ((1, 1024), (3, 1000), (2, 8), (5, 512)):
        hv, dv = np.ascontiguousarray(h[:, :, lo:lo + n]), d[:, :, lo:lo + n]
        for axis in (2, 1, 0, (0, 1), (1, 2), None):
            for name in ("sum", "min", "max", "argmax", "argmin"):
                assert_bits_equal(getattr(dv, name)(axis=axis).to_numpy(), oracle.reduce(name, hv, axis=axis), "%s %r %r" % (name, (lo, n), axis))
            # the moments against the exact value (the sequential float32 loop is itself further from it)
            exact = hv.astype(np.float64).var(axis=axis, ddof=1)
            assert np.allclose(dv.var(axis=axis).to_numpy(), exact, rtol=2e-5 if dt == np.float32 else 1e-12, atol=0), ("var", lo, n, axis)
    i = rng.integers(-1000, 1000, size=(50, 1030)).astype(np.int32)
    import cumo_amd
    di = cumo_amd.Int32.cast(i)
    for axis in (0, 1, None):
        assert (di[:, 3:1027].sum(axis=axis).to_numpy() == oracle.reduce("sum", np.ascontiguousarray(i[:, 3:1027]), axis=axis)).all()
        assert (di[:, 3:1027].argmax(axis=axis).to_numpy() == oracle.reduce("argmax", np.ascontiguousarray(i[:, 3:1027]), axis=axis)).all()
