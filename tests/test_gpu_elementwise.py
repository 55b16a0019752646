"""Elementwise parity: the HIP path through the C-ABI against the CPU oracle on the
same seeded inputs. Bit-exact for arithmetic that is a single IEEE operation, for
Int32 and for Bit results; <= 1 ulp for libm functions."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import numo_oracle as oracle  # noqa: E402

from helpers import assert_bits_equal, assert_ulp  # noqa: E402

pytestmark = pytest.mark.gpu

FLOATS = [("sfloat", np.float32), ("dfloat", np.float64)]
PYOP = {"add": "__add__", "sub": "__sub__", "mul": "__mul__", "div": "__truediv__", "mod": "__mod__"}
RPYOP = {"add": "__radd__", "sub": "__rsub__", "mul": "__rmul__", "div": "__rtruediv__", "mod": "__rmod__"}


def cls_of(name):
    import cumo_amd
    return {"sfloat": cumo_amd.SFloat, "dfloat": cumo_amd.DFloat, "int32": cumo_amd.Int32}[name]


def views_of(shape_kind, host, dev):
    """Pairs (numpy view, device view) built by the same slicing."""
    if shape_kind == "contig":
        return host, dev
    if shape_kind == "colslice":
        return host[..., 1::2], dev[..., 1::2]
    if shape_kind == "rowslice":
        return host[::3], dev[::3]
    if shape_kind == "transpose":
        return host.T, dev.transpose()
    if shape_kind == "reverse":
        return host[::-1, ::-1], dev[::-1, ::-1]
    if shape_kind == "offset":
        return host[1:, 3:], dev[1:, 3:]
    raise ValueError(shape_kind)


VIEW_KINDS = ["contig", "colslice", "rowslice", "transpose", "reverse", "offset"]


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "mod"])
@pytest.mark.parametrize("kind", VIEW_KINDS)
def test_float_binary_over_views(tname, dt, op, kind):
    rng = np.random.default_rng(100)
    cls = cls_of(tname)
    hx = rng.standard_normal((96, 200)).astype(dt)
    hy = (rng.standard_normal((96, 200)) + 0.5).astype(dt)
    hx[2, 5] = np.nan
    hy[4, 7] = 0.0
    dx, dy = cls.cast(hx), cls.cast(hy)
    vx, wx = views_of(kind, hx, dx)
    vy, wy = views_of(kind, hy, dy)
    with np.errstate(all="ignore"):
        want = oracle.binary(op, vx, vy)
    got = getattr(wx, PYOP[op])(wy).to_numpy()
    assert_bits_equal(got, want, "%s %s %s" % (tname, op, kind))
    # scalar on either side
    with np.errstate(all="ignore"):
        assert_bits_equal(getattr(wx, PYOP[op])(2.5).to_numpy(), oracle.binary(op, vx, 2.5), "scalar right")
        assert_bits_equal(getattr(wx, RPYOP[op])(2.5).to_numpy(), oracle.binary(op, 2.5, vx, scalar_is_left=True), "scalar left")


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_broadcast_shapes(tname, dt):
    rng = np.random.default_rng(101)
    cls = cls_of(tname)
    a = rng.standard_normal((33, 64)).astype(dt)
    for other_shape in [(1, 64), (64,), (33, 1), (1, 1), (1,)]:
        b = rng.standard_normal(other_shape).astype(dt)
        assert_bits_equal((cls.cast(a) + cls.cast(b)).to_numpy(), oracle.binary("add", a, b), str(other_shape))
        assert_bits_equal((cls.cast(b) - cls.cast(a)).to_numpy(), oracle.binary("sub", b, a), str(other_shape))
    # more dims, both sides broadcasting
    p = rng.standard_normal((5, 1, 7, 1)).astype(dt)
    q = rng.standard_normal((4, 1, 9)).astype(dt)
    assert_bits_equal((cls.cast(p) * cls.cast(q)).to_numpy(), oracle.binary("mul", p, q))
    import cumo_amd
    with pytest.raises(cumo_amd.ShapeError):
        cls.cast(a) + cls.cast(np.zeros((32, 64), dtype=dt))


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_matrices_with_rows_of_an_odd_length_and_a_second_operand(tname, dt):
    """A contiguous matrix whose rows are not a whole number of 128-bit vectors (op) a row vector, a
    column vector or a strided view of its own shape, on either side: the matrix and the result go
    as one run each, the other operand is addressed by row and column. Totals that end in part of
    a vector; a row shorter than two vectors from the end (vectors that straddle two rows)."""
    import cumo_amd
    rng = np.random.default_rng(303)
    cls = cls_of(tname)
    for (R, Cn) in [(37, 65), (130, 4095), (5, 1001), (64, 67), (3, 70001), (1025, 129)]:
        a = rng.standard_normal((R, Cn)).astype(dt)
        da = cls.cast(a)
        wide = rng.standard_normal((R, 2 * Cn)).astype(dt)
        for what, b, db in [("row", None, None), ("column", None, None), ("view", None, None)]:
            if what == "row":
                b = rng.standard_normal((1, Cn)).astype(dt); db = cls.cast(b)
            elif what == "column":
                b = rng.standard_normal((R, 1)).astype(dt); db = cls.cast(b)
            else:
                b = np.ascontiguousarray(wide[:, ::2]); db = cls.cast(wide)[:, ::2]
            for name, f in (("add", lambda x, y: x + y), ("sub", lambda x, y: x - y), ("mul", lambda x, y: x * y), ("div", lambda x, y: x / y)):
                assert_bits_equal(f(da, db).to_numpy(), oracle.binary(name, a, b), "%s: matrix %s %s" % ((R, Cn), name, what))
                assert_bits_equal(f(db, da).to_numpy(), oracle.binary(name, b, a), "%s: %s %s matrix" % ((R, Cn), what, name))
    # Int32: wrapping arithmetic, and a division that meets a zero raises as everywhere else
    hi = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(33, 131)).astype(np.int32)
    hr = rng.integers(-1000, 1000, size=(1, 131)).astype(np.int32)
    di, dr = cumo_amd.Int32.cast(hi), cumo_amd.Int32.cast(hr)
    assert ((di + dr).to_numpy() == oracle.binary("add", hi, hr)).all()
    assert ((dr * di).to_numpy() == oracle.binary("mul", hr, hi)).all()
    hz = hr.copy()
    hz[hz == 0] = 7
    assert ((di / cumo_amd.Int32.cast(hz)).to_numpy() == oracle.binary("div", hi, hz)).all()
    hz[0, 100] = 0
    with pytest.raises(ZeroDivisionError):
        (di / cumo_amd.Int32.cast(hz)).to_numpy()


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_stacked_matrices_with_rows_of_an_odd_length_and_a_second_operand(tname, dt):
    """Three dimensions, the innermost not a whole number of vectors: a contiguous array (op) an operand
    that repeats along the first or the second dimension (or both), on either side, into a typed
    result and, for comparisons, into Bit."""
    import cumo_amd
    rng = np.random.default_rng(505)
    cls = cls_of(tname)
    for (O, M, Cn) in [(3, 37, 65), (7, 5, 1023), (2, 130, 259), (5, 3, 70001), (64, 2, 67)]:
        a = (rng.integers(-8, 8, size=(O, M, Cn)) / 4.0).astype(dt)
        da = cls.cast(a)
        for bshape in [(M, 1), (O, 1, Cn), (1, M, Cn), (O, 1, 1), (1, 1, Cn), (O, M, 1)]:
            b = (rng.integers(-8, 8, size=bshape) / 4.0).astype(dt)
            db = cls.cast(b)
            for name, f in (("add", lambda x, y: x + y), ("sub", lambda x, y: x - y)):
                assert_bits_equal(f(da, db).to_numpy(), oracle.binary(name, a, b), "%s %s %s" % ((O, M, Cn), name, bshape))
                assert_bits_equal(f(db, da).to_numpy(), oracle.binary(name, b, a), "%s %s %s (swapped)" % ((O, M, Cn), name, bshape))
            assert ((da > db).to_numpy() == (a > b)).all(), ((O, M, Cn), bshape)
            assert ((db >= da).to_numpy() == (b >= a)).all(), ((O, M, Cn), bshape)


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_transposed_operands_whose_extents_are_not_whole_vectors(tname, dt):
    """Transposed views go through LDS tiles with 128-bit accesses on both sides; neither extent need be
    a whole number of vectors, and rows need their element's alignment only: extents of 4k + 1, 2, 3,
    one and both inputs transposed, a transposed input beside a plain one and beside a scalar, a heavy
    function, stacked matrices, and Int32 with a division that meets a zero at the ragged edge."""
    import cumo_amd
    rng = np.random.default_rng(404)
    cls = cls_of(tname)
    for (R, Cn) in [(67, 131), (130, 4095), (4095, 130), (33, 65), (258, 1027), (5, 70), (1001, 9)]:
        a = rng.standard_normal((R, Cn)).astype(dt)
        b = rng.standard_normal((Cn, R)).astype(dt)
        c = rng.standard_normal((R, Cn)).astype(dt)
        da, db, dc = cls.cast(a), cls.cast(b), cls.cast(c)
        at = np.ascontiguousarray(a.T)
        assert_bits_equal((da.transpose() + 1.5).to_numpy(), oracle.binary("add", at, 1.5), ((R, Cn), "transposed + scalar"))
        assert_bits_equal((da.transpose() * db).to_numpy(), oracle.binary("mul", at, b), ((R, Cn), "transposed * plain"))
        assert_bits_equal((db - da.transpose()).to_numpy(), oracle.binary("sub", b, at), ((R, Cn), "plain - transposed"))
        assert_bits_equal((da.transpose() / dc.transpose()).to_numpy(), oracle.binary("div", at, np.ascontiguousarray(c.T)), ((R, Cn), "both transposed"))
        assert_bits_equal((-da.transpose()).to_numpy(), oracle.unary("minus", at), ((R, Cn), "unary"))
        assert_ulp(cumo_amd.NMath.exp(da.transpose()).to_numpy(), oracle.unary("exp", at), 1)
        assert_ulp((da.transpose().abs() ** 2.5).to_numpy(), oracle.binary("pow", np.abs(at), 2.5), 1 if dt == np.float32 else 2)
    s = rng.standard_normal((3, 37, 66)).astype(dt)
    assert_bits_equal((cls.cast(s).transpose(0, 2, 1) + 0.25).to_numpy(), oracle.binary("add", np.ascontiguousarray(s.transpose(0, 2, 1)), 0.25), "stacked")
    hi = rng.integers(-1000, 1000, size=(67, 131)).astype(np.int32)
    hz = rng.integers(1, 50, size=(131, 67)).astype(np.int32)
    di, dz = cumo_amd.Int32.cast(hi), cumo_amd.Int32.cast(hz)
    assert ((di.transpose() / dz).to_numpy() == oracle.binary("div", np.ascontiguousarray(hi.T), hz)).all()
    hz[130, 66] = 0
    with pytest.raises(ZeroDivisionError):
        di.transpose() / cumo_amd.Int32.cast(hz)


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_three_dimensions_with_an_operand_repeating_along_one(tname, dt):
    """[B,T,C] with [T,1], [B,1,C], [1,T,C], [B,1,1] and a column on both sides: the shapes whose two
    outer dimensions do not merge; C a whole number of 128-bit vectors and not; outer views."""
    rng = np.random.default_rng(202)
    cls = cls_of(tname)
    for (B, T, Cn) in [(6, 10, 64), (3, 7, 36), (2, 300, 8), (5, 4, 30)]:
        a = rng.standard_normal((B, T, Cn)).astype(dt)
        da = cls.cast(a)
        for shp in [(T, 1), (B, 1, Cn), (1, T, Cn), (B, 1, 1), (1, T, 1), (B, T, 1)]:
            b = rng.standard_normal(shp).astype(dt)
            db = cls.cast(b)
            assert_bits_equal((da + db).to_numpy(), oracle.binary("add", a, b), "%s + %s" % ((B, T, Cn), shp))
            assert_bits_equal((db / da).to_numpy(), oracle.binary("div", b, a), "%s / %s" % (shp, (B, T, Cn)))
        # both operands repeat, along different dimensions; a scalar rides along
        p_ = rng.standard_normal((B, 1, Cn)).astype(dt)
        q_ = rng.standard_normal((1, T, 1)).astype(dt)
        assert_bits_equal((cls.cast(p_) * cls.cast(q_)).to_numpy(), oracle.binary("mul", p_, q_))
        # views: every second outer slice, reversed middle dimension
        b = rng.standard_normal((T, 1)).astype(dt)
        assert_bits_equal((da[::2] - cls.cast(b)).to_numpy(), oracle.binary("sub", np.ascontiguousarray(a[::2]), b))
        assert_bits_equal((da[:, ::-1] - cls.cast(b)).to_numpy(), oracle.binary("sub", np.ascontiguousarray(a[:, ::-1]), b))
        # into a given result that is itself a view with padded rows
        out = cls.zeros(B, T, Cn + 4)
        out[:, :, :Cn].store(da * cls.cast(b))
        assert_bits_equal(out.to_numpy()[:, :, :Cn], oracle.binary("mul", a, b))
    import cumo_amd
    x = rng.integers(-100, 100, size=(4, 5, 8)).astype(np.int32)
    y = rng.integers(1, 9, size=(5, 1)).astype(np.int32)
    assert ((cumo_amd.Int32.cast(x) / cumo_amd.Int32.cast(y)).to_numpy() == oracle.binary("div", x, y)).all()
    y[2, 0] = 0
    with pytest.raises(ZeroDivisionError):
        cumo_amd.Int32.cast(x) / cumo_amd.Int32.cast(y)


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_rows_that_run_backwards_in_memory(tname, dt):
    """An input whose rows are reversed (x[true, (-1..0)], fliplr) is read by 128-bit vectors from the vector that ends
    at the lane's column, its elements turned round: one operand or both, against forward operands, a row vector, a
    scalar on either side, three dimensions, rows that are not a whole number of vectors (the general row kernel),
    windows that start inside a vector, a comparison into Bit."""
    rng = np.random.default_rng(104)
    cls = cls_of(tname)
    def rnd(*shape):
        return (rng.integers(-50, 50, size=shape) if dt == np.int32 else rng.standard_normal(shape)).astype(dt)
    for shape in [(70, 256), (33, 1000), (9, 520), (40, 1001), (5, 7, 64), (3, 20, 131)]:
        a, b = rnd(*shape), rnd(*shape)
        da, db = cls.cast(a), cls.cast(b)
        r = rnd(*((1,) * (len(shape) - 1) + (shape[-1],)))
        dr = cls.cast(r)
        rev = (Ellipsis, slice(None, None, -1))
        both = (slice(None, None, -1),) + (slice(None),) * (len(shape) - 2) + (slice(None, None, -1),)
        win = (Ellipsis, slice(shape[-1] - 3, 1, -1))
        with np.errstate(all="ignore"):
            assert_bits_equal((da[rev] + db).to_numpy(), oracle.binary("add", np.ascontiguousarray(a[rev]), b), "rev + fwd %r" % (shape,))
            assert_bits_equal((da - db[rev]).to_numpy(), oracle.binary("sub", a, np.ascontiguousarray(b[rev])), "fwd - rev %r" % (shape,))
            assert_bits_equal((da[rev] * db[rev]).to_numpy(), oracle.binary("mul", np.ascontiguousarray(a[rev]), np.ascontiguousarray(b[rev])), "rev * rev")
            assert_bits_equal((da[both] - db[rev]).to_numpy(), oracle.binary("sub", np.ascontiguousarray(a[both]), np.ascontiguousarray(b[rev])), "both - rev")
            assert_bits_equal((da[rev] + dr).to_numpy(), oracle.binary("add", np.ascontiguousarray(a[rev]), r), "rev + row vector")
            assert_bits_equal((da + dr[rev]).to_numpy(), oracle.binary("add", a, np.ascontiguousarray(r[rev])), "fwd + reversed row vector")
            assert_bits_equal((da[rev] + 3).to_numpy(), oracle.binary("add", np.ascontiguousarray(a[rev]), np.asarray(3, dtype=dt)), "rev + scalar")
            assert_bits_equal((7 - da[rev]).to_numpy(), oracle.binary("sub", np.asarray(7, dtype=dt), np.ascontiguousarray(a[rev])), "scalar - rev")
            assert_bits_equal((da[win] * db[win]).to_numpy(), oracle.binary("mul", np.ascontiguousarray(a[win]), np.ascontiguousarray(b[win])), "windows")
            assert_bits_equal(da[rev].copy().to_numpy(), np.ascontiguousarray(a[rev]), "copy of rev")
            assert ((da[rev] > db).to_numpy() == (a[rev] > b)).all(), "rev > fwd into Bit %r" % (shape,)
            assert (da[rev].gt(db[both]).to_numpy() == (a[rev] > b[both])).all() if hasattr(da, "gt") else True


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_inputs_that_start_off_a_16_byte_boundary(tname, dt):
    """Slices that begin at an odd column (rows and flat runs whose length is still a whole number of
    128-bit accesses): the lean kernels read them with 128-bit loads on 4- or 8-byte boundaries."""
    rng = np.random.default_rng(303)
    cls = cls_of(tname)
    mk = (lambda shp: rng.integers(-1000, 1000, size=shp).astype(dt)) if dt == np.int32 else (lambda shp: rng.standard_normal(shp).astype(dt))
    a, b = mk((37, 1030)), mk((37, 1030))
    da, db = cls.cast(a), cls.cast(b)
    for lo in (1, 2, 3, 5):
        for n in (1000, 1024, 8, 4):
            va, vb = a[:, lo:lo + n], b[:, lo + 1:lo + 1 + n]
            assert_bits_equal((da[:, lo:lo + n] * 2).to_numpy(), oracle.binary("mul", np.ascontiguousarray(va), 2), "scalar %d %d" % (lo, n))
            assert_bits_equal((da[:, lo:lo + n] + db[:, lo + 1:lo + 1 + n]).to_numpy(),
                              oracle.binary("add", np.ascontiguousarray(va), np.ascontiguousarray(vb)), "two views %d %d" % (lo, n))
            assert_bits_equal((da[:, lo:lo + n] - db[:, :n]).to_numpy(),
                              oracle.binary("sub", np.ascontiguousarray(va), np.ascontiguousarray(b[:, :n])), "one view %d %d" % (lo, n))
    # a flat run, a row vector and a column against it, rows in reverse
    f = mk(4099 * 3)
    df = cls.cast(f)
    for lo in (1, 3):
        assert_bits_equal((df[lo:lo + 12288] + df[lo + 2:lo + 2 + 12288]).to_numpy(), oracle.binary("add", f[lo:lo + 12288].copy(), f[lo + 2:lo + 2 + 12288].copy()))
    r, c = mk((1, 1030)), mk((37, 1))
    assert_bits_equal((da[:, 3:1003] + cls.cast(r)[:, 1:1001]).to_numpy(), oracle.binary("add", a[:, 3:1003].copy(), r[:, 1:1001].copy()))
    assert_bits_equal((da[:, 3:1003] * cls.cast(c)).to_numpy(), oracle.binary("mul", a[:, 3:1003].copy(), c))
    assert_bits_equal((da[::-1, 3:1003] - db[:, 2:1002]).to_numpy(), oracle.binary("sub", a[::-1, 3:1003].copy(), b[:, 2:1002].copy()))
    if dt != np.int32:
        import cumo_amd
        got = cumo_amd.NMath.exp(da[:, 1:1001]).to_numpy()
        assert_ulp(got, oracle.unary("exp", a[:, 1:1001].copy()), 1 if dt == np.float32 else 2)


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_many_dims_and_permuted_views(tname, dt):
    # past the reference's specialised accessors (ndim 5..8: test/narray_test.rb:41-51)
    rng = np.random.default_rng(102)
    cls = cls_of(tname)
    for nd in (5, 6, 8):
        shape = tuple(rng.integers(2, 4, size=nd))
        h = rng.standard_normal(shape).astype(dt)
        perm = tuple(rng.permutation(nd))
        d = cls.cast(h)
        got = (d.transpose(*perm) * 2.0 + d.transpose(*perm)).to_numpy()
        want = oracle.binary("add", oracle.binary("mul", h.transpose(perm), 2.0), h.transpose(perm))
        assert_bits_equal(got, want, "nd=%d" % nd)


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("n", [0, 1, 3, 31, 32, 33, 255, 256, 257, 1023, 4097, 100003])
def test_sizes_and_tails(tname, dt, n):
    rng = np.random.default_rng(103 + n)
    cls = cls_of(tname)
    hx = rng.standard_normal(n).astype(dt)
    hy = rng.standard_normal(n).astype(dt)
    got = (cls.cast(hx) * 2.5 + cls.cast(hy)).to_numpy()
    want = oracle.binary("add", oracle.binary("mul", hx, 2.5), hy) if n else np.zeros(0, dtype=dt)
    assert_bits_equal(got, want)
    # unaligned start: a view one element in
    if n > 4:
        got = (cls.cast(hx)[1:] + cls.cast(hy)[:-1]).to_numpy()
        assert_bits_equal(got, oracle.binary("add", hx[1:], hy[:-1]))


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_unary_and_rounding(tname, dt):
    rng = np.random.default_rng(104)
    cls = cls_of(tname)
    h = (rng.standard_normal((40, 50)) * 7).astype(dt)
    h[0, :6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 2.5]
    d = cls.cast(h)
    for view in ("contig", "transpose", "colslice"):
        hv, dv = views_of(view, h, d)
        for name in ["minus", "square", "sign", "floor", "round", "ceil", "trunc", "rint", "abs", "reciprocal"]:
            with np.errstate(all="ignore"):
                want = oracle.unary(name, hv)
            assert_bits_equal(getattr(dv, name)().to_numpy(), want, "%s %s" % (name, view))


MATH1 = ["sqrt", "cbrt", "log", "log2", "log10", "exp", "exp2", "exp10", "sin", "cos", "tan", "asin", "acos", "atan", "sinh",
         "cosh", "tanh", "asinh", "acosh", "atanh", "sinc", "erf", "erfc", "log1p", "expm1"]


def _math_domain(name, rng, dt):
    x = rng.standard_normal(20000).astype(dt) * 3
    if name in ("sqrt", "log", "log2", "log10"):
        x = np.abs(x) + dt(1e-3)
    elif name in ("asin", "acos", "atanh"):
        x = np.clip(x / 4, -0.99, 0.99).astype(dt)
    elif name == "acosh":
        x = np.abs(x) + dt(1)
    elif name == "log1p":
        x = np.abs(x)
    elif name in ("exp10",):
        x = x * 2
    return x


@pytest.mark.parametrize("tname,dt", FLOATS)
@pytest.mark.parametrize("name", MATH1)
def test_nmath(tname, dt, name):
    """Device against the oracle on random arguments, a consistency check beside
    test_gpu_nmath_vectors.py, which holds the device to 1 ulp of the correctly rounded value
    (and test_nmath_vectors.py, which measures the oracle against the same vectors).
    SFloat: evaluated in double and rounded once on both sides: within 1 ulp of each other.
    DFloat: the device is within 1 ulp of the true value and glibc within 1 (3 for cbrt, 2 for
    erfc), so the two are within the sum of each other."""
    import cumo_amd
    rng = np.random.default_rng(105)
    cls = cls_of(tname)
    x = _math_domain(name, rng, dt)
    got = getattr(cumo_amd.NMath, name)(cls.cast(x)).to_numpy()
    want = oracle.unary(name, x)
    # device bound + glibc's own bound, both measured against the correctly rounded vectors
    loose = {"cbrt": 1 + 3, "erfc": 1 + 2}
    assert_ulp(got, want, 1 if dt == np.float32 else loose.get(name, 2), "%s %s" % (tname, name))


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_nmath_two_args(tname, dt):
    import cumo_amd
    rng = np.random.default_rng(106)
    cls = cls_of(tname)
    x = rng.standard_normal((50, 40)).astype(dt)
    y = rng.standard_normal((50, 40)).astype(dt)
    # DFloat: device and glibc are each within 1 ulp of the correctly rounded value (the vector tests), so within 2 of each other
    for name in ("atan2", "hypot"):
        f = getattr(cumo_amd.NMath, name)
        assert_ulp(f(cls.cast(x), cls.cast(y)).to_numpy(), oracle.binary(name, x, y), 1 if dt == np.float32 else 2, name)
        assert_ulp(f(cls.cast(x), 0.5).to_numpy(), oracle.binary(name, x, 0.5), 1 if dt == np.float32 else 2, name)
        assert_ulp(f(0.5, cls.cast(x)).to_numpy(), oracle.binary(name, 0.5, x, scalar_is_left=True), 1 if dt == np.float32 else 2, name)
    assert_bits_equal(cls.cast(x).copysign(cls.cast(y)).to_numpy(), oracle.binary("copysign", x, y))


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_slices_whose_rows_are_not_whole_vectors(tname, dt):
    """Functions of slices that drop a column (rows of an odd length that start anywhere), their differences, a slice and
    a scalar, a slice and a row or column vector, three dimensions: the result is one run and every input is addressed
    by row and column, a 128-bit load wherever a result vector lies inside one row."""
    import cumo_amd
    rng = np.random.default_rng(109)
    cls = cls_of(tname)
    if dt == np.int32:
        h = rng.integers(-1000, 1000, size=(300, 260)).astype(dt)
        h3 = rng.integers(-1000, 1000, size=(6, 50, 131)).astype(dt)
    else:
        h = rng.standard_normal((300, 260)).astype(dt)
        h3 = rng.standard_normal((6, 50, 131)).astype(dt)
    d, d3 = cls.cast(h), cls.cast(h3)
    pairs = [(d[:, 1:], h[:, 1:]), (d[:, :-1], h[:, :-1]), (d[1:, 2:-1], h[1:, 2:-1]), (d[::2, 3:], h[::2, 3:]), (d[::-1, 1:], h[::-1, 1:]),
             (d3[:, :, 1:], h3[:, :, 1:]), (d3[1:, ::2, :-2], h3[1:, ::2, :-2])]
    for dv, hv in pairs:
        what = "%r" % (hv.shape,)
        assert_bits_equal((-dv).to_numpy(), oracle.unary("minus", hv), "minus " + what)
        assert_bits_equal(dv.abs().to_numpy(), oracle.unary("abs", hv), "abs " + what)
        assert_bits_equal((dv * 3).to_numpy(), oracle.binary("mul", hv, 3), "slice * scalar " + what)
        assert_bits_equal((7 - dv).to_numpy(), oracle.binary("sub", 7, hv, scalar_is_left=True), "scalar - slice " + what)
        assert_bits_equal(dv.copy().to_numpy(), hv, "copy " + what)
        if dt != np.int32:
            assert_ulp(cumo_amd.NMath.exp(dv).to_numpy(), oracle.unary("exp", hv), 1 if dt == np.float32 else 2, "exp " + what)
            assert_ulp(cumo_amd.NMath.erfc(dv).to_numpy(), oracle.unary("erfc", hv), 1 if dt == np.float32 else 3, "erfc " + what)
    # two slices of one array, a slice and a row vector, a slice and a column vector
    assert_bits_equal((d[:, 1:] - d[:, :-1]).to_numpy(), oracle.binary("sub", h[:, 1:], h[:, :-1]), "difference along rows")
    assert_bits_equal((d[1:, 1:] + d[:-1, :-1]).to_numpy(), oracle.binary("add", h[1:, 1:], h[:-1, :-1]), "diagonal neighbours")
    assert_bits_equal((d3[:, :, 1:] - d3[:, :, :-1]).to_numpy(), oracle.binary("sub", h3[:, :, 1:], h3[:, :, :-1]), "three dimensions")
    assert_bits_equal((d[:, 1:] + d[0:1, 1:]).to_numpy(), oracle.binary("add", h[:, 1:], h[0:1, 1:]), "slice + row vector")
    assert_bits_equal((d[:, 1:] * d[:, 0:1]).to_numpy(), oracle.binary("mul", h[:, 1:], h[:, 0:1]), "slice * column vector")
    # casts of slices: the result's vectors are whole, the input's elements of another width
    import cumo_amd
    for target, tdt in ((cumo_amd.DFloat, np.float64), (cumo_amd.SFloat, np.float32), (cumo_amd.Int32, np.int32)):
        if tdt == dt:
            continue
        src = h if dt == np.int32 or tdt != np.int32 else np.trunc(h * 10).astype(dt)
        dsrc = cls.cast(src)
        assert_bits_equal(target.cast(dsrc[:, 1:]).to_numpy(), src[:, 1:].astype(tdt), "cast of a slice to %s" % tdt.__name__)
        assert_bits_equal(target.cast(dsrc[::2, 2:-1]).to_numpy(), src[::2, 2:-1].astype(tdt), "cast of a slice to %s" % tdt.__name__)
    # comparisons into Bit: the bits are one run, every input is addressed
    v = (rng.integers(-3, 3, size=70001)).astype(dt)
    dv1 = cls.cast(v)
    for dx, hx, dy, hy, what in ((d[:, 1:], h[:, 1:], d[:, :-1], h[:, :-1], "two slices"), (dv1[1:], v[1:], dv1[:-1], v[:-1], "one dimension"),
                                 (d3[:, :, 1:], h3[:, :, 1:], d3[:, :, :-1], h3[:, :, :-1], "three dimensions"),
                                 (d[:, 1:], h[:, 1:], d[0:1, 1:], h[0:1, 1:], "slice against row vector")):
        assert_bits_equal((dx > dy).to_numpy(), (hx > hy).astype(np.uint8), "gt " + what)
        assert_bits_equal(dx.eq(dy).to_numpy(), (hx == hy).astype(np.uint8), "eq " + what)
        assert_bits_equal((dx <= dy).to_numpy(), (hx <= hy).astype(np.uint8), "le " + what)
        assert_bits_equal((dx > 0).to_numpy(), (hx > 0).astype(np.uint8), "gt scalar " + what)
        assert_bits_equal(dx.ne(1).to_numpy(), (hx != 1).astype(np.uint8), "ne scalar " + what)
    if dt != np.int32:
        hn = h.copy()
        hn[rng.random(h.shape) < 0.1] = np.nan
        assert_bits_equal(cls.cast(hn)[:, 1:].isnan().to_numpy(), np.isnan(hn[:, 1:]).astype(np.uint8), "isnan of a slice")
    if dt == np.int32:
        # a rejected element (division by zero) in a slice: the flag is raised, the other elements are stored
        z = h.copy()
        z[5, 7] = 0
        with pytest.raises(ZeroDivisionError):
            (d[:, 1:] / cls.cast(z)[:, 1:]).to_numpy()


def test_dfloat_power_of_arrays_with_every_kind_of_argument():
    """DFloat ** DFloat: positive normal bases with finite exponents take the library's own arithmetic (log2 of the base
    and its product with the exponent as pairs of doubles), every other argument the device library's pow. Both
    against the host's pow: within 2 ulp (each side is within 1 of the true value) and equal where the rules decide
    (signs, zeros, infinities, NaN, results beyond the range at either end)."""
    import cumo_amd
    rng = np.random.default_rng(108)
    n = 200000
    x = np.exp(rng.uniform(-700, 700, n))
    y = rng.uniform(-1, 1, n) * 1080.0 / np.abs(np.log2(x))            # results over the whole range and past both ends
    x[::5] = 1.0 + rng.uniform(-1, 1, x[::5].size) * np.exp2(rng.uniform(-50, -2, x[::5].size))
    y[::5] = rng.uniform(-1, 1, y[::5].size) * np.exp2(rng.uniform(0, 40, y[::5].size))
    x[1::5] = rng.uniform(0.01, 100, x[1::5].size)
    y[1::5] = rng.uniform(-20, 20, y[1::5].size)
    x[2::11] = -x[2::11]
    y[2::22] = np.round(y[2::22])                                        # negative bases with whole exponents
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 5e-324, 2.2250738585072014e-308, 1.7976931348623157e308, 0.5, 2.0, 3.0])
    x[3::101] = rng.choice(special, x[3::101].size)
    y[4::103] = rng.choice(special, y[4::103].size)
    y[5::107] = rng.choice(np.array([0.5, 2.0, 3.0, -1.0, 1.0, 0.0]), y[5::107].size)
    with np.errstate(all="ignore"):
        want = oracle.binary("pow", x, y)
    got = (cumo_amd.DFloat.cast(x) ** cumo_amd.DFloat.cast(y)).to_numpy()
    ruled = ~np.isfinite(want) | (want == 0) | ~np.isfinite(got) | (got == 0)
    # (a result that rounds to the largest double or to a subnormal next to zero may fall on either side of the end)
    edge = ruled & np.isfinite(x) & np.isfinite(y) & (x > 0) & (
        (np.abs(want) >= 1.7976931348623157e308) | (np.abs(got) >= 1.7976931348623157e308) | ((np.abs(want) <= 1e-323) & (np.abs(got) <= 1e-323)))
    strict = ruled & ~edge
    assert_bits_equal(got[strict], want[strict], "rule-decided results")
    assert_ulp(got[~ruled], want[~ruled], 2, "dfloat pow")
    # one exponent for the whole array, and one base
    for e in (2.5, -0.75, 1.0 / 3.0, 0.0, 7.0):
        with np.errstate(all="ignore"):
            want = oracle.binary("pow", x, e)
        got = (cumo_amd.DFloat.cast(x) ** e).to_numpy()
        ok = np.isfinite(want) & (want != 0) & np.isfinite(got) & (got != 0)
        assert_ulp(got[ok], want[ok], 2, "dfloat pow %r" % e)
        assert (np.isnan(got) == np.isnan(want)).all() and (np.isinf(got) == np.isinf(want))[~np.isnan(want) & (np.abs(want) < 1e308)].all()


def test_int32_arithmetic():
    rng = np.random.default_rng(107)
    cls = cls_of("int32")
    hx = rng.integers(-100000, 100000, size=(70, 90), dtype=np.int32)
    hy = rng.integers(1, 300, size=(70, 90), dtype=np.int32) * rng.choice(np.array([-1, 1], dtype=np.int32), size=(70, 90))
    dx, dy = cls.cast(hx), cls.cast(hy)
    for kind in ("contig", "transpose", "colslice", "reverse"):
        vx, wx = views_of(kind, hx, dx)
        vy, wy = views_of(kind, hy, dy)
        for op in ("add", "sub", "mul", "div", "mod"):
            assert_bits_equal(getattr(wx, PYOP[op])(wy).to_numpy(), oracle.binary(op, vx, vy), "%s %s" % (op, kind))
            assert_bits_equal(getattr(wx, PYOP[op])(7).to_numpy(), oracle.binary(op, vx, 7), "%s scalar" % op)
        assert_bits_equal((wx & wy).to_numpy(), oracle.binary("bit_and", vx, vy))
        assert_bits_equal((wx | wy).to_numpy(), oracle.binary("bit_or", vx, vy))
        assert_bits_equal((wx ^ wy).to_numpy(), oracle.binary("bit_xor", vx, vy))
        assert_bits_equal((~wx).to_numpy(), oracle.unary("bit_not", vx))
        assert_bits_equal((-wx).to_numpy(), oracle.unary("minus", vx))
        assert_bits_equal(wx.abs().to_numpy(), oracle.unary("abs", vx))
        assert_bits_equal(wx.square().to_numpy(), oracle.unary("square", vx))
        assert_bits_equal(wx.sign().to_numpy(), oracle.unary("sign", vx))
    sh = cls.cast((np.abs(hy) % 31).astype(np.int32))
    assert_bits_equal((dx >> sh).to_numpy(), oracle.binary("right_shift", hx, (np.abs(hy) % 31).astype(np.int32)))
    small = (np.abs(hx) % 1000).astype(np.int32)
    sh2 = (np.abs(hy) % 20).astype(np.int32)
    assert_bits_equal((cls.cast(small) << cls.cast(sh2)).to_numpy(), oracle.binary("left_shift", small, sh2))
    # scalar on the left of a non-commutative op
    assert_bits_equal((7000 - dx).to_numpy(), oracle.binary("sub", 7000, hx, scalar_is_left=True))
    assert_bits_equal((7000 / dy).to_numpy(), oracle.binary("div", 7000, hy, scalar_is_left=True))
    # Float on Int32 upcasts to DFloat (reference: gen/def/int32.rb:22-23)
    import cumo_amd
    r = dx * 0.5
    assert isinstance(r, cumo_amd.DFloat)
    assert_bits_equal(r.to_numpy(), hx.astype(np.float64) * 0.5)


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_float_remainder_with_every_kind_of_argument(tname, dt):
    """x % y of floats is the C fmod, exact: quotients small and beyond 2^29, whole-number quotients and their
    neighbours, subnormals, zeros of both signs on either side, infinities, NaN; arrays and one divisor."""
    import cumo_amd
    rng = np.random.default_rng(111)
    cls = cls_of(tname)
    n = 100000
    x = (rng.standard_normal(n) * np.exp2(rng.uniform(-20, 40, n))).astype(dt)
    y = (rng.standard_normal(n) * np.exp2(rng.uniform(-20, 10, n))).astype(dt)
    k = rng.integers(-1000, 1000, n)
    x[::3] = (y[::3].astype(np.float64) * k[::3]).astype(dt)                          # whole-number quotients (as far as the product is exact)
    x[1::7] = np.nextafter(x[1::7], dt(0))
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, np.finfo(dt).tiny / 4, np.finfo(dt).max, 1.5], dtype=dt)
    x[5::101] = rng.choice(special, x[5::101].size)
    y[7::103] = rng.choice(special, y[7::103].size)
    with np.errstate(all="ignore"):
        want = oracle.binary("mod", x, y)
    assert_bits_equal((cls.cast(x) % cls.cast(y)).to_numpy(), want, "array % array")
    for d in (1.0, 1.5, -0.75, 6.283185307179586, 1e-30, 3e38 if dt == np.float32 else 1e300):
        with np.errstate(all="ignore"):
            want = oracle.binary("mod", x, d)
        assert_bits_equal((cls.cast(x) % d).to_numpy(), want, "array %% %r" % d)


def test_int32_division_and_remainder_by_one_divisor():
    """array / d and array % d with one divisor for the whole launch go by multiplication and shift: every divisor
    kind (small, powers of two and their neighbours, the extremes, negative), dividends next to multiples and at the
    ends of the range; truncating, wrapping where C's would overflow; views; a zero divisor still raises."""
    import cumo_amd
    rng = np.random.default_rng(110)
    x = rng.integers(-2**31, 2**31, size=(257, 129), dtype=np.int64).astype(np.int32)
    x.flat[:6] = [0, 1, -1, 2**31 - 1, -2**31, -2**31 + 1]
    dx = cumo_amd.Int32.cast(x)
    for d in (1, -1, 2, -2, 3, 7, -7, 10, 255, 256, 257, 65536, 1000003, 2**30 - 1, 2**30, 2**30 + 1, 2**31 - 2, 2**31 - 1, -2**31, -2**31 + 1):
        near = (np.arange(-30, 30, dtype=np.int64)[:, None] * d + np.arange(-1, 2)[None, :]).reshape(-1)
        near = near[(near >= -2**31) & (near < 2**31)].astype(np.int32)
        for h, dv in ((x, dx), (near, cumo_amd.Int32.cast(near)), (x[::2, 1:], dx[::2, 1:]), (x.T, dx.transpose())):
            assert_bits_equal((dv / d).to_numpy(), oracle.binary("div", h, d), "div by %d" % d)
            assert_bits_equal((dv % d).to_numpy(), oracle.binary("mod", h, d), "mod by %d" % d)
    with pytest.raises(ZeroDivisionError):
        (dx / 0).to_numpy()
    with pytest.raises(ZeroDivisionError):
        (dx % 0).to_numpy()


def test_int32_error_flags():
    # reference: test/narray_test.rb:4887-4905 -- the flag raises, also through views,
    # and the rejected element is left alone
    cls = cls_of("int32")
    x = cls.cast(np.array([[6, 7, 8], [9, 10, 11]], dtype=np.int32))
    y = cls.cast(np.array([[2, 0, 4], [3, 5, 1]], dtype=np.int32))
    with pytest.raises(ZeroDivisionError):
        x / y
    with pytest.raises(ZeroDivisionError):
        x % y
    with pytest.raises(ZeroDivisionError):
        x.transpose() / y.transpose()
    with pytest.raises(ZeroDivisionError):
        x / 0
    assert (x / y[:, 2:]).to_numpy().tolist() == [[1, 1, 2], [9, 10, 11]]
    with pytest.raises(ValueError):
        cls.cast(np.array([1, -2**31], dtype=np.int32)).abs()
    with pytest.raises(ZeroDivisionError):
        cls.cast(np.array([1, 0], dtype=np.int32)).reciprocal()
    assert cls.cast(np.array([1, -1, 5], dtype=np.int32)).reciprocal().to_numpy().tolist() == [1, -1, 0]


@pytest.mark.parametrize("src,dst", [("sfloat", "dfloat"), ("dfloat", "sfloat"), ("int32", "sfloat"), ("int32", "dfloat"),
                                     ("sfloat", "int32"), ("dfloat", "int32"), ("sfloat", "sfloat"), ("int32", "int32")])
def test_casts_and_copies(src, dst):
    rng = np.random.default_rng(108)
    npdt = {"sfloat": np.float32, "dfloat": np.float64, "int32": np.int32}
    h = (rng.standard_normal((64, 48)) * 1000).astype(npdt[src])
    d = cls_of(src).cast(h)
    for kind in ("contig", "transpose", "colslice", "rowslice"):
        hv, dv = views_of(kind, h, d)
        assert_bits_equal(cls_of(dst).cast(dv).to_numpy(), oracle.store(npdt[dst], hv), "%s->%s %s" % (src, dst, kind))
        assert_bits_equal(dv.copy().to_numpy(), oracle.copy(hv))
    # mixed-type binary op upcasts (reference: gen/def/*.rb upcast tables)
    if src != dst:
        a, b = cls_of(src).cast(h), cls_of(dst).cast(h.astype(npdt[dst]))
        r = a + b
        rank = {"int32": 0, "sfloat": 1, "dfloat": 2}
        assert r.type_name == (src if rank[src] > rank[dst] else dst)


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_an_operand_that_is_an_array_of_one_element(tname, dt):
    """x - x.mean, x / x.sum, m - x, x.eq(x.max): an array of a single element (of no dimension or of size one) on either
    side of a contiguous array is read by the kernel as the scalar form's number is; the bits of the broadcast."""
    cls = cls_of(tname)
    rng = np.random.default_rng(641)
    for shape in [(1,), (5,), (4096,), (4099,), (37, 65), (3, 5, 128), ((1 << 20) + 3,), (1024, 4096)]:
        if dt == np.int32:
            hx = rng.integers(-1000, 1000, size=shape).astype(dt)
            hx[hx == 0] = 5
        else:
            hx = (rng.standard_normal(shape) * 8).astype(dt)
            hx[hx == 0] = 5
        x = cls.cast(hx)
        ones = [(x.max(), hx.max()), (cls.cast(np.array([3], dtype=dt)), dt(3)), (cls.cast(np.array([[-7]], dtype=dt)).reshape(*([1] * len(shape))), dt(-7))]
        for m, hm in ones:
            hmv = np.full(shape, hm, dtype=dt)
            for op in ("add", "sub", "mul", "div"):
                got = getattr(x, PYOP[op])(m)
                assert tuple(got.shape) == tuple(shape), (op, shape)
                assert_bits_equal(got.to_numpy(), oracle.binary(op, hx, hmv), (op, shape, "element on the right"))
                got = getattr(m, PYOP[op])(x)
                assert tuple(got.shape) == tuple(shape), (op, shape)
                assert_bits_equal(got.to_numpy(), oracle.binary(op, hmv, hx), (op, shape, "element on the left"))
            for op in ("eq", "gt", "le"):
                assert (getattr(x, op)(m).to_numpy() == oracle.compare(op, hx, hmv)).all(), (op, shape)
                assert (getattr(m, op)(x).to_numpy() == oracle.compare(op, hmv, hx)).all(), (op, shape, "left")
        if dt != np.int32:
            import cumo_amd
            m = cls.cast(np.array([2.5], dtype=dt))
            assert_ulp((x.abs() ** m).to_numpy(), oracle.binary("pow", np.abs(hx), np.full(shape, 2.5, dtype=dt)), 2)
            assert_bits_equal(cls.maximum(x, m).to_numpy(), np.maximum(hx, dt(2.5)))
    # views of the array keep their own paths and answer the same
    hx = (rng.integers(-50, 50, size=(130, 260))).astype(dt)
    hx[hx == 0] = 5
    x = cls.cast(hx)
    m = x.max()
    for dv, hv in ((x[:, 1:], hx[:, 1:]), (x.transpose(), hx.T), (x[::2, ::3], hx[::2, ::3])):
        hv = np.ascontiguousarray(hv)
        assert_bits_equal((dv - m).to_numpy(), oracle.binary("sub", hv, np.full(hv.shape, hx.max(), dtype=dt)))
        assert_bits_equal((m - dv).to_numpy(), oracle.binary("sub", np.full(hv.shape, hx.max(), dtype=dt), hv))
    if dt == np.int32:
        import cumo_amd
        with pytest.raises(ZeroDivisionError):
            x / cls.cast(np.array([0], dtype=dt))


MIXED_PAIRS = [("sfloat", "dfloat"), ("dfloat", "sfloat"), ("int32", "sfloat"), ("sfloat", "int32"), ("int32", "dfloat"), ("dfloat", "int32")]


@pytest.mark.parametrize("ta,tb", MIXED_PAIRS)
def test_arithmetic_on_two_element_types(ta, tb):
    """x op y for arrays of different types answers what casting both to the higher type and then running that type's
    operation answers, bit for bit (gen/tmpl/binary.c:38-97): two contiguous arrays of one shape go through one launch
    that converts on the way in; views, repeated operands and starts off a 16-byte boundary cast first."""
    npdt = {"sfloat": np.float32, "dfloat": np.float64, "int32": np.int32}
    rank = {"int32": 0, "sfloat": 1, "dfloat": 2}
    up = ta if rank[ta] > rank[tb] else tb
    rng = np.random.default_rng(613)

    def draw(t, shape):
        if t == "int32":
            v = rng.integers(-(1 << 30), 1 << 30, size=shape).astype(np.int32)   # beyond 2^24: the conversion to float rounds
            v[v == 0] = 7
            return v
        return ((rng.standard_normal(shape) + 3.0) * 10.0 ** rng.integers(-3, 4, size=shape)).astype(npdt[t])

    for shape in [(1,), (5,), (4096,), (4099,), (33, 65), (3, 5, 128), ((1 << 20) + 3,), (2048, 4096)]:
        hx, hy = draw(ta, shape), draw(tb, shape)
        x, y = cls_of(ta).cast(hx), cls_of(tb).cast(hy)
        ux, uy = hx.astype(npdt[up]), hy.astype(npdt[up])
        for op in ("add", "sub", "mul", "div"):
            r = getattr(x, PYOP[op])(y)
            assert r.type_name == up and tuple(r.shape) == tuple(shape)
            with np.errstate(all="ignore"):
                assert_bits_equal(r.to_numpy(), oracle.binary(op, ux, uy), (op, shape))
            # the same through the higher type's own operation on arrays cast beforehand
            assert_bits_equal(r.to_numpy(), getattr(cls_of(up).cast(x), PYOP[op])(cls_of(up).cast(y)).to_numpy(), (op, shape, "cast first"))
    # layouts that cast first: a start off a 16-byte boundary, a transposed operand, a repeated row, a strided slice
    hx, hy = draw(ta, (130, 260)), draw(tb, (130, 260))
    x, y = cls_of(ta).cast(hx), cls_of(tb).cast(hy)
    cases = [(x.reshape(130 * 260)[1:], y.reshape(130 * 260)[:-1], hx.reshape(-1)[1:], hy.reshape(-1)[:-1]),
             (x[:, 1:], y[:, :-1], hx[:, 1:], hy[:, :-1]),
             (x, y[:1, :], hx, hy[:1, :]),
             (x[::2], y[1::2], hx[::2], hy[1::2])]
    hs, ht = draw(ta, (260, 130)), None
    cases.append((cls_of(ta).cast(hs).transpose(), y, hs.T, hy))
    for dx, dy, ax, ay in cases:
        for op in ("add", "mul", "div"):
            with np.errstate(all="ignore"):
                want = oracle.binary(op, np.ascontiguousarray(ax).astype(npdt[up]), np.ascontiguousarray(np.broadcast_to(ay, ax.shape)).astype(npdt[up]))
            assert_bits_equal(getattr(dx, PYOP[op])(dy).to_numpy(), want, (op, ax.shape))


@pytest.mark.parametrize("ta,tb", MIXED_PAIRS)
def test_comparisons_of_two_element_types(ta, tb):
    """x cmp y for arrays of different types compares in the higher type (an Int32 beyond 2^24 is rounded to SFloat
    first, as the cast the reference makes rounds it): contiguous arrays in one launch, views through the cast."""
    npdt = {"sfloat": np.float32, "dfloat": np.float64, "int32": np.int32}
    rank = {"int32": 0, "sfloat": 1, "dfloat": 2}
    up = npdt[ta if rank[ta] > rank[tb] else tb]
    rng = np.random.default_rng(619)

    def draw(t, shape):
        if t == "int32":
            v = rng.integers(-4, 5, size=shape).astype(np.int32)
            big = rng.random(shape) < 0.1
            v[big] = 16777217 + rng.integers(-2, 3, size=shape)[big]     # around 2^24 + 1: not all representable in float
            return v
        v = rng.integers(-4, 5, size=shape).astype(npdt[t])
        big = rng.random(shape) < 0.1
        v[big] = np.asarray(16777217 + rng.integers(-2, 3, size=shape), dtype=npdt[t])[big]
        if shape != (1,):
            v.reshape(-1)[1] = np.nan
        return v

    for shape in [(1,), (31,), (128,), (129,), (1000,), (4096,), (37, 65), (3, 5, 96), ((1 << 20) + 77,), (2048, 4096)]:
        hx, hy = draw(ta, shape), draw(tb, shape)
        x, y = cls_of(ta).cast(hx), cls_of(tb).cast(hy)
        for op in ("eq", "ne", "gt", "ge", "lt", "le"):
            got = getattr(x, op)(y)
            assert tuple(got.shape) == tuple(shape)
            with np.errstate(all="ignore"):
                want = oracle.compare(op, hx.astype(up), hy.astype(up))
            assert (got.to_numpy() == want).all(), (op, shape)
    hx, hy = draw(ta, (130, 260)), draw(tb, (130, 260))
    x, y = cls_of(ta).cast(hx), cls_of(tb).cast(hy)
    for dx, dy, ax, ay in ((x[:, 1:], y[:, :-1], hx[:, 1:], hy[:, :-1]), (x, y[:1, :], hx, hy[:1, :]), (x.transpose(), y.transpose(), hx.T, hy.T)):
        for op in ("eq", "gt", "le"):
            want = oracle.compare(op, np.ascontiguousarray(ax).astype(up), np.ascontiguousarray(np.broadcast_to(ay, ax.shape)).astype(up))
            assert (getattr(dx, op)(dy).to_numpy() == want).all(), (op, ax.shape)


def test_int32_array_with_a_float_number_answers_dfloat():
    """An Int32 array meeting a Ruby Float is computed in DFloat (gen/def/int32.rb:22-23): the bits of casting the array
    first and running DFloat's scalar form, for contiguous arrays (one launch) and for views (cast first)."""
    import cumo_amd
    rng = np.random.default_rng(617)
    for shape in [(1,), (7,), (4096,), (4101,), (33, 65), ((1 << 20) + 1,), (2048, 2048)]:
        h = rng.integers(-(1 << 31), 1 << 31, size=shape).astype(np.int32)
        h[h == 0] = 3
        d = cumo_amd.Int32.cast(h)
        hd = h.astype(np.float64)
        for op in ("add", "sub", "mul", "div"):
            for sv in (2.5, -1.0 / 3.0):
                r = getattr(d, PYOP[op])(sv)
                assert isinstance(r, cumo_amd.DFloat) and tuple(r.shape) == tuple(shape)
                assert_bits_equal(r.to_numpy(), oracle.binary(op, hd, sv), (op, shape, sv))
                r = getattr(d, RPYOP[op])(sv)
                assert isinstance(r, cumo_amd.DFloat)
                assert_bits_equal(r.to_numpy(), oracle.binary(op, sv, hd, scalar_is_left=True), (op, shape, sv, "number on the left"))
    h = rng.integers(-1000, 1000, size=(130, 260)).astype(np.int32)
    h[h == 0] = 3
    d = cumo_amd.Int32.cast(h)
    for dv, hv in ((d[:, 1:], h[:, 1:]), (d.transpose(), h.T), (d[::2, ::3], h[::2, ::3]), (d.reshape(130 * 260)[1:], h.reshape(-1)[1:])):
        hd = np.ascontiguousarray(hv).astype(np.float64)
        assert_bits_equal((dv * 0.3).to_numpy(), oracle.binary("mul", hd, 0.3))
        assert_bits_equal((2.5 / dv).to_numpy(), oracle.binary("div", 2.5, hd, scalar_is_left=True))
    # an integer number keeps the array Int32; other operations with a Float still answer DFloat
    assert isinstance(d * 3, cumo_amd.Int32)
    assert isinstance(d % 2.5, cumo_amd.DFloat)
    assert_bits_equal((d % 2.5).to_numpy(), oracle.binary("mod", h.astype(np.float64), 2.5))


def test_fill_and_store_into_views():
    cls = cls_of("sfloat")
    a = cls.zeros(6, 8)
    a[::2, 1::3].fill(7.5)
    want = np.zeros((6, 8), dtype=np.float32)
    want[::2, 1::3] = 7.5
    assert_bits_equal(a.to_numpy(), want)
    b = cls_of("dfloat").cast(np.arange(8, dtype=np.float64))
    a[1].store(b)
    want[1] = np.arange(8)
    assert_bits_equal(a.to_numpy(), want)
    i = cls_of("int32").zeros(5).fill(-3)
    assert i.to_numpy().tolist() == [-3] * 5


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
@pytest.mark.parametrize("op", ["eq", "ne", "gt", "ge", "lt", "le"])
def test_compare_into_bit(tname, dt, op):
    rng = np.random.default_rng(109)
    cls = cls_of(tname)
    # (from 64 columns on, matrix (op) row / column / view goes flat over the matrix and the bits, the other
    # operand addressed by row and column: row lengths that are and are not whole vectors, totals that end
    # inside a group of 128 bits)
    for shape in [(1,), (31,), (32,), (33,), (64,), (1000,), (5, 67), (7, 64), (3, 5, 96), (129, 33), (37, 65), (130, 4095), (64, 128),
                  (9, 1001), (33, 256)]:
        hx = rng.integers(-3, 4, size=shape).astype(dt)
        hy = rng.integers(-3, 4, size=shape).astype(dt)
        if dt != np.int32:
            hx.reshape(-1)[0] = np.nan
        dx, dy = cls.cast(hx), cls.cast(hy)
        assert (getattr(dx, op)(dy).to_numpy() == oracle.compare(op, hx, hy)).all(), (shape, op)
        assert (getattr(dx, op)(1).to_numpy() == oracle.compare(op, hx, 1)).all(), (shape, op, "scalar")
        if len(shape) == 2:
            assert (getattr(dx.transpose(), op)(dy.transpose()).to_numpy() == oracle.compare(op, hx.T, hy.T)).all(), (shape, op, "T")
            assert (getattr(dx[:, ::2], op)(0).to_numpy() == oracle.compare(op, hx[:, ::2], 0)).all()
            assert (getattr(dx, op)(dy[0]).to_numpy() == oracle.compare(op, hx, hy[0])).all(), (shape, op, "bcast")
            assert (getattr(dy[0], op)(dx).to_numpy() == oracle.compare(op, hy[0], hx)).all(), (shape, op, "row on the left")
            col, hcol = dy[:, :1], hy[:, :1]
            assert (getattr(dx, op)(col).to_numpy() == oracle.compare(op, hx, hcol)).all(), (shape, op, "column")
            assert (getattr(col, op)(dx).to_numpy() == oracle.compare(op, hcol, hx)).all(), (shape, op, "column on the left")
            wide = cls.cast(np.repeat(hy, 2, axis=1))
            assert (getattr(dx, op)(wide[:, ::2]).to_numpy() == oracle.compare(op, hx, hy)).all(), (shape, op, "view")


@pytest.mark.parametrize("tname,dt", FLOATS + [("int32", np.int32)])
def test_compare_of_transposed_views_into_bit(tname, dt):
    """A comparison whose input walks another dimension fastest than the result's bits do is copied into the result's
    order first (from 65536 elements on): one or both operands transposed, against a scalar, a row that repeats, three
    dimensions permuted two ways, a NaN among the values."""
    rng = np.random.default_rng(111)
    cls = cls_of(tname)
    hx = rng.integers(-3, 4, size=(300, 420)).astype(dt)
    hy = rng.integers(-3, 4, size=(420, 300)).astype(dt)
    if dt != np.int32:
        hx[5, 7] = np.nan
    dx, dy = cls.cast(hx), cls.cast(hy)
    for op in ("gt", "eq", "le"):
        assert (getattr(dx.transpose(), op)(dy).to_numpy() == oracle.compare(op, hx.T, hy)).all(), op
        assert (getattr(dy, op)(dx.transpose()).to_numpy() == oracle.compare(op, hy, hx.T)).all(), op
        assert (getattr(dx.transpose(), op)(0).to_numpy() == oracle.compare(op, hx.T, 0)).all(), op
        assert (getattr(dx.transpose(), op)(dy[0]).to_numpy() == oracle.compare(op, hx.T, hy[0])).all(), op
        assert (getattr(dx.transpose()[::2, 1:], op)(dy[::2, 1:]).to_numpy() == oracle.compare(op, hx.T[::2, 1:], hy[::2, 1:])).all(), op
    ht = rng.integers(-3, 4, size=(20, 70, 64)).astype(dt)
    dtn = cls.cast(ht)
    for perm in ((0, 2, 1), (2, 1, 0), (1, 2, 0)):
        assert (dtn.transpose(*perm).gt(1).to_numpy() == oracle.compare("gt", ht.transpose(perm), 1)).all(), perm


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_float_classification(tname, dt):
    cls = cls_of(tname)
    rng = np.random.default_rng(110)
    h = rng.standard_normal(5000).astype(dt)
    h[::7] = np.nan
    h[1::11] = np.inf
    h[2::13] = -np.inf
    h[3::17] = -0.0
    d = cls.cast(h)
    for name in ("isnan", "isinf", "isposinf", "isneginf", "isfinite", "signbit"):
        assert (getattr(d, name)().to_numpy() == oracle.cond_unary(name, h)).all(), name
        assert (getattr(d[5::3], name)().to_numpy() == oracle.cond_unary(name, h[5::3])).all(), name
    x = np.array([1.0, 1.0 + 1e-7, 1.001, 0.0], dtype=dt)
    y = np.array([1.0, 1.0, 1.0, 0.0], dtype=dt)
    assert (cls.cast(x).nearly_eq(cls.cast(y)).to_numpy() == oracle.compare("nearly_eq", x, y)).all()
