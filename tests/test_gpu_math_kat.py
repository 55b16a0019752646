"""The device against the literal cases of the reference's test/math_test.rb (tests/kat_math.py),
at the reference's own bar, and NMath.ldexp / frexp against the CPU oracle bit for bit."""
import os
import sys

import numpy as np
import pytest

import kat_math

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import numo_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu

TYPES = [("SFloat", np.float32), ("DFloat", np.float64)]


@pytest.mark.parametrize("cls,dt", TYPES)
@pytest.mark.parametrize("case", kat_math.CLOSE, ids=[c[0] for c in kat_math.CLOSE])
def test_one_argument_functions(case, cls, dt):
    import cumo_amd
    fn, args, want, _ = case
    got = getattr(cumo_amd.NMath, fn)(getattr(cumo_amd, cls).cast(np.array(args, dtype=dt)))
    assert isinstance(got, getattr(cumo_amd, cls))
    assert kat_math.close(want, got.to_numpy())


@pytest.mark.parametrize("cls,dt", TYPES)
def test_two_argument_functions_ldexp_and_frexp(cls, dt):
    import cumo_amd
    T = getattr(cumo_amd, cls)
    for fn, a, b, want, _ in kat_math.EQUAL2:
        got = getattr(cumo_amd.NMath, fn)(T.cast(np.array(a, dtype=dt)), T.cast(np.array(b, dtype=dt)))
        assert isinstance(got, T) and (got.to_numpy() == np.array(want, dtype=dt)).all(), fn
    a, b, want = kat_math.LDEXP
    got = cumo_amd.NMath.ldexp(T.cast(np.array(a, dtype=dt)), cumo_amd.Int32.cast(np.array(b, dtype=np.int32)))
    assert isinstance(got, T) and (got.to_numpy() == np.array(want, dtype=dt)).all()
    a, mant, expo = kat_math.FREXP
    m, e = cumo_amd.NMath.frexp(T.cast(np.array(a, dtype=dt)))
    assert isinstance(m, T) and isinstance(e, cumo_amd.Int32)
    assert (m.to_numpy() == np.array(mant, dtype=dt)).all() and (e.to_numpy() == np.array(expo)).all()


@pytest.mark.parametrize("cls,dt", TYPES)
def test_ldexp_and_frexp_bit_for_bit_with_the_oracle(cls, dt):
    """Both are exact operations (a scaling by a power of two rounded once, a split of the
    representation), so the device must give the C library's bits: over every binade,
    subnormals, zeros, through views, and with the scalar forms."""
    import cumo_amd
    T = getattr(cumo_amd, cls)
    rng = np.random.default_rng(7)
    tiny = np.finfo(dt).tiny
    x = np.concatenate([rng.standard_normal(5000) * 10.0 ** rng.integers(-30, 30, 5000),
                        rng.random(500) * tiny, [0.0, -0.0, 1.0, -1.0, tiny, np.finfo(dt).max, -np.finfo(dt).max]]).astype(dt)
    m, e = cumo_amd.NMath.frexp(T.cast(x))
    wm, we = oracle.frexp(x)
    assert (m.to_numpy().view(np.uint8) == wm.view(np.uint8)).all() and (e.to_numpy() == we).all()
    # x = mantissa * 2**exponent comes back exactly
    back = cumo_amd.NMath.ldexp(m, e)
    assert (back.to_numpy().view(np.uint8) == x.view(np.uint8)).all()
    # the special values (the exponent of an infinity or a NaN is unspecified in C: the mantissa is checked)
    sp = np.array([np.inf, -np.inf, np.nan], dtype=dt)
    ms, _ = cumo_amd.NMath.frexp(T.cast(sp))
    assert (np.isinf(ms.to_numpy()[:2])).all() and np.isnan(ms.to_numpy()[2])
    n = rng.integers(-200 if dt == np.float32 else -1200, 200 if dt == np.float32 else 1200, x.size).astype(np.int32)
    got = cumo_amd.NMath.ldexp(T.cast(x), cumo_amd.Int32.cast(n)).to_numpy()
    with np.errstate(all="ignore"):
        want = oracle.binary("ldexp", x, n.astype(dt))
    assert (got.view(np.uint8) == want.view(np.uint8)).all()
    # a 2-D strided view against a row of exponents, and the scalar forms
    h = x[:4800].reshape(60, 80)
    d = T.cast(h)
    nn = np.arange(-3, 37, dtype=np.int32)
    got = cumo_amd.NMath.ldexp(d[::2, ::2], cumo_amd.Int32.cast(nn)).to_numpy()
    with np.errstate(all="ignore"):
        assert (got == oracle.binary("ldexp", np.ascontiguousarray(h[::2, ::2]), np.broadcast_to(nn.astype(dt), (30, 40)).copy())).all()
        assert (cumo_amd.NMath.ldexp(d, 3).to_numpy() == h * dt(8)).all()
        assert (cumo_amd.NMath.ldexp(2.0, cumo_amd.Int32.cast(nn)).to_numpy() == np.ldexp(2.0, nn)).all()
    mv, ev = cumo_amd.NMath.frexp(d.transpose()[1::3])
    wm, we = oracle.frexp(np.ascontiguousarray(h.T[1::3]))
    assert (mv.to_numpy() == wm).all() and (ev.to_numpy() == we).all()
    # an Int32 argument is computed in DFloat
    mi, ei = cumo_amd.NMath.frexp(cumo_amd.Int32.cast(np.array([0, 1, 5, -12], dtype=np.int32)))
    assert isinstance(mi, cumo_amd.DFloat) and (mi.to_numpy() == [0.0, 0.5, 0.625, -0.75]).all() and (ei.to_numpy() == [0, 1, 3, 4]).all()


@pytest.mark.parametrize("cls,dt", TYPES + [("Int32", np.int32)])
def test_seq_logseq_and_eye(cls, dt):
    """The reference's literal cases (narray_alt_coverage_test.rb:263-272), then the oracle on
    strided views, many dimensions and the error cases of eye."""
    import cumo_amd
    T = getattr(cumo_amd, cls)
    for args, want in kat_math.SEQ:
        assert (T.new(5).seq(*args).to_numpy() == np.array(want, dtype=dt)).all()
    rng = np.random.default_rng(3)
    for shape in [(1,), (1000003,), (7, 11), (3, 1, 5, 4), (2, 3, 2, 2, 3)]:
        beg, step = (float(rng.integers(-9, 9)), float(rng.integers(-4, 5))) if dt == np.int32 else (rng.standard_normal(), rng.standard_normal())
        assert (T.new(*shape).seq(beg, step).to_numpy().view(np.uint8) == oracle.seq(shape, dt, beg, step).view(np.uint8)).all(), shape
    # through a view: the element number runs over the view in row-major order, the rest stays
    h = np.full((6, 8), 9, dtype=dt)
    d = T.cast(h)
    d[1::2, ::3].seq(1, 2)
    h[1::2, ::3] = oracle.seq((3, 3), dt, 1, 2)
    d.transpose()[:2].seq(100)
    h.T[:2] = oracle.seq((2, 6), dt, 100)
    assert (d.to_numpy() == h).all()
    if dt == np.int32:
        assert (T.new(4).seq(-1.5, 0.75).to_numpy() == [-1, 0, 0, 0]).all()
        with pytest.raises(Exception):
            T.new(3).logseq(0, 1)
    else:
        for n, args, want in kat_math.LOGSEQ:
            assert (T.new(n).logseq(*args).to_numpy() == np.array(want, dtype=dt)).all()
        got = T.new(4, 25).logseq(-3, 0.11, 2.5).to_numpy()
        want = oracle.logseq((4, 25), dt, -3, 0.11, 2.5)
        from helpers import assert_ulp
        # DFloat: device and glibc each within 1 ulp of the correctly rounded value (test_gpu_nmath_vectors.py, test_nmath_vectors.py)
        assert_ulp(got, want, 1 if dt == np.float32 else 2)
        v = T.zeros(5, 12)
        v[:, ::2].logseq(0, 1, 2)
        assert_ulp(np.ascontiguousarray(v.to_numpy()[:, ::2]), oracle.logseq((5, 6), dt, 0, 1, 2), 0 if dt == np.float32 else 2)
        assert (v.to_numpy()[:, 1::2] == 0).all()
    for shape, el, k in [((3, 4), 1, 0), ((4, 4), 2.0, 1), ((2, 3, 5), 7, -2), ((2, 2, 3, 3), 1, 2)]:
        assert (T.new(*shape).eye(el, k).to_numpy() == oracle.eye(shape, dt, el, k)).all()
    e = T.cast(np.full((5, 7), 3, dtype=dt))
    e[1:4, 2:6].eye()
    want = np.full((5, 7), 3, dtype=dt)
    want[1:4, 2:6] = np.eye(3, 4)
    assert (e.to_numpy() == want).all()
    with pytest.raises(Exception):
        T.new(5).eye()
    with pytest.raises(Exception):
        T.new(3, 3).eye(1, 3)
    with pytest.raises(Exception):
        T.new(3, 3).eye(1, -3)


def test_divmod_and_modf_reference_cases():
    """narray_test.rb:1413-1420, 2248-2252, 2472-2511 (modf keeps the argument's sign in both parts,
    zero included; NaN gives NaN twice; an infinity gives a signed zero and itself) and
    narray_alt_coverage_test.rb:719,741 (Int32 divmod, and by zero)."""
    import cumo_amd
    q, r = cumo_amd.Int32.cast(np.array([17, 20, 23], np.int32)).divmod(cumo_amd.Int32.cast(np.array([5, 6, 7], np.int32)))
    assert (q.to_numpy() == [3, 3, 3]).all() and (r.to_numpy() == [2, 2, 2]).all()
    q, r = cumo_amd.Int32.cast(np.array([10, 20, 30], np.int32)).divmod(cumo_amd.Int32.cast(np.array([3, 4, 5], np.int32)))
    assert (q.to_numpy() == [3, 5, 6]).all() and (r.to_numpy() == [1, 0, 0]).all()
    with pytest.raises(ZeroDivisionError):
        cumo_amd.Int32.cast(np.array([1, 2, 3], np.int32)).divmod(cumo_amd.Int32.cast(np.array([1, 0, 3], np.int32)))
    with pytest.raises(ZeroDivisionError):
        cumo_amd.Int32.cast(np.arange(12, dtype=np.int32).reshape(3, 4))[:, 1:-1].divmod(0)
    f, w = (cumo_amd.DFloat.new(8).seq(1) / 4).modf()
    assert (f.to_numpy()[:2] == [0.25, 0.5]).all() and (w.to_numpy()[:2] == [0.0, 0.0]).all()
    inf = np.inf
    specials = {0: np.nan, 1: inf, 2: -inf, 3: -0.0}
    values = np.array([specials.get(i % 9, (i - 100) / 8.0) for i in range(200)])
    for cls, dt in TYPES:
        T = getattr(cumo_amd, cls)
        stored = values.astype(dt)
        a = T.cast(stored)
        for view, src in ((a, stored), (a[::3], stored[::3]), (a[::-1], stored[::-1])):
            f, w = view.modf()
            wf, ww = oracle.modf(np.ascontiguousarray(src))
            assert isinstance(f, T) and isinstance(w, T)
            assert (f.to_numpy().view(np.uint8) == wf.view(np.uint8))[~np.isnan(wf).repeat(wf.itemsize)].all()
            assert (np.isnan(f.to_numpy()) == np.isnan(wf)).all() and (np.isnan(w.to_numpy()) == np.isnan(ww)).all()
            assert (w.to_numpy().view(np.uint8) == ww.view(np.uint8))[~np.isnan(ww).repeat(ww.itemsize)].all()
            m, e = cumo_amd.NMath.frexp(view)
            wm, we = oracle.frexp(np.ascontiguousarray(src))
            fin = np.isfinite(src)
            assert (m.to_numpy()[fin].view(np.uint8) == wm[fin].view(np.uint8)).all() and (e.to_numpy()[fin] == we[fin]).all()
        # float divmod: the quotient is the plain division, the remainder fmod; broadcast and a number
        rng = np.random.default_rng(5)
        x = rng.standard_normal((6, 40)).astype(dt) * 50
        y = (rng.standard_normal(40).astype(dt) * 7)
        q, r = T.cast(x).divmod(T.cast(y))
        wq, wr = oracle.divmod_(x, np.broadcast_to(y, x.shape).copy())
        assert (q.to_numpy() == wq).all() and (r.to_numpy() == wr).all()
        q, r = T.cast(x)[::2, 1::2].divmod(4.0)
        wq, wr = oracle.divmod_(np.ascontiguousarray(x[::2, 1::2]), np.full((3, 20), 4.0, dtype=dt))
        assert (q.to_numpy() == wq).all() and (r.to_numpy() == wr).all()


def test_empty_and_single_element_arrays():
    """total_size == 0 is a no-op without a launch (template_kernel.h:76-81); one element works."""
    import cumo_amd
    for cls, dt in TYPES + [("Int32", np.int32)]:
        T = getattr(cumo_amd, cls)
        e = T.new(0)
        assert e.seq().shape == (0,) and T.new(0, 3).eye().shape == (0, 3)
        q, r = e.divmod(T.new(0))
        assert q.shape == (0,) and r.shape == (0,)
        assert (T.new(1).seq(7).to_numpy() == [7]).all()
        q, r = T.cast(np.array([7], dtype=dt)).divmod(2)
        assert q.to_numpy()[0] == (3 if dt == np.int32 else 3.5) and r.to_numpy()[0] == 1
        if dt != np.int32:
            f, w = e.modf()
            m, x = cumo_amd.NMath.frexp(e)
            assert f.shape == w.shape == m.shape == x.shape == (0,)
            assert e.logseq(0, 1).shape == (0,)
            assert cumo_amd.NMath.ldexp(e, cumo_amd.Int32.new(0)).shape == (0,)


@pytest.mark.parametrize("cls,dt", TYPES + [("Int32", np.int32)])
def test_poly(cls, dt):
    """The reference's cases (narray_test.rb:1944-1963), then the oracle bit for bit: number
    coefficients (one launch, more than six coefficients continue from the result), array
    coefficients with broadcasting (the chain of array operations), views, the constant alone."""
    import cumo_amd
    T = getattr(cumo_amd, cls)
    x = T.new(4).seq(1)
    assert (x.poly(1, 2).to_numpy() == [3, 5, 7, 9]).all()
    assert (x.poly(1, 2, 3).to_numpy() == [6, 17, 34, 57]).all()
    assert (x.poly(3).to_numpy() == [3, 3, 3, 3]).all() and (x.poly().to_numpy() == [1, 2, 3, 4]).all()
    assert (T.cast(np.array([2], dtype=dt)).poly(1, 2).to_numpy() == [5]).all()
    assert (x.poly(T.cast(np.ones(4, dtype=dt)), T.cast(np.full(4, 2, dtype=dt))).to_numpy() == [3, 5, 7, 9]).all()
    rng = np.random.default_rng(11)
    if dt == np.int32:
        h = rng.integers(-50000, 50000, size=(37, 53)).astype(dt)
        coefs = [int(c) for c in rng.integers(-9, 9, size=15)]
    else:
        h = rng.standard_normal((37, 53)).astype(dt)
        coefs = [float(c) for c in rng.standard_normal(15)]
    d = T.cast(h)
    for n in (1, 2, 6, 7, 12, 13, 15):
        got = d.poly(*coefs[:n]).to_numpy()
        assert (got.view(np.uint8) == oracle.poly(h, *coefs[:n]).view(np.uint8)).all(), n
    got = d.transpose()[1::2, ::3].poly(*coefs[:8]).to_numpy()
    assert (got == oracle.poly(np.ascontiguousarray(h.T[1::2, ::3]), *coefs[:8])).all()
    # one run that starts off a 16-byte boundary and ends in part of a vector
    flat = T.cast(h.reshape(-1))
    for lo, hi in ((5, None), (1, -2), (3, 1030)):
        got = flat[lo:hi].poly(*coefs[:9]).to_numpy()
        assert (got.view(np.uint8) == oracle.poly(np.ascontiguousarray(h.reshape(-1)[lo:hi]), *coefs[:9]).view(np.uint8)).all(), (lo, hi)
    row = (rng.integers(-5, 5, size=53) if dt == np.int32 else rng.standard_normal(53)).astype(dt)
    col = (rng.integers(-5, 5, size=(37, 1)) if dt == np.int32 else rng.standard_normal((37, 1))).astype(dt)
    for cs in ((row,), (row, col), (coefs[0], row, col, coefs[1]), (col, coefs[2], row)):
        got = d.poly(*[T.cast(c) if isinstance(c, np.ndarray) else c for c in cs]).to_numpy()
        assert (got.view(np.uint8) == oracle.poly(h, *cs).view(np.uint8)).all()
    small = T.cast(h[:1])                      # [1, 53] against a column: the constant alone spreads over both
    assert (small.poly(T.cast(col)).to_numpy() == np.broadcast_to(col, (37, 53))).all()


def test_two_result_operations_over_whole_runs():
    """modf, frexp and divmod where every operand is one contiguous run (128-bit vectors per lane, from
    any element boundary, lengths that end in part of a vector) against the oracle bit for bit; an
    Int32 division that meets a zero somewhere inside raises."""
    import cumo_amd
    rng = np.random.default_rng(77)
    for cls, dt in TYPES:
        T = getattr(cumo_amd, cls)
        for shape in [(37, 53), (5000,), (3, 7, 101)]:
            x = (rng.standard_normal(shape) * 50).astype(dt)
            y = (rng.standard_normal(shape) * 7).astype(dt)
            x.reshape(-1)[::97] = np.inf
            x.reshape(-1)[5::89] = -0.0
            f, w = T.cast(x).modf()
            wf, ww = oracle.modf(x)
            assert (f.to_numpy().view(np.uint8) == wf.view(np.uint8)).all() and (w.to_numpy().view(np.uint8) == ww.view(np.uint8)).all(), shape
            fin = np.isfinite(x)
            m, e = cumo_amd.NMath.frexp(T.cast(x))
            wm, we = oracle.frexp(x)
            assert (m.to_numpy()[fin].view(np.uint8) == wm[fin].view(np.uint8)).all() and (e.to_numpy()[fin] == we[fin]).all(), shape
            xf = np.where(fin, x, 1.0).astype(dt)
            q, r = T.cast(xf).divmod(T.cast(y))
            wq, wr = oracle.divmod_(xf, y)
            assert (q.to_numpy().view(np.uint8) == wq.view(np.uint8)).all() and (r.to_numpy().view(np.uint8) == wr.view(np.uint8)).all(), shape
        flat = (rng.standard_normal(3000) * 9).astype(dt)
        d = T.cast(flat)
        for lo, hi in ((1, None), (3, -2), (5, 1500)):
            f, w = d[lo:hi].modf()
            wf, ww = oracle.modf(np.ascontiguousarray(flat[lo:hi]))
            assert (f.to_numpy().view(np.uint8) == wf.view(np.uint8)).all() and (w.to_numpy().view(np.uint8) == ww.view(np.uint8)).all(), (lo, hi)
    a = rng.integers(-10 ** 6, 10 ** 6, size=(41, 67)).astype(np.int32)
    b = rng.integers(1, 500, size=(41, 67)).astype(np.int32) * rng.choice([-1, 1], size=(41, 67)).astype(np.int32)
    a[3, 5] = -2 ** 31
    b[3, 5] = -1
    q, r = cumo_amd.Int32.cast(a).divmod(cumo_amd.Int32.cast(b))
    wq, wr = oracle.divmod_(a, b)
    assert (q.to_numpy() == wq).all() and (r.to_numpy() == wr).all()
    b[20, 33] = 0
    with pytest.raises(ZeroDivisionError):
        cumo_amd.Int32.cast(a).divmod(cumo_amd.Int32.cast(b))
