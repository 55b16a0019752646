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
