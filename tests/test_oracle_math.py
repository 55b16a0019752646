"""The oracle against the literal cases of the reference's test/math_test.rb (CPU only)."""
import os
import sys

import numpy as np
import pytest

import kat_math

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import numo_oracle as oracle  # noqa: E402


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("case", kat_math.CLOSE, ids=[c[0] for c in kat_math.CLOSE])
def test_one_argument_functions(case, dt):
    fn, args, want, _ = case
    got = oracle.unary(fn, np.array(args, dtype=dt))
    assert got.dtype == dt and kat_math.close(want, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_two_argument_functions_ldexp_and_frexp(dt):
    for fn, a, b, want, _ in kat_math.EQUAL2:
        got = oracle.binary(fn, np.array(a, dtype=dt), np.array(b, dtype=dt))
        assert (got == np.array(want, dtype=dt)).all(), fn
    a, b, want = kat_math.LDEXP
    assert (oracle.binary("ldexp", np.array(a, dtype=dt), np.array(b, dtype=dt)) == np.array(want, dtype=dt)).all()
    a, mant, expo = kat_math.FREXP
    m, e = oracle.frexp(np.array(a, dtype=dt))
    assert m.dtype == dt and e.dtype == np.int32
    assert (m == np.array(mant, dtype=dt)).all() and (e == np.array(expo)).all()


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.int32])
def test_seq_logseq_and_eye(dt):
    for args, want in kat_math.SEQ:
        assert (oracle.seq((5,), dt, *args) == np.array(want, dtype=dt)).all()
    if dt != np.int32:
        for n, args, want in kat_math.LOGSEQ:
            assert (oracle.logseq((n,), dt, *args) == np.array(want, dtype=dt)).all()
        # a step that is not a binary fraction: the float types round beg + step * i once from double
        got = oracle.seq((7,), dt, 1, -0.2)
        want = [dt(np.float64(dt(1)) + np.float64(dt(-0.2)) * i) for i in range(7)]
        assert (got == np.array(want, dtype=dt)).all()
    else:
        # Int32 truncates toward zero through a 64-bit integer
        assert (oracle.seq((4,), dt, -1.5, 0.75) == [-1, 0, 0, 0]).all()
    assert (oracle.seq((2, 3), dt) == np.arange(6).reshape(2, 3)).all()
    assert (oracle.eye((3, 4), dt) == np.eye(3, 4)).all()
    assert (oracle.eye((2, 3, 3), dt, 5, -1) == 5 * np.eye(3, 3, -1)).all()


def test_modf_keeps_the_sign_in_both_parts():
    """narray_test.rb:2472-2484 (modf_expect) restated case by case."""
    x = np.array([2.75, -2.75, 0.0, -0.0, np.inf, -np.inf, 3.0, -3.0, 0.25])
    f, w = oracle.modf(x)
    assert (f == [0.75, -0.75, 0.0, -0.0, 0.0, -0.0, 0.0, -0.0, 0.25]).all()
    assert (np.signbit(f) == [False, True, False, True, False, True, False, True, False]).all()
    assert (w == [2.0, -2.0, 0.0, -0.0, np.inf, -np.inf, 3.0, -3.0, 0.0]).all()
    assert (np.signbit(w) == [False, True, False, True, False, True, False, True, False]).all()
    fn, wn = oracle.modf(np.array([np.nan], dtype=np.float32))
    assert np.isnan(fn[0]) and np.isnan(wn[0]) and fn.dtype == np.float32
    q, r = oracle.divmod_(np.array([17, 20, 23, -7], np.int32), np.array([5, 6, 7, 3], np.int32))
    assert (q == [3, 3, 3, -2]).all() and (r == [2, 2, 2, -1]).all()   # C truncation, as xint_macro.h:19-20


def test_poly_reference_cases():
    """narray_test.rb:1944-1963."""
    x = np.arange(1, 5, dtype=np.float64)
    assert (oracle.poly(x, 1.0, 2.0) == [3, 5, 7, 9]).all()
    assert (oracle.poly(x, 1.0, 2.0, 3.0) == [6, 17, 34, 57]).all()
    assert (oracle.poly(x, 3.0) == [3, 3, 3, 3]).all() and (oracle.poly(x) == x).all()
    assert (oracle.poly(np.array([2.0]), 1.0, 2.0) == [5.0]).all()
    assert (oracle.poly(x, np.ones(4), np.full(4, 2.0)) == [3, 5, 7, 9]).all()
    assert (oracle.poly(x.astype(np.float32), 1.0, 2.0) == [3, 5, 7, 9]).all()
    assert (oracle.poly(np.arange(1, 5, dtype=np.int32), 1, 2) == [3, 5, 7, 9]).all()
    # against exact integer arithmetic, wrapping for Int32
    xi = np.array([3, -7, 100000, 46341], dtype=np.int32)
    want = [(5 + 4 * int(v) + 3 * int(v) ** 2 + 2 * int(v) ** 3 + 2 ** 31) % 2 ** 32 - 2 ** 31 for v in xi]
    assert (oracle.poly(xi, 5, 4, 3, 2) == want).all()
