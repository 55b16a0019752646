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
