"""Pins the CPU oracle (oracle/numo_oracle.c) without the device:
 - against the literals the reference's own tests hold (tests/golden/reference_kats.json),
 - against what arithmetic fixes: IEEE single operations via numpy, closed forms,
   exact rational arithmetic, brute-force addressing.
A mistake in the oracle (dropped term, wrong sign, transposed operand, wrong index)
fails at least one of these."""
import fractions
import math
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import numo_oracle as oracle  # noqa: E402

from helpers import assert_bits_equal  # noqa: E402
import kat  # noqa: E402

CASES = kat.load_cases()


@pytest.mark.parametrize("tc", CASES, ids=[kat.case_id(tc) for tc in CASES])
def test_reference_literals(tc):
    t, c = tc
    kat.check(t, c, kat.run_oracle(t, c, oracle))


# ---- IEEE single operations: bit-exact against numpy ---------------------------------
@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("op,npf", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)])
def test_binary_ieee(dt, op, npf):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((37, 53)).astype(dt)
    y = rng.standard_normal((37, 53)).astype(dt)
    y[3, 4] = 0
    x[5, 6] = np.inf
    x[7, 8] = np.nan
    with np.errstate(all="ignore"):
        want = npf(x, y)
    assert_bits_equal(oracle.binary(op, x, y), want, op)
    # a dropped/transposed operand shows on the non-commutative ones
    with np.errstate(all="ignore"):
        assert_bits_equal(oracle.binary(op, x, 2.5), npf(x, dt(2.5)), op + " scalar right")
        assert_bits_equal(oracle.binary(op, 2.5, x, scalar_is_left=True), npf(dt(2.5), x), op + " scalar left")


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_unary_closed_forms(dt):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(1000) * 10).astype(dt)
    x[:4] = [0.0, -0.0, np.inf, np.nan]
    with np.errstate(all="ignore"):
        assert_bits_equal(oracle.unary("minus", x), -x)
        assert_bits_equal(oracle.unary("abs", x), np.abs(x))
        assert_bits_equal(oracle.unary("square", x), x * x)
        assert_bits_equal(oracle.unary("reciprocal", x), (dt(1) / x).astype(dt))
        assert_bits_equal(oracle.unary("floor", x), np.floor(x))
        assert_bits_equal(oracle.unary("ceil", x), np.ceil(x))
        assert_bits_equal(oracle.unary("trunc", x), np.trunc(x))
        assert_bits_equal(oracle.unary("rint", x), np.rint(x))
        assert_bits_equal(oracle.unary("sqrt", np.abs(x)), np.sqrt(np.abs(x)))
        s = oracle.unary("sign", x)
    assert s[0] == 0 and s[1] == 0 and s[2] == 1 and np.isnan(s[3])
    # round: half away from zero (C round), not numpy's half-to-even
    r = oracle.unary("round", np.array([0.5, 1.5, 2.5, -0.5, -2.5], dtype=dt))
    assert r.tolist() == [1.0, 2.0, 3.0, -1.0, -3.0]


def test_sfloat_math_is_double_rounded_once():
    # the host macro is the double function on the promoted argument
    # (types/float_macro.h:84-118), so it equals numpy's float64 function rounded to float32
    rng = np.random.default_rng(12)
    x = (rng.standard_normal(4096) * 3).astype(np.float32)
    for name, f in [("exp", np.exp), ("sin", np.sin), ("cos", np.cos), ("tanh", np.tanh), ("log1p", None), ("expm1", np.expm1)]:
        arg = np.abs(x) if name == "log1p" else x
        f = np.log1p if name == "log1p" else f
        want = f(arg.astype(np.float64)).astype(np.float32)
        got = oracle.unary(name, arg)
        # numpy's float64 functions are glibc's or within 1 ulp of it in double, which
        # can move the float32 rounding by at most one unit in rare ties
        from helpers import assert_ulp
        assert_ulp(got, want, 1, name)
    assert oracle.unary("sinc", np.array([0.0], dtype=np.float32))[0] == 1.0
    assert oracle.unary("exp", np.array([0.0], dtype=np.float64))[0] == 1.0
    assert oracle.unary("log", np.array([1.0], dtype=np.float64))[0] == 0.0
    assert oracle.unary("exp2", np.array([10.0], dtype=np.float64))[0] == 1024.0
    assert abs(oracle.unary("exp10", np.array([3.0], dtype=np.float64))[0] - 1000.0) < 1e-12  # glibc's exp10 is not exact here
    assert abs(oracle.unary("cbrt", np.array([27.0], dtype=np.float64))[0] - 3.0) < 1e-15  # nor is its cbrt
    assert oracle.binary("hypot", np.array([3.0]), np.array([4.0]))[0] == 5.0
    assert oracle.binary("atan2", np.array([1.0]), np.array([1.0]))[0] == math.atan2(1, 1)
    assert oracle.binary("mod", np.array([7.5]), np.array([2.0]))[0] == 1.5
    assert oracle.binary("mod", np.array([-7.5]), np.array([2.0]))[0] == -1.5  # fmod keeps the dividend's sign
    assert oracle.binary("copysign", np.array([3.0]), np.array([-0.0]))[0] == -3.0


# ---- Int32: C integer semantics -------------------------------------------------------
def test_int32_ops():
    rng = np.random.default_rng(13)
    x = rng.integers(-1000, 1000, size=(31, 17), dtype=np.int32)
    y = rng.integers(1, 50, size=(31, 17), dtype=np.int32) * rng.choice(np.array([-1, 1], dtype=np.int32), size=(31, 17))
    assert_bits_equal(oracle.binary("add", x, y), x + y)
    assert_bits_equal(oracle.binary("sub", x, y), x - y)
    assert_bits_equal(oracle.binary("mul", x, y), x * y)
    # C division truncates toward zero and % keeps the dividend's sign
    q = np.trunc(x.astype(np.float64) / y).astype(np.int32)
    assert_bits_equal(oracle.binary("div", x, y), q)
    assert_bits_equal(oracle.binary("mod", x, y), (x - q * y).astype(np.int32))
    assert_bits_equal(oracle.binary("bit_and", x, y), x & y)
    assert_bits_equal(oracle.binary("bit_or", x, y), x | y)
    assert_bits_equal(oracle.binary("bit_xor", x, y), x ^ y)
    sh = np.abs(y) % 31
    assert_bits_equal(oracle.binary("left_shift", np.abs(x) % 1000, sh % 20), ((np.abs(x) % 1000) << (sh % 20)).astype(np.int32))
    assert_bits_equal(oracle.binary("right_shift", x, sh), x >> sh)  # arithmetic shift
    assert_bits_equal(oracle.unary("bit_not", x), ~x)
    assert_bits_equal(oracle.unary("abs", x), np.abs(x))
    # wrap-around
    big = np.array([2**31 - 1], dtype=np.int32)
    assert oracle.binary("add", big, np.array([1], dtype=np.int32))[0] == -2**31
    assert oracle.unary("reciprocal", np.array([1, -1, 2, -7], dtype=np.int32)).tolist() == [1, -1, 0, 0]


def test_int32_flags():
    x = np.array([6, 7, 8], dtype=np.int32)
    y = np.array([2, 0, 4], dtype=np.int32)
    out = np.full(3, -99, dtype=np.int32)
    with pytest.raises(oracle.FlagError):
        oracle.binary("div", x, y, out=out)
    assert out.tolist() == [3, -99, 2]  # the rejected element is not stored
    with pytest.raises(oracle.FlagError):
        oracle.unary("abs", np.array([-2**31], dtype=np.int32))
    with pytest.raises(oracle.FlagError):
        oracle.unary("reciprocal", np.array([0], dtype=np.int32))


# ---- addressing: views and broadcast by brute force -------------------------------------
def test_views_and_broadcast_brute_force():
    rng = np.random.default_rng(14)
    base = rng.standard_normal((6, 8, 10))
    views = [base[::2, 1::3, ::-1], base.transpose(2, 0, 1), base[1:, :, 3], base[:, ::-2, 1:9:4]]
    for v in views:
        w = rng.standard_normal(v.shape[-1])
        want = np.empty(v.shape)
        for idx in np.ndindex(*v.shape):
            want[idx] = v[idx] - w[idx[-1]]
        assert_bits_equal(oracle.binary("sub", v, w), want)
        col = rng.standard_normal(v.shape[:-1] + (1,))
        assert_bits_equal(oracle.binary("sub", col, v), col - v)
        assert_bits_equal(oracle.copy(v), np.ascontiguousarray(v))
    # writing through a strided destination
    dst = np.zeros((4, 10))
    oracle.binary("add", base[0, :4, :5], base[1, :4, :5], out=dst[:, ::2])
    assert_bits_equal(dst[:, ::2], base[0, :4, :5] + base[1, :4, :5])
    assert (dst[:, 1::2] == 0).all()


def test_casts():
    x = np.array([1.75, -2.5, 3.999, -0.0, 1e9], dtype=np.float64)
    assert oracle.store(np.int32, x).tolist() == [1, -2, 3, 0, 1000000000]  # truncation
    assert_bits_equal(oracle.store(np.float32, x), x.astype(np.float32))
    i = np.array([2**31 - 1, -2**31, 16777217], dtype=np.int32)
    assert_bits_equal(oracle.store(np.float32, i), i.astype(np.float32))
    assert_bits_equal(oracle.store(np.float64, i), i.astype(np.float64))
    assert_bits_equal(oracle.fill(np.float32, (3, 2), 1.1), np.full((3, 2), 1.1, dtype=np.float32))


# ---- Bit ---------------------------------------------------------------------------------
def test_bit_packing_lsb_first():
    x = np.array([0, 1, 2, 3, 4, 5, 6, 7, 8, 9] * 5, dtype=np.int32)
    bits = oracle.compare("gt", x, 4)
    assert bits.tolist() == (x > 4).astype(np.uint8).tolist()
    w = oracle.pack(bits)
    # element k is bit k%32 of word k//32
    for k in range(x.size):
        assert (int(w[k // 32]) >> (k % 32)) & 1 == int(x[k] > 4)
    assert oracle.bit_count(w, 0, 1, x.size) == int((x > 4).sum())
    assert oracle.bit_count(w, 0, 1, x.size, count_false=True) == int((x <= 4).sum())
    assert oracle.bit_count(w, 3, 2, 20) == int((x[3:43:2] > 4).sum())
    assert oracle.bit_count(w, 49, -1, 50) == int((x > 4).sum())


def test_bit_logic_and_compare_cases():
    rng = np.random.default_rng(15)
    a = rng.integers(0, 2, size=(5, 67)).astype(np.uint8)
    b = rng.integers(0, 2, size=(5, 67)).astype(np.uint8)
    assert (oracle.bit_binary("and", a, b) == (a & b)).all()
    assert (oracle.bit_binary("or", a, b) == (a | b)).all()
    assert (oracle.bit_binary("xor", a, b) == (a ^ b)).all()
    assert (oracle.bit_binary("eq", a, b) == (a == b)).all()
    assert (oracle.bit_binary("not", a) == 1 - a).all()
    assert (oracle.bit_binary("and", a, b[0]) == (a & b[0])).all()
    x = np.array([1.0, np.nan, np.inf, -np.inf, -0.0, 0.0], dtype=np.float32)
    assert oracle.cond_unary("isnan", x).tolist() == [0, 1, 0, 0, 0, 0]
    assert oracle.cond_unary("isinf", x).tolist() == [0, 0, 1, 1, 0, 0]
    assert oracle.cond_unary("isposinf", x).tolist() == [0, 0, 1, 0, 0, 0]
    assert oracle.cond_unary("isneginf", x).tolist() == [0, 0, 0, 1, 0, 0]
    assert oracle.cond_unary("isfinite", x).tolist() == [1, 0, 0, 0, 1, 1]
    assert oracle.cond_unary("signbit", x).tolist() == [0, 0, 0, 1, 1, 0]
    assert oracle.compare("ne", x, x).tolist() == [0, 1, 0, 0, 0, 0]
    assert oracle.compare("lt", 0.5, x, scalar_is_left=True).tolist() == [1, 0, 1, 0, 0, 0]
    assert oracle.compare("nearly_eq", np.array([1.0], dtype=np.float32), np.array([1.0 + 2e-7], dtype=np.float32)).tolist() == [1]
    assert oracle.compare("nearly_eq", np.array([1.0], dtype=np.float32), np.array([1.001], dtype=np.float32)).tolist() == [0]
    assert (oracle.store_bit(np.float64, a) == a).all()


# ---- reductions -----------------------------------------------------------------------------
def test_sum_is_sequential_in_row_major_order():
    # float32 values chosen so that the order of addition shows in the last bits
    rng = np.random.default_rng(16)
    x = (rng.standard_normal((7, 5, 11)) * 1000).astype(np.float32)
    for axes in [(2,), (0,), (1, 2), (0, 2), None]:
        got = oracle.reduce("sum", x, axis=axes)
        ax = tuple(range(3)) if axes is None else axes
        keep = [d for d in range(3) if d not in ax]
        xt = x.transpose(keep + list(ax)).reshape([x.shape[d] for d in keep] + [-1])
        want = np.zeros(xt.shape[:-1], dtype=np.float32)
        for idx in np.ndindex(*xt.shape[:-1]):
            acc = np.float32(0)
            for v in xt[idx]:
                acc = np.float32(v + acc)
            want[idx] = acc
        assert_bits_equal(got, want, str(axes))


def test_moments_against_exact_rationals():
    # test/narray_test.rb:2969-3046 checks var/mean against exact rational arithmetic
    xs = [1000.0 + ((i * 7919) % 2003) / 1000.0 for i in range(4000)]
    fr = [fractions.Fraction(v) for v in xs]
    mean = sum(fr) / len(fr)
    var = sum((v - mean) ** 2 for v in fr) / (len(fr) - 1)
    rms = math.sqrt(float(sum(v * v for v in fr) / len(fr)))
    x = np.array(xs)
    assert abs(oracle.reduce("mean", x) - float(mean)) <= abs(float(mean)) * 1e-13
    assert abs(oracle.reduce("var", x) - float(var)) <= float(var) * 1e-9
    assert abs(oracle.reduce("stddev", x) - math.sqrt(float(var))) <= math.sqrt(float(var)) * 1e-9
    assert abs(oracle.reduce("rms", x) - rms) <= rms * 1e-12
    # n-1 in the divisor, not n
    assert oracle.reduce("var", np.array([1.0, 3.0])) == 2.0


def test_integer_valued_sums_are_exact_on_every_axis():
    rng = np.random.default_rng(17)
    x = rng.integers(-50, 50, size=(6, 7, 8)).astype(np.float32)
    for ax in [0, 1, 2, (0, 1), (1, 2), (0, 2), None]:
        assert_bits_equal(oracle.reduce("sum", x, axis=ax), x.sum(axis=ax, dtype=np.float32).astype(np.float32), str(ax))
        assert_bits_equal(oracle.reduce("max", x, axis=ax), x.max(axis=ax))
        assert_bits_equal(oracle.reduce("min", x, axis=ax), x.min(axis=ax))
    xi = x.astype(np.int32)
    assert_bits_equal(oracle.reduce("sum", xi, axis=1), xi.sum(axis=1, dtype=np.int64))
    assert oracle.reduce("sum", xi).dtype == np.int64
    v = x[::2, :, ::-1]
    assert_bits_equal(oracle.reduce("sum", v, axis=2), v.sum(axis=2, dtype=np.float32))
    assert oracle.reduce("sum", x, axis=1, keepdims=True).shape == (6, 1, 8)


def test_arg_reductions_brute_force():
    rng = np.random.default_rng(18)
    x = rng.integers(0, 4, size=(5, 9, 6)).astype(np.float64)  # many ties
    for ax in [0, 1, 2]:
        assert (oracle.reduce("argmax", x, axis=ax) == np.argmax(x, axis=ax)).all()  # numpy: first occurrence
        assert (oracle.reduce("argmin", x, axis=ax) == np.argmin(x, axis=ax)).all()
    # max_index is the flat index into the array
    mi = oracle.reduce("max_index", x, axis=2)
    assert (x.reshape(-1)[mi] == x.max(axis=2)).all()
    assert (mi == np.argmax(x, axis=2) + np.arange(45).reshape(5, 9) * 6).all()
    # ... also when the axis is not the innermost one, and over two axes
    m1 = oracle.reduce("max_index", x, axis=1)
    assert (m1 == np.arange(5).reshape(5, 1) * 54 + np.argmax(x, axis=1) * 6 + np.arange(6)).all()
    m02 = oracle.reduce("min_index", x, axis=(0, 2))
    for j in range(9):
        sl = x[:, j, :]
        i, k = np.unravel_index(np.argmin(sl), sl.shape)
        assert m02[j] == i * 54 + j * 6 + k
    # NaN: skipped unless nan: true, where the first NaN wins
    y = np.array([2.0, np.nan, 5.0, np.nan, 5.0])
    assert oracle.reduce("argmax", y) == 2
    assert oracle.reduce("argmin", y) == 0
    assert oracle.reduce("argmax", y, nan=True) == 1
    assert oracle.reduce("argmin", y, nan=True) == 1
    assert oracle.reduce("argmax", np.array([np.nan, np.nan])) == 0


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_nd_driver_walks_a_strided_axis_like_the_1d_loops(dt):
    """The N-d driver hands each run to the same sequential loop as the 1-d entry point:
    a reduction along a strided axis equals the 1-d loop over the copied-out column."""
    rng = np.random.default_rng(19)
    a = rng.standard_normal((9, 14)).astype(dt)
    a[3, 5] = np.nan
    for op in ("sum", "max", "min", "mean", "var", "sum_nan", "max_nan"):
        nan = op.endswith("_nan")
        got = oracle.reduce(op[:-4] if nan else op, a, axis=0, nan=nan)
        for j in range(14):
            want = np.array([oracle.f1d(op, np.ascontiguousarray(a[:, j]))], dtype=dt)
            assert_bits_equal(np.array([got[j]], dtype=dt), want, "%s column %d" % (op, j))
