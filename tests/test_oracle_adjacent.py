"""The oracle's pow, clip and maximum/minimum against the literals of the
reference's own tests (tests/kat_adjacent.py) and against what the mathematics
fixes: integer powers by repeated exact multiplication, pow against Python's
correctly rounded float power on exactly representable cases, NaN rules of
types/real_accum.h:444-486 enumerated."""
import math

import numpy as np
import pytest

import kat_adjacent as K

oracle = K.OracleEngine().o


@pytest.mark.parametrize("name,fn,t", K.all_cases(), ids=lambda v: v if isinstance(v, str) else None)
def test_reference_literals(name, fn, t):
    K.run(K.OracleEngine(), name, fn, t)


def test_int32_pow_is_wrapping_repeated_multiplication():
    rng = np.random.default_rng(1)
    x = rng.integers(-50, 50, size=400).astype(np.int32)
    p = rng.integers(-3, 12, size=400).astype(np.int32)
    got = oracle.binary("pow", x, p)
    want = []
    for a, e in zip(x.tolist(), p.tolist()):
        if e < 0:
            want.append(0 if e not in (0, 1, 2, 3) else None)
        else:
            v = (a ** e) & 0xFFFFFFFF
            want.append(v - (1 << 32) if v >= (1 << 31) else v)
    assert got.tolist() == want


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_float_pow_int_small_exponents_are_exact_products(dt):
    # integers small enough that every product is exact in the element type
    x = np.array([1, 2, 3, -2, 0.5, -0.25, 10], dtype=dt)
    for e in range(0, 8):
        got = oracle.pow_int(x, e)
        want = np.array([float(v) ** e for v in x.tolist()], dtype=dt)
        assert (got == want).all(), e
    got = oracle.pow_int(x[:6], -2)
    assert (got == np.array([1 / (float(v) ** 2) for v in x[:6].tolist()], dtype=dt)).all()
    # beyond 64 the macro calls pow(): 2 ** 100 is still exact in both types
    assert oracle.pow_int(np.array([2], dtype=dt), 100)[0] == dt(2.0 ** 100)


def test_float_pow_rounds_the_double_result_once():
    x = np.array([2.0, 9.0, 0.25, 10.0, 1e-3], dtype=np.float32)
    y = np.array([0.5, 0.5, 1.5, -2.0, 3.0], dtype=np.float32)
    got = oracle.binary("pow", x, y)
    want = np.array([np.float32(math.pow(float(a), float(b))) for a, b in zip(x, y)], dtype=np.float32)
    assert (got == want).all()
    d = oracle.binary("pow", x.astype(np.float64), y.astype(np.float64))
    assert d.tolist() == [math.pow(float(a), float(b)) for a, b in zip(x, y)]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_maximum_minimum_nan_rules(dt):
    nan = math.nan
    x = np.array([1, 3, nan, 2, nan, -0.0, 0.0], dtype=dt)
    y = np.array([2, 1, 5, nan, nan, 0.0, -0.0], dtype=dt)
    # plain: the other operand when one is NaN (real_accum.h:444-453,466-475)
    assert K.same(oracle.binary("maximum", x, y).tolist(), [2, 3, 5, 2, nan, -0.0, 0.0])
    assert K.same(oracle.binary("minimum", x, y).tolist(), [1, 1, 5, 2, nan, -0.0, 0.0])
    # _nan: the NaN (real_accum.h:455-464,477-486)
    assert K.same(oracle.binary("maximum_nan", x, y).tolist(), [2, 3, nan, nan, nan, -0.0, 0.0])
    assert K.same(oracle.binary("minimum_nan", x, y).tolist(), [1, 1, nan, nan, nan, -0.0, 0.0])
    # x >= y decides first, so equal zeros answer x with its own sign
    assert np.signbit(oracle.binary("maximum", x, y)[5]) and not np.signbit(oracle.binary("maximum", x, y)[6])


def test_clip_by_brute_force_on_random_views():
    rng = np.random.default_rng(2)
    for dt in (np.float32, np.float64, np.int32):
        x = rng.integers(-20, 20, size=(7, 9)).astype(dt)
        lo = rng.integers(-10, 0, size=(7, 9)).astype(dt)
        hi = rng.integers(0, 10, size=(7, 9)).astype(dt)
        got = oracle.clip(np.ascontiguousarray(x[::2, 1::3]), np.ascontiguousarray(lo[::2, 1::3]), np.ascontiguousarray(hi[::2, 1::3]))
        assert (got == np.minimum(np.maximum(x, lo), hi)[::2, 1::3]).all()
        assert (oracle.clip(x, -3, 4) == np.clip(x, -3, 4)).all()


def test_where_mask_and_index_arrays_against_the_reference_literals():
    """test/bit_test.rb:20-37,50-69,161-163 and test/narray_test.rb:124-134,171,294-310,528."""
    src = [0, 1, 1, 0, 1, 0, 0, 1]
    for shape in ((8,), (2, 4)):
        b = np.array(src, dtype=np.uint8).reshape(shape)
        assert oracle.where(b).tolist() == [1, 2, 4, 7]
        assert oracle.where(b, invert=True).tolist() == [0, 3, 5, 6]
        assert oracle.mask(b, np.arange(1.0, 9.0).reshape(shape)).tolist() == [2, 3, 5, 8]
    assert oracle.where(np.zeros(0, dtype=np.uint8)).tolist() == []
    assert oracle.mask(np.zeros(0, dtype=np.uint8), np.zeros(0)).tolist() == []
    with pytest.raises(ValueError):
        oracle.mask(np.ones(3, dtype=np.uint8), np.ones(4))
    a = np.array([1, 2, 3, 5, 7, 11], dtype=np.float64)
    assert oracle.at(a, [3, 4]).tolist() == [5, 7]
    assert oracle.at(a[2:], [1, 2]).tolist() == [5, 7]
    assert oracle.at(a, range(3, 5)).tolist() == [5, 7]
    assert oracle.at(a, [-1]).tolist() == [11]
    assert oracle.take(a, ([4, 3, 0, 1, 5, 2],)).tolist() == [7, 5, 1, 2, 11, 3]
    m = np.array([[1, 2, 3], [5, 7, 11]], dtype=np.float64)
    assert oracle.at(m, [0, 1], [1, 2]).tolist() == [2, 11]
    assert oracle.at(m, [0, 1], range(0, 3, 2)).tolist() == [1, 11]
    assert oracle.at(m, range(0, 2), [0, 2]).tolist() == [1, 11]
    assert oracle.take(m, ([0, 1], [0, 2])).tolist() == [[1, 3], [5, 11]]
    assert oracle.take(m, (slice(None), [2, 0, 1])).tolist() == [[3, 1, 2], [11, 5, 7]]
    assert oracle.take(m, (1, [2, 0, 0])).tolist() == [11, 5, 5]
    c = np.array([[[1, 2], [3, 4]], [[5, 6], [7, 8]]], dtype=np.float64)
    assert oracle.at(c, [0, 1], [1, 0], [0, 1]).tolist() == [3, 6]
    with pytest.raises(ValueError):
        oracle.at(m, [0, 1], [0, 1, 2])
    with pytest.raises(IndexError):
        oracle.take(m, ([2], 0))
    z = m.copy()
    oracle.put(z, ([1, 0], [0, 2]), 9)
    assert z.tolist() == [[9, 2, 9], [9, 7, 9]]
    oracle.put(z, ([0],), np.array([1.0, 2.0, 3.0]))
    assert z.tolist() == [[1, 2, 3], [9, 7, 9]]
    # where against a sequential scan on a larger array, mask against where
    rng = np.random.default_rng(0)
    bits = (rng.random((37, 41)) < 0.3).astype(np.uint8)
    seq = [i for i, v in enumerate(bits.reshape(-1).tolist()) if v]
    assert oracle.where(bits).tolist() == seq
    vals = rng.standard_normal((37, 41))
    assert oracle.mask(bits, vals).tolist() == [vals.reshape(-1)[i] for i in seq]
