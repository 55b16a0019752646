"""pow, clip and maximum/minimum on the device: the reference's own literals
(tests/kat_adjacent.py) and parity with the CPU oracle on seeded inputs over
contiguous arrays, views and repeated operands. Bars: Int32 and clip/maximum/
minimum bit-exact; Float ** Int32 (products in the element type) bit-exact;
SFloat pow <= 1 ulp (the device evaluates pow in double and rounds once, as the
host macro does); DFloat pow <= 2 ulp against glibc."""
import numpy as np
import pytest

import kat_adjacent as K
from helpers import assert_bits_equal, assert_ulp

pytestmark = pytest.mark.gpu

oracle = K.OracleEngine().o
FLOATS = [("sfloat", np.float32), ("dfloat", np.float64)]
ALL = FLOATS + [("int32", np.int32)]


def cls_of(t):
    import cumo_amd
    return {"sfloat": cumo_amd.SFloat, "dfloat": cumo_amd.DFloat, "int32": cumo_amd.Int32}[t]


@pytest.mark.parametrize("name,fn,t", K.all_cases(), ids=lambda v: v if isinstance(v, str) else None)
def test_reference_literals(name, fn, t):
    K.run(K.DeviceEngine(), name, fn, t)


@pytest.mark.parametrize("tname,dt", ALL)
def test_clip_parity_over_views(tname, dt):
    cls = cls_of(tname)
    rng = np.random.default_rng(41)
    for shape in [(1,), (5,), (1023,), (4096,), (33, 65), (4, 5, 128), (100003,)]:
        hx = rng.integers(-50, 50, size=shape).astype(dt)
        hlo = rng.integers(-30, 0, size=shape).astype(dt)
        hhi = rng.integers(0, 30, size=shape).astype(dt)
        if dt != np.int32:
            hx.reshape(-1)[::7] = np.nan
        x, lo, hi = cls.cast(hx), cls.cast(hlo), cls.cast(hhi)
        assert_bits_equal(x.clip(-7, 9).to_numpy(), oracle.clip(hx, -7, 9), (shape, "scalars"))
        assert_bits_equal(x.clip(-7, None).to_numpy(), oracle.clip(hx, -7, None), (shape, "min"))
        assert_bits_equal(x.clip(None, 9).to_numpy(), oracle.clip(hx, None, 9), (shape, "max"))
        assert_bits_equal(x.clip(lo, hi).to_numpy(), oracle.clip(hx, hlo, hhi), (shape, "arrays"))
        assert_bits_equal(x.clip(lo, None).to_numpy(), oracle.clip(hx, hlo, None), (shape, "min array"))
        assert_bits_equal(x.clip(None, hi).to_numpy(), oracle.clip(hx, None, hhi), (shape, "max array"))
        assert_bits_equal(x.clip(lo, 12).to_numpy(), oracle.clip(hx, hlo, 12), (shape, "array, scalar"))
        if len(shape) == 2:
            assert_bits_equal(x.transpose().clip(lo.transpose(), 3).to_numpy(), oracle.clip(np.ascontiguousarray(hx.T), np.ascontiguousarray(hlo.T), 3))
            assert_bits_equal(x[::2, 1::3].clip(-1, 1).to_numpy(), oracle.clip(np.ascontiguousarray(hx[::2, 1::3]), -1, 1))
            assert_bits_equal(x.clip(lo[0], hi[:, :1]).to_numpy(),
                              oracle.clip(hx, np.ascontiguousarray(np.broadcast_to(hlo[0], shape)), np.ascontiguousarray(np.broadcast_to(hhi[:, :1], shape))))


@pytest.mark.parametrize("tname,dt", ALL)
def test_maximum_minimum_parity(tname, dt):
    cls = cls_of(tname)
    rng = np.random.default_rng(42)
    for shape in [(3,), (1000,), (65, 33), (3, 4, 64)]:
        hx = rng.integers(-9, 9, size=shape).astype(dt)
        hy = rng.integers(-9, 9, size=shape).astype(dt)
        if dt != np.int32:
            hx.reshape(-1)[::5] = np.nan
            hy.reshape(-1)[::7] = np.nan
            hx.reshape(-1)[1::11] = -0.0
            hy.reshape(-1)[1::11] = 0.0
        x, y = cls.cast(hx), cls.cast(hy)
        for op in ("maximum", "minimum"):
            assert_bits_equal(getattr(cls, op)(x, y).to_numpy(), oracle.binary(op, hx, hy), (shape, op))
            if dt != np.int32:
                assert_bits_equal(getattr(cls, op)(x, y, nan=True).to_numpy(), oracle.binary(op + "_nan", hx, hy), (shape, op, "nan"))
            if len(shape) == 2:
                assert_bits_equal(getattr(cls, op)(x.transpose(), y.transpose()).to_numpy(),
                                  oracle.binary(op, np.ascontiguousarray(hx.T), np.ascontiguousarray(hy.T)))
                assert_bits_equal(getattr(cls, op)(x, y[0]).to_numpy(), oracle.binary(op, hx, np.ascontiguousarray(np.broadcast_to(hy[0], shape))))
    # mixed types move to the higher one (Int32 < SFloat < DFloat)
    import cumo_amd
    a = cumo_amd.Int32.cast(np.array([1, 5, -3], dtype=np.int32))
    b = cumo_amd.SFloat.cast(np.array([2.5, 4.5, -3.5], dtype=np.float32))
    r = cumo_amd.SFloat.maximum(a, b)
    assert isinstance(r, cumo_amd.SFloat) and r.to_numpy().tolist() == [2.5, 5.0, -3.0]


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_float_pow_parity(tname, dt):
    cls = cls_of(tname)
    import cumo_amd
    rng = np.random.default_rng(43)
    ulp = 1 if dt == np.float32 else 2
    for shape in [(7,), (1024,), (4100,), (33, 65), (2, 3, 128)]:
        hx = rng.uniform(0.1, 9.0, size=shape).astype(dt)
        hy = rng.uniform(-3.0, 3.0, size=shape).astype(dt)
        hp = rng.integers(-6, 70, size=shape).astype(np.int32)
        x, y, p = cls.cast(hx), cls.cast(hy), cumo_amd.Int32.cast(hp)
        assert_ulp((x ** y).to_numpy(), oracle.binary("pow", hx, hy), ulp, (shape, "array ** array"))
        assert_ulp((x ** 2.5).to_numpy(), oracle.binary("pow", hx, 2.5), ulp, (shape, "array ** 2.5"))
        assert_ulp((2.5 ** y).to_numpy(), oracle.binary("pow", 2.5, hy, scalar_is_left=True), ulp, (shape, "2.5 ** array"))
        # Int32 exponents: products in the element type, so the bits agree (pow() beyond 64: <= ulp)
        small = hp <= 64
        got = (x ** p).to_numpy()
        want = oracle.pow_int(hx, hp)
        assert_bits_equal(got[small], want[small], (shape, "array ** Int32 array"))
        assert_ulp(got, want, ulp, (shape, "array ** Int32 array, large exponents"))
        for e in (0, 1, 2, 3, 4, 5, 17, 64, -1, -3):
            assert_bits_equal((x ** e).to_numpy(), oracle.pow_int(hx, e), (shape, "array **", e))
        assert_ulp((x ** 65).to_numpy(), oracle.pow_int(hx, 65), ulp)
        got = (1.5 ** p)
        assert isinstance(got, cumo_amd.DFloat)
        assert_bits_equal(got.to_numpy()[small], oracle.pow_int(np.float64(1.5), hp)[small], (shape, "1.5 ** Int32 array"))
        if len(shape) == 2:
            assert_ulp((x.transpose() ** y.transpose()).to_numpy(), oracle.binary("pow", np.ascontiguousarray(hx.T), np.ascontiguousarray(hy.T)), ulp)
            assert_bits_equal((x[:, ::2] ** p[:, ::2]).to_numpy()[small[:, ::2]], oracle.pow_int(hx[:, ::2], hp[:, ::2])[small[:, ::2]])
    # special values of pow()
    hx = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 2.0, -8.0], dtype=dt)
    for e in (0.0, 0.5, -1.0, 2.0, np.inf, np.nan, 1.0 / 3):
        with np.errstate(all="ignore"):
            assert_ulp((cls.cast(hx) ** float(e)).to_numpy(), oracle.binary("pow", hx, float(e)), ulp, ("special", e))


def test_int32_pow_parity_and_type_rules():
    import cumo_amd
    rng = np.random.default_rng(44)
    hx = rng.integers(-40, 40, size=(37, 65)).astype(np.int32)
    hp = rng.integers(-3, 12, size=(37, 65)).astype(np.int32)
    x, p = cumo_amd.Int32.cast(hx), cumo_amd.Int32.cast(hp)
    assert_bits_equal((x ** p).to_numpy(), oracle.binary("pow", hx, hp))
    assert_bits_equal((x.transpose() ** p.transpose()).to_numpy(), oracle.binary("pow", np.ascontiguousarray(hx.T), np.ascontiguousarray(hp.T)))
    for e in (0, 1, 2, 3, 7, 31, -1):
        assert_bits_equal((x ** e).to_numpy(), oracle.binary("pow", hx, e), e)
    assert_bits_equal((3 ** p).to_numpy(), oracle.binary("pow", 3, hp, scalar_is_left=True))
    # Int32 ** Float moves the array to DFloat; Int32 ** SFloat array answers SFloat
    r = x ** 0.5
    assert isinstance(r, cumo_amd.DFloat)
    with np.errstate(invalid="ignore"):
        assert_ulp(r.to_numpy(), oracle.binary("pow", hx.astype(np.float64), 0.5), 2)
    y = cumo_amd.SFloat.cast(np.full((37, 65), 2.0, dtype=np.float32))
    r = x ** y
    assert isinstance(r, cumo_amd.SFloat)
    assert_ulp(r.to_numpy(), oracle.binary("pow", hx.astype(np.float32), np.full((37, 65), 2.0, dtype=np.float32)), 1)
