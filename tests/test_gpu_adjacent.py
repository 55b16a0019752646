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
def test_float_pow_by_whole_numbers_of_halves(tname, dt):
    """array ** y for one exponent that is a whole number of halves (squarings, multiplications, one square root on
    the device) against pow: ordinary bases, bases at the ends of the range, zeros, infinities, negatives and NaN."""
    cls = cls_of(tname)
    rng = np.random.default_rng(47)
    ulp = 1 if dt == np.float32 else 2
    info = np.finfo(dt)
    ordinary = np.exp2(rng.uniform(-20.0, 20.0, size=5000)).astype(dt)
    ends = np.concatenate([np.exp2(rng.uniform(info.minexp - 20, info.minexp + 30, size=500)),
                           np.exp2(rng.uniform(info.maxexp - 30, info.maxexp - 0.001, size=500))]).astype(dt)
    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 2.0, -8.0, -0.25, info.tiny, info.max,
                        info.smallest_subnormal], dtype=dt)
    hx = np.concatenate([ordinary, ends, special, -ordinary[:100]])
    x = cls.cast(hx)
    for twice in range(-17, 18):
        e = 0.5 * twice
        with np.errstate(all="ignore"):
            assert_ulp((x ** e).to_numpy(), oracle.binary("pow", hx, e), ulp, ("array **", e))
    hm = ordinary.reshape(50, 100)
    with np.errstate(all="ignore"):
        assert_ulp((cls.cast(hm)[:, 1:] ** 1.5).to_numpy(), oracle.binary("pow", np.ascontiguousarray(hm[:, 1:]), 1.5), ulp)
        assert_ulp((cls.cast(hm).transpose() ** -2.5).to_numpy(), oracle.binary("pow", np.ascontiguousarray(hm.T), -2.5), ulp)


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_float_pow_parity(tname, dt):
    cls = cls_of(tname)
    import cumo_amd
    rng = np.random.default_rng(43)
    # against the oracle: SFloat is the double pow rounded once on both sides; DFloat pow is
    # within 1 ulp of the correctly rounded value on the device and in glibc alike
    # (test_gpu_nmath_vectors.py, test_nmath_vectors.py), so within 2 of each other
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


def _cum_close(got, want_exact, scale, n, dt, what):
    """Float scans against the exactly accumulated value: rel 1e-5*log2(n) for SFloat,
    1e-12*log2(n) for DFloat, of the running sum of magnitudes (the bar the parity
    contract sets for float reductions)."""
    tol = (1e-5 if dt == np.float32 else 1e-12) * max(1.0, np.log2(max(n, 2)))
    err = np.abs(got.astype(np.float64) - want_exact)
    bad = err > tol * np.maximum(scale, 1e-300)
    assert not bad.any(), (what, float(err.max()), int(bad.sum()))


@pytest.mark.parametrize("tname,dt", ALL)
def test_cumsum_cumprod_parity(tname, dt):
    cls = cls_of(tname)
    rng = np.random.default_rng(51)
    for shape, axes in [((5,), [None]), ((2049,), [None]), ((70001,), [None]), ((300001,), [None]), ((37, 129), [None, 0, 1, -1]),
                        ((3, 5, 130), [None, 0, 1, 2, (1, 2), (0, 2), (0, 1)]), ((700, 300), [0, 1]), ((2, 70000), [1])]:
        if dt == np.int32:
            h = rng.integers(-5, 6, size=shape).astype(dt)
        else:
            h = rng.standard_normal(shape).astype(dt)
        d = cls.cast(h)
        for ax in axes:
            got = d.cumsum(axis=ax).to_numpy()
            want = oracle.cum("cumsum", h, axis=ax)
            if dt == np.int32:
                assert_bits_equal(got, want, (shape, ax))
            else:
                axs = tuple(range(h.ndim)) if ax is None else ((ax,) if isinstance(ax, int) else ax)
                n = int(np.prod([shape[a] for a in axs]))
                exact = oracle.cum("cumsum", h.astype(np.float64), axis=ax) if dt == np.float32 else None
                if exact is None:
                    exact = np.asarray(oracle.cum("cumsum", h.astype(np.longdouble).astype(np.float64), axis=ax))
                scale = oracle.cum("cumsum", np.abs(h).astype(np.float64), axis=ax)
                _cum_close(got, exact, scale, n, dt, (shape, ax, "cumsum"))
                # and the oracle's own sequential answer lies within the same bar of it
                _cum_close(want, exact, scale, n, dt, (shape, ax, "oracle cumsum"))
        # views: strided, reversed, transposed
        if len(shape) == 1 and shape[0] > 100:
            for sl in (slice(3, None, 2), slice(None, None, -1), slice(7, shape[0] - 5)):
                got = d[sl].cumsum().to_numpy()
                hv = np.ascontiguousarray(h[sl])
                if dt == np.int32:
                    assert_bits_equal(got, oracle.cum("cumsum", hv), (shape, sl))
                else:
                    _cum_close(got, oracle.cum("cumsum", hv.astype(np.float64)), oracle.cum("cumsum", np.abs(hv).astype(np.float64)), hv.size, dt, (shape, sl))
        if len(shape) == 2:
            got = d.transpose().cumsum(axis=1).to_numpy()
            hv = np.ascontiguousarray(h.T)
            if dt == np.int32:
                assert_bits_equal(got, oracle.cum("cumsum", hv, axis=1))
            else:
                _cum_close(got, oracle.cum("cumsum", hv.astype(np.float64), axis=1), oracle.cum("cumsum", np.abs(hv).astype(np.float64), axis=1),
                           hv.shape[1], dt, (shape, "T"))
    # cumprod: powers of two stay exact in every order
    h = np.where(rng.integers(0, 2, size=(33, 200)) == 0, 2.0, 0.5).astype(dt if dt != np.int32 else np.float32)
    if dt != np.int32:
        assert_bits_equal(cls.cast(h).cumprod(axis=1).to_numpy(), oracle.cum("cumprod", h, axis=1))
        assert_bits_equal(cls.cast(h).cumprod(axis=0).to_numpy(), oracle.cum("cumprod", h, axis=0))
    else:
        hi = rng.integers(-3, 4, size=(33, 40)).astype(np.int32)
        assert_bits_equal(cls.cast(hi).cumprod(axis=1).to_numpy(), oracle.cum("cumprod", hi, axis=1))   # wraps identically


@pytest.mark.parametrize("tname,dt", FLOATS)
def test_cum_nan_forms_on_random_placements(tname, dt):
    cls = cls_of(tname)
    rng = np.random.default_rng(52)
    h = rng.integers(-4, 5, size=(9, 5000)).astype(dt)      # small integers: exact in any order
    h[rng.integers(0, 9, 300), rng.integers(0, 5000, 300)] = np.nan
    h[3, :40] = np.nan                                         # a run that starts with NaN
    h[5, :] = np.nan                                           # and one that is nothing but NaN
    d = cls.cast(h)
    for ax in (1, 0, None):
        assert_bits_equal(d.cumsum(axis=ax, nan=True).to_numpy(), oracle.cum("cumsum", h, axis=ax, nan=True), ("nan", ax))
        assert_bits_equal(d.cumsum(axis=ax).to_numpy(), oracle.cum("cumsum", h, axis=ax), ("plain", ax))


@pytest.mark.parametrize("tname,dt", ALL)
def test_cum_along_contiguous_runs_of_whole_chunks(tname, dt):
    """Many contiguous runs whose length is a whole number of vectors (64 at least) take a kernel
    that scans a run chunk by chunk in registers: one, two, four and eight rows of 256 vectors per
    chunk, one and several chunks per run, the last chunk full or partly there (down to one vector
    past a chunk, and a run of 65 vectors), outer dimensions with padding between the runs.
    Small integers (float sums exact in any order): bit for bit against the sequential scan."""
    cls = cls_of(tname)
    rng = np.random.default_rng(59)
    per = 256 * (16 // np.dtype(dt).itemsize)
    vec = 16 // np.dtype(dt).itemsize
    for shape in [(33, per), (7, 3 * per), (5, 2 * per), (6, 4 * per), (5, 8 * per), (3, 16 * per), (4, 6, 2 * per), (3, 24 * per),
                  (33, per - vec), (7, 3 * per + 5 * vec), (5, 8 * per + vec), (9, 65 * vec), (4, 6, 2 * per - 3 * vec), (3, 13 * per + 77 * vec),
                  (40, 250 * vec), (11, 5 * per - vec), (33, per + 1), (7, 3 * per - 1), (5, 8 * per + vec + 1), (9, 65 * vec + 2 % vec + 1),
                  (4, 6, 2 * per - 3), (20, 4095), (6, 1001)]:
        h = rng.integers(-3, 4, size=shape).astype(dt)
        if dt != np.int32:
            h[..., ::3] = 0
        d = cls.cast(h)
        assert_bits_equal(d.cumsum(axis=-1).to_numpy(), oracle.cum("cumsum", h, axis=len(shape) - 1), (shape, "cumsum"))
        f = rng.choice(np.array([1, -1], dtype=dt), size=shape)
        f.reshape(-1)[rng.integers(0, f.size, 12)] = 2
        assert_bits_equal(cls.cast(f).cumprod(axis=-1).to_numpy(), oracle.cum("cumprod", f, axis=len(shape) - 1), (shape, "cumprod"))
        if dt != np.int32:
            g = h.copy()
            g.reshape(-1)[rng.integers(0, g.size, 200)] = np.nan
            g[0, ..., :700] = np.nan
            d = cls.cast(g)
            assert_bits_equal(d.cumsum(axis=-1, nan=True).to_numpy(), oracle.cum("cumsum", g, axis=len(shape) - 1, nan=True), (shape, "nan: true"))
            assert_bits_equal(d.cumsum(axis=-1).to_numpy(), oracle.cum("cumsum", g, axis=len(shape) - 1), (shape, "NaN carried"))
        if len(shape) == 2:
            # every other run of a wider array: the runs stay contiguous, the step between them doubles
            wide = rng.integers(-3, 4, size=(2 * shape[0], shape[1])).astype(dt)
            hv = np.ascontiguousarray(wide[::2])
            assert_bits_equal(cls.cast(wide)[::2].cumsum(axis=1).to_numpy(), oracle.cum("cumsum", hv, axis=1), (shape, "every other run"))


@pytest.mark.parametrize("tname,dt", ALL)
def test_one_long_run_in_one_pass(tname, dt):
    """Runs from 64 tiles of 64 KiB on are scanned in one pass (four-byte elements: by blocks of
    eight waves with tiles of 128 KiB once there are 64 of those), tiles handing their totals on
    through groups of 64 and supergroups of 64 groups: sizes that end exactly on a group, one
    element past it, the same for the larger tiles, and 4096 small (2048 large) tiles with
    a ragged tail; small integers (float sums
    exact in any order), so every result is compared bit for bit with the sequential scan.
    Then what only the order-free comparison can hold: products of +-1 and 2, NaN skipped
    (the run starts with a tile of nothing but NaN) and carried, a strided view on each side,
    and the same call twice giving the same bits on random floats."""
    cls = cls_of(tname)
    rng = np.random.default_rng(57)
    tile = 65536 // np.dtype(dt).itemsize
    for n in (64 * tile, 64 * tile + 1, 65 * tile + 3001, 128 * tile, 128 * tile + 1, 131 * tile + 77, 64 * 64 * tile + 70001):
        h = rng.integers(-3, 4, size=n).astype(dt)
        if dt != np.int32:
            h[::3] = 0   # keeps the running float sums far below 2^24
        d = cls.cast(h)
        assert_bits_equal(d.cumsum().to_numpy(), oracle.cum("cumsum", h), (n, "cumsum"))
    n = 64 * tile * 3 + 17
    f = rng.choice(np.array([1, -1], dtype=dt), size=n)
    f[rng.integers(0, n, 25)] = 2
    assert_bits_equal(cls.cast(f).cumprod().to_numpy(), oracle.cum("cumprod", f), "cumprod")
    h = rng.integers(-3, 4, size=2 * n).astype(dt)
    hv = np.ascontiguousarray(h[::2])
    assert_bits_equal(cls.cast(h)[::2].cumsum().to_numpy(), oracle.cum("cumsum", hv), "strided input")
    if dt != np.int32:
        g = rng.integers(-3, 4, size=n).astype(dt)
        g[rng.integers(0, n, 3000)] = np.nan
        g[:5000] = np.nan
        d = cls.cast(g)
        assert_bits_equal(d.cumsum(nan=True).to_numpy(), oracle.cum("cumsum", g, nan=True), "nan: true")
        assert_bits_equal(d.cumsum().to_numpy(), oracle.cum("cumsum", g), "NaN carried")
        r = rng.standard_normal(n).astype(dt)
        d = cls.cast(r)
        first = d.cumsum().to_numpy()
        for _ in range(3):
            assert_bits_equal(d.cumsum().to_numpy(), first, "same bits from launch to launch")
        exact = np.cumsum(r.astype(np.float64)) if dt == np.float32 else np.asarray(np.cumsum(r.astype(np.longdouble))).astype(np.float64)
        _cum_close(first, exact, np.cumsum(np.abs(r).astype(np.float64)), n, dt, "random floats")


@pytest.mark.parametrize("tname,dt", ALL)
def test_cum_along_columns_of_tall_wide_and_stacked_arrays(tname, dt):
    """Runs that lie across memory: few segments (the second pass folds their totals
    itself), many (the totals are scanned first, by the same routine), several planes.
    Small integers, so float sums are exact in any order and every result is compared
    bit for bit; products use factors of 1 and -1 and a few 2s."""
    cls = cls_of(tname)
    rng = np.random.default_rng(55)
    for shape, ax in [((70000, 12), 0), ((5000, 2048), 0), ((4, 3000, 64), 1), ((100000, 4), 0), ((3, 40000, 8), 1), ((33000, 1028), 0)]:
        h = rng.integers(-3, 4, size=shape).astype(dt)
        d = cls.cast(h)
        assert_bits_equal(d.cumsum(axis=ax).to_numpy(), oracle.cum("cumsum", h, axis=ax), (shape, "cumsum"))
        f = rng.choice(np.array([1, -1], dtype=dt), size=shape)
        f[tuple(rng.integers(0, n, 20) for n in shape)] = 2
        assert_bits_equal(cls.cast(f).cumprod(axis=ax).to_numpy(), oracle.cum("cumprod", f, axis=ax), (shape, "cumprod"))
        if dt != np.int32:
            h[tuple(rng.integers(0, n, 500) for n in shape)] = np.nan
            if len(shape) == 2:
                h[:50] = np.nan                                    # every run starts with NaN
            d = cls.cast(h)
            assert_bits_equal(d.cumsum(axis=ax, nan=True).to_numpy(), oracle.cum("cumsum", h, axis=ax, nan=True), (shape, "nan: true"))
            assert_bits_equal(d.cumsum(axis=ax).to_numpy(), oracle.cum("cumsum", h, axis=ax), (shape, "NaN carried"))
        # a view: every other column, rows reversed
        if len(shape) == 2 and shape[1] >= 8:
            hb = h if dt == np.int32 else np.nan_to_num(h)
            hv = np.ascontiguousarray(hb[::-1, ::2])
            assert_bits_equal(cls.cast(hb).reverse(0)[:, ::2].cumsum(axis=0).to_numpy(), oracle.cum("cumsum", hv, axis=0), (shape, "view"))


@pytest.mark.parametrize("tname,dt", ALL)
def test_long_columns_in_one_pass(tname, dt):
    """Runs across memory whose matrix cuts into at least 16 tiles of 256 rows by 64 vectors are
    scanned in one pass: tiles publish their column totals and gather what lies above them through
    groups of 8 tiles and supergroups of 8 groups. Depths of 70 tiles (two supergroups), 35 tiles
    in four planes and 8 tiles (one group, closed by the last tile); tiles at the lower and right
    edges that are only partly there (845 rows by two strips and three vectors; three planes of
    1000 rows by a strip and a vector). Small integers (float sums
    exact in any order): bit for bit against the sequential scan; products of +-1 and a few 2s;
    NaN skipped (every run starts with more than a tile of NaN) and carried; every other row of a
    taller array; random floats give the same bits from launch to launch and stay close."""
    cls = cls_of(tname)
    rng = np.random.default_rng(61)
    sw = 64 * (16 // np.dtype(dt).itemsize)
    vec = 16 // np.dtype(dt).itemsize
    for shape, ax in [((256 * 70, 4 * sw), 0), ((4, 256 * 35, 2 * sw), 1), ((256 * 8, 32 * sw), 0), ((256 * 9, 2 * sw), 0), ((512, 8 * sw), 0),
                      ((256 * 3 + 77, 6 * sw + 3 * vec), 0), ((3, 1000, 2 * sw + vec), 1), ((257, 16 * sw), 0),
                      ((256 * 3 + 5, 6 * sw + 1), 0), ((1000, 4095), 0), ((3, 700, 2 * sw + vec + 1), 1)]:
        h = rng.integers(-3, 4, size=shape).astype(dt)
        if dt != np.int32:
            h[..., ::3] = 0
        d = cls.cast(h)
        assert_bits_equal(d.cumsum(axis=ax).to_numpy(), oracle.cum("cumsum", h, axis=ax), (shape, "cumsum"))
        f = rng.choice(np.array([1, -1], dtype=dt), size=shape)
        f[tuple(rng.integers(0, n, 40) for n in shape)] = 2
        assert_bits_equal(cls.cast(f).cumprod(axis=ax).to_numpy(), oracle.cum("cumprod", f, axis=ax), (shape, "cumprod"))
        if dt != np.int32:
            g = h.copy()
            g[tuple(rng.integers(0, n, 3000) for n in shape)] = np.nan
            if len(shape) == 2:
                g[:300] = np.nan
            else:
                g[:, :300] = np.nan
            d = cls.cast(g)
            assert_bits_equal(d.cumsum(axis=ax, nan=True).to_numpy(), oracle.cum("cumsum", g, axis=ax, nan=True), (shape, "nan: true"))
            assert_bits_equal(d.cumsum(axis=ax).to_numpy(), oracle.cum("cumsum", g, axis=ax), (shape, "NaN carried"))
        del d
    shape = (256 * 16, 16 * sw)
    wide = rng.integers(-3, 4, size=(2 * shape[0], shape[1])).astype(dt)
    hv = np.ascontiguousarray(wide[::2])
    assert_bits_equal(cls.cast(wide)[::2].cumsum(axis=0).to_numpy(), oracle.cum("cumsum", hv, axis=0), "every other row")
    if dt != np.int32:
        r = rng.standard_normal(shape).astype(dt)
        d = cls.cast(r)
        first = d.cumsum(axis=0).to_numpy()
        for _ in range(3):
            assert_bits_equal(d.cumsum(axis=0).to_numpy(), first, "same bits from launch to launch")
        exact = np.cumsum(r.astype(np.float64), axis=0) if dt == np.float32 else np.asarray(np.cumsum(r.astype(np.longdouble), axis=0)).astype(np.float64)
        _cum_close(first, exact, np.cumsum(np.abs(r).astype(np.float64), axis=0), shape[0], dt, "random floats")


@pytest.mark.parametrize("tname,dt", ALL)
def test_mulsum_parity(tname, dt):
    cls = cls_of(tname)
    rng = np.random.default_rng(53)

    def make(shape):
        if dt == np.int32:
            return rng.integers(-1000, 1000, size=shape).astype(dt)
        return rng.standard_normal(shape).astype(dt)

    def check(got, hx, hy, axis, what, nan=False):
        want = np.asarray(oracle.mulsum(hx, hy, axis=axis, nan=nan))
        got = np.asarray(got)
        assert got.shape == want.shape, (what, got.shape, want.shape)
        if dt == np.int32:
            assert_bits_equal(got.astype(np.int32), want.astype(np.int32), what)
            return
        bx = np.broadcast_to(hx, np.broadcast_shapes(hx.shape, hy.shape)).astype(np.float64)
        by = np.broadcast_to(hy, bx.shape).astype(np.float64)
        if nan:
            ok = ~(np.isnan(bx) | np.isnan(by))
            bx, by = np.where(ok, bx, 0), np.where(ok, by, 0)
        exact = (bx * by).sum(axis=axis)
        scale = np.abs(bx * by).sum(axis=axis)
        n = bx.size // max(1, np.asarray(exact).size)
        tol = (1e-5 if dt == np.float32 else 1e-12) * max(1.0, np.log2(max(n, 2)))
        assert (np.abs(got.astype(np.float64) - exact) <= tol * np.maximum(scale, 1e-300)).all(), what
        assert (np.abs(want.astype(np.float64) - exact) <= tol * np.maximum(scale, 1e-300) * 4).all(), (what, "oracle")

    for n in (1, 7, 1000, 4096, 100003, (1 << 22) + 3):
        hx, hy = make((n,)), make((n,))
        x, y = cls.cast(hx), cls.cast(hy)
        check(x.mulsum(y).to_numpy(), hx, hy, None, ("dot", n))
        if n > 100:
            check(x[1::2].mulsum(y[:n // 2]).to_numpy(), np.ascontiguousarray(hx[1::2]), np.ascontiguousarray(hy[:n // 2]), None, ("strided dot", n))
            check(x[::-1].mulsum(y).to_numpy(), np.ascontiguousarray(hx[::-1]), hy, None, ("reversed dot", n))
    hx, hy = make((37, 65)), make((37, 65))
    x, y = cls.cast(hx), cls.cast(hy)
    for ax in (None, 0, 1, -1):
        check(x.mulsum(y, axis=ax).to_numpy(), hx, hy, ax, ("matrix", ax))
    check(x.mulsum(y[0], axis=1).to_numpy(), hx, hy[0], 1, "row vector operand")
    check(x.transpose().mulsum(y.transpose(), axis=0).to_numpy(), np.ascontiguousarray(hx.T), np.ascontiguousarray(hy.T), 0, "transposed")
    assert x.mulsum(y, axis=1, keepdims=True).to_numpy().shape == (37, 1)
    # more inner runs than are launched one by one: the products go through the reduction engine
    hx, hy = make((3000, 40)), make((3000, 40))
    check(cls.cast(hx).mulsum(cls.cast(hy), axis=1).to_numpy(), hx, hy, 1, "3000 runs")
    # every row in one launch: 16, 64 and 256 lanes per row, a repeated row operand, rows a step apart
    # (and rows that end in part of a 128-bit vector, which also start off a 16-byte boundary)
    for shape in ((5000, 8), (700, 512), (300, 4096), (64, 20000), (3, 1 << 16), (300, 4095), (700, 131), (64, 20001), (50, 67), (10, 4094)):
        hx, hy = make(shape), make(shape)
        x, y = cls.cast(hx), cls.cast(hy)
        check(x.mulsum(y, axis=1).to_numpy(), hx, hy, 1, ("rows", shape))
        check(x.mulsum(y[0], axis=-1).to_numpy(), hx, hy[0], 1, ("rows, one operand repeated", shape))
        check(x[::2].mulsum(y[1::2], axis=1).to_numpy(), np.ascontiguousarray(hx[::2]), np.ascontiguousarray(hy[1::2]), 1, ("every other row", shape))
    hx, hy = make((6, 50, 128)), make((6, 50, 128))
    check(cls.cast(hx).mulsum(cls.cast(hy), axis=2).to_numpy(), hx, hy, 2, "rows over two outer dimensions")
    check(cls.cast(hx).mulsum(cls.cast(hy), axis=(1, 2)).to_numpy(), hx, hy, (1, 2), "two reduced dimensions as one run")
    # no reduced dimension left after broadcasting rules: the elementwise form
    hx, hy = make((5, 1)), make((5, 1))
    check(cls.cast(hx).mulsum(cls.cast(hy), axis=1).to_numpy(), hx, hy, 1, "runs of one element")
    if dt != np.int32:
        hx, hy = make((4, 5000)), make((4, 5000))
        hx[rng.integers(0, 4, 50), rng.integers(0, 5000, 50)] = np.nan
        hy[rng.integers(0, 4, 50), rng.integers(0, 5000, 50)] = np.nan
        check(cls.cast(hx).mulsum(cls.cast(hy), axis=1, nan=True).to_numpy(), hx, hy, 1, "nan: true", nan=True)
        assert np.isnan(cls.cast(hx).mulsum(cls.cast(hy), axis=1).to_numpy()).all()
    # mixed types move to the higher one
    import cumo_amd
    r = cumo_amd.Int32.cast(np.array([1, 2, 3], dtype=np.int32)).mulsum(cumo_amd.DFloat.cast(np.array([0.5, 0.25, 2.0])))
    assert isinstance(r, cumo_amd.DFloat) and float(r) == 0.5 + 0.5 + 6.0


def test_cum_and_mulsum_launchers_called_directly():
    """The reference's per-run symbols: narray/gen/tmpl/cum.c:3, accum_binary.c:4-5."""
    import ctypes as C
    from cumo_amd import _lib
    from test_gpu_raw_abi import dev, fetch, free
    rng = np.random.default_rng(54)
    n = 50001
    h = rng.integers(-3, 4, size=2 * n + 5).astype(np.float32)
    px = dev(h)
    pz = dev(np.full(n, -7.0, dtype=np.float32))
    f = _lib.fn("cumo_sfloat_cumsum_kernel_launch", C.c_int, [C.c_void_p, C.c_void_p, C.c_ssize_t, C.c_ssize_t, C.c_uint64])
    # every other element, starting at element 3, written backwards
    rc = _lib.call(f, px + 12, pz + 4 * (n - 1), 8, -4, n)
    assert rc == 0
    got = fetch(pz, (n,), np.float32)
    assert_bits_equal(got[::-1], np.cumsum(h[3:3 + 2 * n:2].astype(np.float64)).astype(np.float32))
    # mulsum adds onto what the result holds
    py = dev(np.full(n, 2.0, dtype=np.float32))
    pacc = dev(np.array([100.0], dtype=np.float32))
    g = _lib.fn("cumo_sfloat_mulsum_reduce_kernel_launch", None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_ssize_t, C.c_ssize_t, C.c_uint64])
    _lib.call(g, px + 12, py, pacc, 8, 4, n)
    assert float(fetch(pacc, (1,), np.float32)[0]) == 100.0 + 2.0 * float(h[3:3 + 2 * n:2].astype(np.float64).sum())
    _lib.call(g, px, py, pacc, 4, 0, 0)                       # an empty run adds nothing
    assert float(fetch(pacc, (1,), np.float32)[0]) == 100.0 + 2.0 * float(h[3:3 + 2 * n:2].astype(np.float64).sum())
    free(px, py, pz, pacc)
