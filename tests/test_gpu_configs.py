"""The five benchmark configurations at their full sizes, on the same seeded
inputs bench.py uses. Where the CPU oracle finishes in seconds it is the
expected value; beyond that the checks are what the arithmetic fixes without it:
a single IEEE operation equals numpy's bit for bit, sums of multiples of 1/16
are exact in any order, softmax rows sum to one, max/argmax agree with a direct
scan, and float reductions sit within the stated tolerance of the exact value.

Tolerances (written out): elementwise float <= 1 ulp (0 ulp for single IEEE
operations); float reductions rel 1e-5*log2(n) for SFloat and 1e-12*log2(n) for
DFloat, relative to sum(|x|); everything integer, Bit or index is bit-exact."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, ROOT)
import numo_oracle as oracle  # noqa: E402

import bench  # noqa: E402  (only its seeded input generators)
from helpers import assert_bits_equal, assert_reduction_close, assert_ulp  # noqa: E402

pytestmark = pytest.mark.gpu


def exact_sum(h, axis=None, keepdims=False):
    return np.asarray(h.astype(np.longdouble).sum(axis=axis, keepdims=keepdims), dtype=np.float64)


def abs_sum(h, axis=None, keepdims=False):
    return np.abs(h.astype(np.float64)).sum(axis=axis, keepdims=keepdims)


@pytest.mark.parametrize("n", [1 << 20, 1 << 26])
def test_c1_axpy_and_full_sum(n):
    import cumo_amd
    h = bench.inputs_c1(n)
    x, b = cumo_amd.SFloat.cast(h["x"]), cumo_amd.SFloat.cast(h["b"])
    t = 2.5 * x
    y = t + b
    s = y.sum()
    ht = np.float32(2.5) * h["x"]
    hy = ht + h["b"]
    assert_bits_equal(t.to_numpy(), ht, "2.5*x")
    assert_bits_equal(y.to_numpy(), hy, "t+b")
    if n <= 1 << 20:  # the oracle's Numo-shaped loops on the reference's own CPU-runnable case
        assert_bits_equal(oracle.binary("add", oracle.binary("mul", 2.5, h["x"], scalar_is_left=True), h["b"]), hy, "oracle axpy")
        o = float(oracle.reduce("sum", hy))
        assert abs(o - float(exact_sum(hy))) <= 2 * n * 2.0 ** -24 * float(abs_sum(hy))
    assert_reduction_close(np.float32(float(s)), np.float32(exact_sum(hy)), n, scale=abs_sum(hy), what="y.sum")
    assert s.shape == () and type(s) is cumo_amd.SFloat


def test_c2_broadcast_add_and_row_reductions():
    import cumo_amd
    h = bench.inputs_c2()
    a, r = cumo_amd.DFloat.cast(h["A"]), cumo_amd.DFloat.cast(h["r"])
    c = a + r
    hc = oracle.binary("add", h["A"], h["r"])
    assert_bits_equal(hc, h["A"] + h["r"], "oracle vs IEEE")
    assert_bits_equal(c.to_numpy(), hc, "A+r")
    n = hc.shape[1]
    got = c.sum(axis=1).to_numpy()
    assert got.shape == (n,)
    assert_reduction_close(got, exact_sum(hc, axis=1), n, scale=abs_sum(hc, axis=1), what="C.sum(axis:1)")
    osum = oracle.reduce("sum", hc, axis=1)
    assert (np.abs(osum - exact_sum(hc, axis=1)) <= 2 * n * 2.0 ** -53 * abs_sum(hc, axis=1)).all()
    assert_bits_equal(c.max(axis=1).to_numpy(), oracle.reduce("max", hc, axis=1), "C.max(axis:1)")
    assert_bits_equal(oracle.reduce("max", hc, axis=1), hc.max(axis=1), "oracle max vs scan")


def test_c3_axis_reductions_with_ties():
    import cumo_amd
    h = bench.inputs_c3()["T"]
    t = cumo_amd.SFloat.cast(h)
    h64 = h.astype(np.float64)
    # multiples of 1/16 below 4 in magnitude: partial sums over 64 or 1024 of them are
    # exact in float32 whatever the order, so the axis sums must equal the exact sums
    for axis in (0, 2):
        want = h64.sum(axis=axis).astype(np.float32)
        assert_bits_equal(t.sum(axis=axis).to_numpy(), want, "sum axis %d" % axis)
        assert_bits_equal(t.mean(axis=axis).to_numpy(), (h64.sum(axis=axis) / h.shape[axis]).astype(np.float32), "mean axis %d" % axis)
        assert_bits_equal(t.max(axis=axis).to_numpy(), h.max(axis=axis), "max axis %d" % axis)
        assert_bits_equal(t.min(axis=axis).to_numpy(), h.min(axis=axis), "min axis %d" % axis)
    assert_bits_equal(oracle.reduce("sum", h, axis=2), h64.sum(axis=2).astype(np.float32), "oracle sum axis 2")
    n = h.size
    assert_reduction_close(np.float32(float(t.sum())), np.float32(h64.sum()), n, scale=np.abs(h64).sum(), what="sum()")
    assert_reduction_close(np.float32(float(t.mean())), np.float32(h64.mean()), n, scale=np.abs(h64).mean(), what="mean()")
    assert float(t.max()) == float(h.max()) and float(t.min()) == float(h.min())
    # lowest index wins ties (numpy's argmax/argmin scan has the same rule; so has the oracle)
    amax, amin = t.argmax(axis=2), t.argmin(axis=2)
    assert type(amax) is cumo_amd.Int32
    assert_bits_equal(amax.to_numpy(), h.argmax(axis=2).astype(np.int32), "argmax axis 2")
    assert_bits_equal(amin.to_numpy(), h.argmin(axis=2).astype(np.int32), "argmin axis 2")
    assert_bits_equal(oracle.reduce("argmax", h, axis=2).astype(np.int32), h.argmax(axis=2).astype(np.int32), "oracle argmax")
    ties = (h == h.max(axis=2, keepdims=True)).sum(axis=2)
    assert (ties > 1).mean() > 0.5, "the input is meant to force ties"


def test_c4_strided_transposed_views():
    import cumo_amd
    h = bench.inputs_c4()
    m, i = cumo_amd.SFloat.cast(h["M"]), cumo_amd.Int32.cast(h["I"])
    v = m.transpose()[:, ::2]
    hv = h["M"].transpose()[:, ::2]
    assert v.shape == hv.shape == (8192, 4096)
    e0 = cumo_amd.NMath.exp(v)
    assert e0.is_contiguous()
    g0 = e0.to_numpy()
    # Numo's SFloat exp is (float)exp((double)x) (types/float_macro.h:84-97): the oracle restates it
    assert_ulp(g0, oracle.unary("exp", np.ascontiguousarray(hv)), 1, "exp(V)")
    assert_ulp(g0, np.exp(hv.astype(np.float64)).astype(np.float32), 1, "exp(V) vs float64 exp rounded once")
    e = e0 - 1.0
    g = e.to_numpy()
    assert_bits_equal(g, g0 - np.float32(1.0), "E0 - 1.0")
    mask = e > 0.5
    assert type(mask) is cumo_amd.Bit
    hm = (g > np.float32(0.5)).astype(np.uint8)
    assert_bits_equal(mask.to_numpy(), hm, "E > 0.5")
    cnt = mask.count_true()
    assert int(cnt) == int(hm.sum()) and type(cnt) is cumo_amd.UInt64
    assert int(mask.count_false()) == hm.size - int(hm.sum())
    rows = mask.count_true(axis=1).to_numpy()
    assert_bits_equal(rows, hm.sum(axis=1).astype(np.uint64), "count_true(axis:1)")
    ic = i[::3].copy()
    assert ic.is_contiguous() and ic.shape == (2731, 8192)
    assert_bits_equal(ic.to_numpy(), h["I"][::3], "I[(0..-1).step(3), true].copy")
    assert_bits_equal(oracle.copy(h["I"][::3]), np.ascontiguousarray(h["I"][::3]), "oracle copy")


def test_c5_softmax_from_array_ops():
    import cumo_amd
    hs = bench.inputs_c5()["S"]
    s = cumo_amd.SFloat.cast(hs)
    n = hs.shape[-1]
    m = s.max(axis=-1, keepdims=True)
    assert m.shape == hs.shape[:-1] + (1,)
    hm = hs.max(axis=-1, keepdims=True)
    assert_bits_equal(m.to_numpy(), hm, "max(axis:-1, keepdims)")
    d = s - m
    hd = hs - hm
    assert_bits_equal(d.to_numpy(), hd, "S - m")
    e = cumo_amd.NMath.exp(d)
    ge = e.to_numpy()
    assert_ulp(ge, np.exp(hd.astype(np.float64)).astype(np.float32), 1, "exp(S - m)")
    z = e.sum(axis=-1, keepdims=True)
    gz = z.to_numpy()
    assert_reduction_close(gz, exact_sum(ge, axis=-1, keepdims=True).astype(np.float32), n, what="e.sum(axis:-1)")
    p = e / z
    gp = p.to_numpy()
    assert_bits_equal(gp, ge / gz, "e / z")
    # properties the arithmetic fixes: rows sum to one, nothing negative, the largest input has probability
    # exp(0)/z
    rows = gp.astype(np.float64).sum(axis=-1)
    assert np.abs(rows - 1.0).max() <= 1e-5 * np.log2(n)
    assert gp.min() >= 0.0
    assert_bits_equal(gp.max(axis=-1, keepdims=True), np.float32(1.0) / gz, "p at the row maximum")
    del s, m, d, e, z, p


def test_c5_layernorm_statistics_from_array_ops():
    import cumo_amd
    hx = bench.inputs_c5()["X"]
    x = cumo_amd.SFloat.cast(hx)
    n = hx.shape[-1]
    mean = x.mean(axis=-1, keepdims=True)
    var = x.var(axis=-1, keepdims=True)
    x64 = hx.astype(np.longdouble)
    gm, gv = mean.to_numpy(), var.to_numpy()
    assert gm.shape == gv.shape == (hx.shape[0], 1)
    assert_reduction_close(gm, np.asarray(x64.mean(axis=-1, keepdims=True), dtype=np.float64).astype(np.float32), n,
                           scale=abs_sum(hx, axis=-1, keepdims=True) / n, what="mean")
    # Numo's var divides by n-1 (types/real_accum.h:114-131)
    assert_reduction_close(gv, np.asarray(x64.var(axis=-1, keepdims=True, ddof=1), dtype=np.float64).astype(np.float32), n, what="var")
    c = x - mean
    gc = c.to_numpy()
    assert_bits_equal(gc, hx - gm, "X - mean")
    v = var + 1e-5
    assert_bits_equal(v.to_numpy(), gv + np.float32(1e-5), "var + 1e-5")
    sd = cumo_amd.NMath.sqrt(v)
    gsd = sd.to_numpy()
    assert_bits_equal(gsd, np.sqrt(gv + np.float32(1e-5)), "sqrt")
    out = c / sd
    go = out.to_numpy()
    assert_bits_equal(go, gc / gsd, "(X - mean) / sqrt(var + 1e-5)")
    # the normalised rows have mean ~0 and variance ~1
    assert np.abs(go.astype(np.float64).mean(axis=-1)).max() < 1e-5
    assert np.abs(go.astype(np.float64).var(axis=-1, ddof=1) - 1.0).max() < 1e-3


def test_small_configs_match_the_oracle_op_for_op():
    """The same five chains at sizes the oracle walks in milliseconds, every step
    against the oracle on the device's own previous result."""
    import cumo_amd
    rng = np.random.default_rng(77)
    # C2 shape family
    a, r = rng.standard_normal((37, 53)), rng.standard_normal((1, 53))
    c = cumo_amd.DFloat.cast(a) + cumo_amd.DFloat.cast(r)
    hc = oracle.binary("add", a, r)
    assert_bits_equal(c.to_numpy(), hc)
    assert_reduction_close(c.sum(axis=1).to_numpy(), oracle.reduce("sum", hc, axis=1), 53, scale=abs_sum(hc, axis=1))
    assert_bits_equal(c.max(axis=1).to_numpy(), oracle.reduce("max", hc, axis=1))
    # C4 shape family
    m = rng.standard_normal((66, 70), dtype=np.float32)
    hv = np.ascontiguousarray(m.transpose()[:, ::2])
    e0 = cumo_amd.NMath.exp(cumo_amd.SFloat.cast(m).transpose()[:, ::2])
    assert_ulp(e0.to_numpy(), oracle.unary("exp", hv), 1)
    g0 = e0.to_numpy()
    e = e0 - 1.0
    assert_bits_equal(e.to_numpy(), oracle.binary("sub", g0, 1.0))
    mask = e > 0.5
    want = oracle.compare("gt", e.to_numpy(), 0.5)
    assert (mask.to_numpy() == want).all()
    assert int(mask.count_true()) == oracle.bit_count(oracle.pack(want), 0, 1, want.size)
    # C5 shape family
    s = (rng.standard_normal((3, 5, 17), dtype=np.float32) * np.float32(2))
    ds = cumo_amd.SFloat.cast(s)
    dm = ds.max(axis=-1, keepdims=True)
    assert_bits_equal(dm.to_numpy(), oracle.reduce("max", s, axis=-1, keepdims=True))
    dd = ds - dm
    assert_bits_equal(dd.to_numpy(), oracle.binary("sub", s, dm.to_numpy()))
    de = cumo_amd.NMath.exp(dd)
    assert_ulp(de.to_numpy(), oracle.unary("exp", dd.to_numpy()), 1)
    dz = de.sum(axis=-1, keepdims=True)
    assert_reduction_close(dz.to_numpy(), oracle.reduce("sum", de.to_numpy(), axis=-1, keepdims=True), 17)
    assert_bits_equal((de / dz).to_numpy(), oracle.binary("div", de.to_numpy(), dz.to_numpy()))
    x = rng.standard_normal((9, 33), dtype=np.float32)
    dx = cumo_amd.SFloat.cast(x)
    assert_reduction_close(dx.var(axis=-1, keepdims=True).to_numpy(), oracle.reduce("var", x, axis=-1, keepdims=True), 33)
    assert_reduction_close(dx.mean(axis=-1, keepdims=True).to_numpy(), oracle.reduce("mean", x, axis=-1, keepdims=True), 33,
                           scale=abs_sum(x, axis=-1, keepdims=True) / 33)
