"""softmax and layernorm along the last dimension: the one-launch form against the
chain of array operations it stands for (run on the device) and against the same
chain on the CPU oracle. Elementwise steps are identical in both; the two row
sums associate differently, so the bar is the float-reduction bar of the parity
contract carried through the division: rel 1e-5*log2(n) SFloat, 1e-12*log2(n)
DFloat."""
import numpy as np
import pytest

import kat_adjacent as K

pytestmark = pytest.mark.gpu
oracle = K.OracleEngine().o


def chain_softmax(m, x):
    mx = x.max(axis=-1, keepdims=True)
    e = m.NMath.exp(x - mx)
    return e / e.sum(axis=-1, keepdims=True)


def chain_layernorm(m, x, eps):
    return (x - x.mean(axis=-1, keepdims=True)) / m.NMath.sqrt(x.var(axis=-1, keepdims=True) + eps)


def oracle_softmax(h):
    mx = oracle.reduce("max", h, axis=h.ndim - 1, keepdims=True)
    e = oracle.unary("exp", oracle.binary("sub", h, np.ascontiguousarray(np.broadcast_to(mx, h.shape))))
    s = oracle.reduce("sum", e, axis=h.ndim - 1, keepdims=True)
    return oracle.binary("div", e, np.ascontiguousarray(np.broadcast_to(s, h.shape)))


def close(got, want, n, dt, what):
    tol = (1e-5 if dt == np.float32 else 1e-12) * max(1.0, np.log2(max(n, 2)))
    g, w = got.astype(np.float64), want.astype(np.float64)
    nan = np.isnan(w)
    assert (np.isnan(g) == nan).all(), what
    err = np.abs(g - w)[~nan]
    bound = tol * np.maximum(np.abs(w[~nan]), 1e-30) + tol * 1e-3
    assert (err <= bound).all(), (what, float(err.max()))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_softmax_matches_the_chain(dt):
    import cumo_amd as m
    cls = m.SFloat if dt == np.float32 else m.DFloat
    rng = np.random.default_rng(61)
    # (rows that end in part of a 128-bit vector, and so start off a 16-byte boundary: 1001, 4095, 13, 131, 7)
    for shape in [(1, 4), (5, 8), (33, 64), (100, 512), (7, 1000), (3, 4, 2048), (9, 4096), (2, 16384), (4, 20000), (6, 7), (2, 3, 5, 128),
                  (7, 1001), (37, 4095), (50, 13), (19, 131), (3, 16383), (5, 4094)]:
        h = (rng.standard_normal(shape) * 2).astype(dt)
        x = cls.cast(h)
        got = m.Fused.softmax(x).to_numpy()
        n = shape[-1]
        close(got, chain_softmax(m, x).to_numpy(), n, dt, (shape, "device chain"))
        if np.prod(shape) <= 200000:
            close(got, oracle_softmax(h), n, dt, (shape, "oracle chain"))
        assert np.allclose(got.astype(np.float64).sum(axis=-1), 1.0, rtol=0, atol=1e-5 if dt == np.float32 else 1e-12)
    # rows that are views: every other row, and a column window that stays 16-byte aligned
    h = (rng.standard_normal((40, 256)) * 2).astype(dt)
    x = cls.cast(h)
    for key in ((slice(None, None, 2), slice(None)), (slice(3, 30), slice(64, 192)), (slice(None), slice(1, 200)), (slice(None), slice(None, None, 2))):
        close(m.Fused.softmax(x[key]).to_numpy(), chain_softmax(m, x[key]).to_numpy(), h[key].shape[-1], dt, key)
    # special values: a NaN poisons its row, -inf entries get weight 0, a row of equal values is uniform
    h = np.zeros((4, 64), dtype=dt)
    h[0, 5] = np.nan
    h[1, :] = -np.inf
    h[1, 7] = 3.0
    h[2, :] = 7.5
    h[3, :] = rng.standard_normal(64)
    got = m.Fused.softmax(cls.cast(h)).to_numpy()
    want = chain_softmax(m, cls.cast(h)).to_numpy()
    assert np.isnan(got[0]).all() and np.isnan(want[0]).all()
    assert got[1, 7] == 1.0 and (np.delete(got[1], 7) == 0).all()
    assert (got[2] == dt(1.0) / dt(64.0)).all()
    close(got[3:], want[3:], 64, dt, "ordinary row")


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_layernorm_matches_the_chain(dt):
    import cumo_amd as m
    cls = m.SFloat if dt == np.float32 else m.DFloat
    rng = np.random.default_rng(62)
    for shape in [(3, 4), (5, 8), (33, 64), (100, 512), (7, 1000), (64, 4096), (3, 16384), (4, 20000), (6, 7), (2, 3, 128),
                  (7, 1001), (37, 4095), (50, 13), (19, 131), (3, 16383), (5, 4094)]:
        h = (rng.standard_normal(shape) * 3 + 1).astype(dt)
        x = cls.cast(h)
        got = m.Fused.layernorm(x, 1e-5).to_numpy()
        want = chain_layernorm(m, x, 1e-5).to_numpy()
        n = shape[-1]
        # the chain's own var is one-pass (Chan); both lie within the bar of the exact statistics
        hd = h.astype(np.float64)
        exact = (hd - hd.mean(axis=-1, keepdims=True)) / np.sqrt(hd.var(axis=-1, ddof=1, keepdims=True) + dt(1e-5))
        tol = (1e-5 if dt == np.float32 else 1e-12) * max(1.0, np.log2(n))
        assert np.abs(got - exact).max() <= tol * 8, (shape, float(np.abs(got - exact).max()))
        assert np.abs(want - exact).max() <= tol * 8, (shape, "chain")
    # a row of one element has no variance: NaN from both
    one = cls.cast(np.array([[2.0], [3.0]], dtype=dt))
    assert np.isnan(m.Fused.layernorm(one).to_numpy()).all() and np.isnan(chain_layernorm(m, one, 1e-5).to_numpy()).all()
