"""Recorded chains of operations replayed as one graph: every replay must give exactly
what the same operations give when launched one by one (same kernels, same order of
summation: bit-exact), also when the inputs change between replays and when ordinary
launches and synchronisations happen in between."""
import numpy as np
import pytest

from helpers import assert_bits_equal

pytestmark = pytest.mark.gpu


def eager_c1(cumo, x, b):
    t = 2.5 * x
    y = t + b
    return t, y, y.sum()


@pytest.mark.parametrize("n", [1000, 1 << 20, (1 << 22) + 3])
def test_axpy_and_sum_chain_replayed_with_changing_inputs(n):
    import cumo_amd as cumo
    rng = np.random.default_rng(n)
    x = cumo.SFloat.cast(rng.uniform(-1, 1, n).astype(np.float32))
    b = cumo.SFloat.cast(rng.uniform(-1, 1, n).astype(np.float32))
    eager_c1(cumo, x, b)  # the pool has seen these sizes
    with cumo.Graph() as g:
        t, y, s = eager_c1(cumo, x, b)
    assert g.nodes >= 3
    for k in range(5):
        if k:
            # ordinary launches and a synchronisation between the replays; new inputs
            x.store(cumo.SFloat.cast(rng.uniform(-1, 1, n).astype(np.float32)))
            (x * 0.5).sum().extract_cpu()
        g.launch()
        et, ey, es = eager_c1(cumo, x, b)
        assert_bits_equal(t.to_numpy(), et.to_numpy(), ("t", k))
        assert_bits_equal(y.to_numpy(), ey.to_numpy(), ("y", k))
        assert_bits_equal(s.to_numpy(), es.to_numpy(), ("s", k))
    g.launch(3)  # back to back
    assert_bits_equal(s.to_numpy(), eager_c1(cumo, x, b)[2].to_numpy())
    g.close()


def chain_mixed(cumo, S, X, M, I):
    NM = cumo.NMath
    m = S.max(axis=-1, keepdims=True)
    e = NM.exp(S - m)
    p = e / e.sum(axis=-1, keepdims=True)
    ln = (X - X.mean(axis=-1, keepdims=True)) / NM.sqrt(X.var(axis=-1, keepdims=True) + 1e-5)
    V = M.transpose()[:, ::2]
    E = NM.exp(V) - 1.0
    mask = (E > 0.5) & ~(E > 2.0)
    cs = X.cumsum(axis=1)
    dot = X.mulsum(X, axis=1)
    big = X.sum()
    am = S.argmax(axis=-1)
    ic = I[::3].copy()
    f = cumo.Fused.softmax(S)
    return [p, ln, E, mask, cs, dot, big, am, ic, f]


def test_mixed_chain_of_every_kernel_family():
    import cumo_amd as cumo
    rng = np.random.default_rng(3)
    S = cumo.SFloat.cast(rng.standard_normal((4, 64, 512)).astype(np.float32))
    X = cumo.SFloat.cast(rng.standard_normal((1024, 4096)).astype(np.float32))   # 16 MiB: two-pass full sum
    M = cumo.SFloat.cast(rng.standard_normal((512, 384)).astype(np.float32))
    I = cumo.Int32.cast(rng.integers(0, 1000, (300, 200)).astype(np.int32))
    want = [r.to_numpy() for r in chain_mixed(cumo, S, X, M, I)]
    used_before = cumo.MemoryPool.used_bytes()
    with cumo.Graph() as g:
        got = chain_mixed(cumo, S, X, M, I)
    # intermediates released inside the block stay reserved for the graph
    pooled = cumo.MemoryPool.enabled()   # with CUMO_MEMORY_POOL=OFF the pool's counters stay at 0
    if pooled:
        assert cumo.MemoryPool.used_bytes() > used_before + sum(r._buf.nbytes for r in got)
    for k in range(3):
        g.launch()
        for i, (r, w) in enumerate(zip(got, want)):
            assert_bits_equal(r.to_numpy(), w, ("replay", k, "result", i))
        # scribble over the results with ordinary launches, so that a replay that did nothing would show
        for r in got:
            if isinstance(r, (cumo.SFloat, cumo.Int32)):
                r.fill(7)
        cumo.synchronize()
    held = cumo.MemoryPool.used_bytes()
    g.close()
    if pooled:
        assert cumo.MemoryPool.used_bytes() < held
    # the same operations still run one by one afterwards
    again = [r.to_numpy() for r in chain_mixed(cumo, S, X, M, I)]
    for a, w in zip(again, want):
        assert_bits_equal(a, w)


def test_operation_that_needs_the_host_ends_the_capture_with_an_error():
    import cumo_amd as cumo
    x = cumo.SFloat.cast(np.arange(100, dtype=np.float32))
    with pytest.raises(Exception):
        with cumo.Graph() as g:
            y = x + 1.0
            y.to_numpy()  # a read-back cannot be recorded
    assert g.nodes == 0
    with pytest.raises(ValueError):
        g.launch()
    # the library is usable afterwards, eagerly and recorded
    assert (x + 1.0).to_numpy()[5] == 6.0
    with cumo.Graph() as g2:
        z = x * 2.0
    g2.launch()
    assert z.to_numpy()[7] == 14.0
    # no second capture inside an open one
    with pytest.raises(ValueError):
        with cumo.Graph():
            with cumo.Graph():
                pass
    assert (x + 2.0).to_numpy()[1] == 3.0
