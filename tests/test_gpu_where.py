"""Bit#where / where2 / mask: compaction of bit positions on the device against
the oracle's where / mask on the same bits (integer work: bit-exact), over contiguous
arrays, views that start inside a word, strided and reversed views, and through
the reference's launcher symbols with a device index array and a cursor carried
across calls (narray/gen/tmpl_bit/where_kernel.cu:91-107, mask_kernel.cu:36-54)."""
import ctypes as C

import numpy as np
import pytest

import kat_adjacent as K

oracle = K.OracleEngine().o

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 31, 32, 33, 1000, 8191, 8192, 100003, (1 << 20) + 5, 1 << 25])
def test_where_matches_nonzero(n):
    import cumo_amd
    rng = np.random.default_rng(900 + n % 1000)
    density = rng.choice([0.02, 0.5, 0.97])
    h = (rng.random(n) < density).astype(np.uint8)
    b = cumo_amd.Bit.cast(h)
    got = b.where()
    assert isinstance(got, cumo_amd.Int32)
    assert (got.to_numpy() == oracle.where(h)).all()
    t, f = b.where2()
    assert (t.to_numpy() == oracle.where(h)).all() and (f.to_numpy() == oracle.where(h, invert=True)).all()
    if n > 40:
        for sl in (slice(3, None), slice(5, n - 7), slice(None, None, 2), slice(1, None, 3), slice(None, None, -1)):
            assert (b[sl].where().to_numpy() == oracle.where(h[sl])).all(), sl


def test_where_on_matrices_and_empty_results():
    import cumo_amd
    rng = np.random.default_rng(91)
    h = (rng.random((300, 777)) < 0.3).astype(np.uint8)
    b = cumo_amd.Bit.cast(h)
    assert (b.where().to_numpy() == oracle.where(h)).all()
    # views that do not contract to one run: one launch sequence per row, the cursor carried on the device
    for key in ((slice(5, 200), slice(7, 600)), (slice(None), slice(None, None, 3)), (slice(None, None, -1), slice(None))):
        assert (b[key].where().to_numpy() == oracle.where(h[key])).all(), key
    assert (b.transpose().where().to_numpy() == oracle.where(h.T)).all()
    z = cumo_amd.Bit.cast(np.zeros(5000, dtype=np.uint8))
    assert z.where().to_numpy().shape == (0,)
    assert (z.where2()[1].to_numpy() == np.arange(5000)).all()


@pytest.mark.parametrize("tname,dt", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_mask_gathers_in_row_major_order(tname, dt):
    import cumo_amd
    cls = getattr(cumo_amd, tname)
    rng = np.random.default_rng(92)
    for shape in [(7,), (100003,), (300, 777), (5, 6, 130)]:
        hx = rng.integers(-1000, 1000, size=shape).astype(dt)
        hm = (rng.random(shape) < 0.4)
        x, m = cls.cast(hx), cumo_amd.Bit.cast(hm.astype(np.uint8))
        got = m.mask(x)
        assert isinstance(got, cls) and (got.to_numpy() == oracle.mask(hm, hx)).all(), shape
        assert (x[m].to_numpy() == oracle.mask(hm, hx)).all()
        if len(shape) == 2:
            # the masked array as a view: transposed, strided; the mask made from a comparison
            assert (m.transpose().mask(x.transpose()).to_numpy() == hx.T[hm.T]).all()
            assert (m[::2, 1::3].mask(x[::2, 1::3]).to_numpy() == hx[::2, 1::3][hm[::2, 1::3]]).all()
            gt = x > 0
            assert (x[gt].to_numpy() == hx[hx > 0]).all()
    with pytest.raises(cumo_amd.ShapeError):
        cumo_amd.Bit.cast(np.ones(4, dtype=np.uint8)).mask(cls.cast(np.zeros(5, dtype=dt)))


def test_where_and_mask_launchers_with_index_arrays_and_a_carried_cursor():
    from cumo_amd import _lib
    from test_gpu_raw_abi import dev, fetch, free
    rng = np.random.default_rng(93)
    nbits = 50000
    h = (rng.random(nbits) < 0.35).astype(np.uint8)
    words = np.packbits(h, bitorder="little").view(np.uint32) if nbits % 32 == 0 else np.frombuffer(
        np.packbits(np.concatenate([h, np.zeros(32 - nbits % 32, np.uint8)]), bitorder="little").tobytes(), dtype=np.uint32)
    pw = dev(words)
    new = _lib.fn("cumo_bit_where_scratch_new", C.c_void_p, [])
    where = _lib.fn("cumo_bit_where_kernel_launch", None,
                    [C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_void_p, C.c_uint64, C.c_int, C.c_void_p, C.c_size_t, C.c_uint64, C.c_void_p])
    scratch = _lib.call(new)
    # two runs, the second through a device index array, both appended to one output
    n1, p1 = 20000, 13
    idx = rng.permutation(nbits - 100)[:15000].astype(np.uint64)
    pidx = dev(idx)
    want = np.concatenate([oracle.where(h[p1:p1 + n1]), n1 + oracle.where(h[7 + idx.astype(np.int64)])])
    pout = dev(np.full(want.size + 4, -1, dtype=np.int64))
    _lib.call(where, pw, p1, 1, None, n1, 0, pout, 8, 0, scratch)
    _lib.call(where, pw, 7, 0, pidx, idx.size, 0, pout, 8, n1, scratch)
    got = fetch(pout, (want.size + 4,), np.int64)
    assert (got[:want.size] == want).all() and (got[want.size:] == -1).all()
    # the zeros keep their own cursor (scratch word 1): a strided run, every third bit
    n3 = 9000
    wantz = oracle.where(h[5:5 + 3 * n3:3] == 0)
    pz = dev(np.full(wantz.size + 2, -1, dtype=np.int32))
    _lib.call(where, pw, 5, 3, None, n3, 1, pz, 4, 0, scratch)
    gz = fetch(pz, (wantz.size + 2,), np.int32)
    assert (gz[:wantz.size] == wantz).all() and (gz[wantz.size:] == -1).all()
    # mask: positions of the masked array's elements, base 40 bytes and 8 bytes apart
    _lib.lib.cumo_cuda_runtime_free(scratch)
    scratch = _lib.call(new)
    mask = _lib.fn("cumo_bit_mask_kernel_launch", None,
                   [C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_void_p, C.c_uint64, C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_void_p, C.c_void_p])
    wantm = 40 + 8 * oracle.where(h[p1:p1 + n1])
    pm = dev(np.zeros(wantm.size + 1, dtype=np.uint64))
    _lib.call(mask, pw, p1, 1, None, n1, pm, 40, 8, None, scratch)
    gm = fetch(pm, (wantm.size + 1,), np.uint64)
    assert (gm[:wantm.size] == wantm.astype(np.uint64)).all() and gm[wantm.size] == 0
    _lib.lib.cumo_cuda_runtime_free(scratch)
    free(pw, pidx, pout, pz, pm)


@pytest.mark.parametrize("nbits", [1, 31, 8193, 1 << 20, (1 << 25) + 77])
def test_count_then_place_launchers(nbits):
    """The two-launch form for a caller that sizes the result in between: block counts, read back and
    added up, then the placement of positions (set or clear bits, 4- or 8-byte) or of elements."""
    from cumo_amd import _lib
    from test_gpu_raw_abi import dev, fetch, free
    rng = np.random.default_rng(nbits)
    lead = 37                                       # the run starts inside a word
    h = (rng.random(lead + 3 * nbits if nbits < 10000 else lead + nbits) < 0.4).astype(np.uint8)
    pad = (-h.size) % 32
    words = np.frombuffer(np.packbits(np.concatenate([h, np.zeros(pad, np.uint8)]), bitorder="little").tobytes(), dtype=np.uint32)
    pw = dev(words)
    blocks = _lib.fn("cumo_hip_bit_where_blocks", C.c_size_t, [C.c_uint64])
    count = _lib.fn("cumo_hip_bit_where_count_kernel_launch", None, [C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint64, C.c_int, C.c_void_p])
    place = _lib.fn("cumo_hip_bit_where_place_kernel_launch", None,
                    [C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint64, C.c_int, C.c_void_p, C.c_void_p, C.c_ssize_t, C.c_size_t, C.c_void_p])
    nb = blocks(nbits)
    assert 1 <= nb <= 1024 and blocks(0) == 0
    x = rng.standard_normal(nbits).astype(np.float32)
    xd = rng.standard_normal(2 * nbits)             # every second double
    px, pxd = dev(x), dev(xd)
    cases = [(1, 0, 8), (1, 1, 4)] + ([(3, 0, 4)] if nbits < 10000 else [])
    for step, invert, elmsz in cases:
        run = h[lead:lead + step * nbits:step]
        hits = np.flatnonzero(run == (0 if invert else 1))
        pc = dev(np.full(nb + 1, 12345, dtype=np.uint64))
        _lib.call(count, pw, lead, step, nbits, invert, pc)
        counts = fetch(pc, (nb + 1,), np.uint64)
        assert int(counts[:nb].sum()) == hits.size and counts[nb] == 12345
        it = np.int64 if elmsz == 8 else np.int32
        po = dev(np.full(hits.size + 3, -1, dtype=it))
        _lib.call(place, pw, lead, step, nbits, invert, pc, None, 0, elmsz, po)
        got = fetch(po, (hits.size + 3,), it)
        assert (got[:hits.size] == hits).all() and (got[hits.size:] == -1).all()
        if step == 1 and not invert:
            pv = dev(np.full(hits.size + 1, 7.0, dtype=np.float32))
            _lib.call(place, pw, lead, 1, nbits, 0, pc, px, 4, 4, pv)
            gv = fetch(pv, (hits.size + 1,), np.float32)
            assert (gv[:hits.size] == x[hits]).all() and gv[hits.size] == 7.0
            pv8 = dev(np.full(hits.size + 1, 7.0, dtype=np.float64))
            _lib.call(place, pw, lead, 1, nbits, 0, pc, pxd, 16, 8, pv8)
            gv8 = fetch(pv8, (hits.size + 1,), np.float64)
            assert (gv8[:hits.size] == xd[::2][hits]).all() and gv8[hits.size] == 7.0
            free(pv, pv8)
        free(pc, po)
    free(pw, px, pxd)


def test_where_and_mask_into_a_given_result():
    """A result array of exactly the count's length is written in place; any other length is a shape error."""
    import ctypes as C
    import cumo_amd
    from cumo_amd import _lib
    rng = np.random.default_rng(21)
    x = rng.standard_normal((50, 70)).astype(np.float32)
    d = cumo_amd.SFloat.cast(x)
    m = d > 0.25
    want_pos = oracle.where(x > np.float32(0.25)).astype(np.int32)
    pos = cumo_amd.Int32.zeros(len(want_pos))
    md, zd = m._desc(), pos._desc()
    _lib.call(_lib.lib.cumo_hip_na_where, C.byref(md), 0, C.byref(zd))
    assert (pos.to_numpy() == want_pos).all()
    vals = cumo_amd.SFloat.zeros(len(want_pos))
    xd, vd = d._desc(), vals._desc()
    _lib.call(_lib.lib.cumo_hip_na_mask, C.byref(md), C.byref(xd), C.byref(vd))
    assert (vals.to_numpy() == x.ravel()[want_pos]).all()
    short = cumo_amd.Int32.zeros(len(want_pos) - 1)
    sd = short._desc()
    with pytest.raises(cumo_amd.ShapeError):
        _lib.call(_lib.lib.cumo_hip_na_where, C.byref(md), 0, C.byref(sd))


@pytest.mark.parametrize("tname,dt", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_mask_of_single_runs_with_offsets_steps_and_reversal(tname, dt):
    """Mask and masked array that each walk as one run (sliced alike) are compacted in place of
    positions: starts inside a word, steps other than 1, a reversed run, different steps on the two sides."""
    import cumo_amd
    cls = getattr(cumo_amd, tname)
    rng = np.random.default_rng(93)
    n = 100003
    hx = rng.integers(-1000, 1000, size=n).astype(dt)
    hm = rng.random(n) < 0.35
    x, m = cls.cast(hx), cumo_amd.Bit.cast(hm.astype(np.uint8))
    for sl in (slice(7, None), slice(33, n - 9), slice(None, None, 2), slice(5, None, 3), slice(None, None, -1), slice(n - 4, 2, -5)):
        got = m[sl].mask(x[sl]).to_numpy()
        assert (got == oracle.mask(hm[sl], hx[sl])).all(), sl
    # the mask contiguous, the masked array every other element of a longer one
    hy = rng.integers(-1000, 1000, size=2 * n).astype(dt)
    y = cls.cast(hy)
    assert (m.mask(y[::2]).to_numpy() == oracle.mask(hm, hy[::2])).all()
    assert (m[::-1].mask(y[1::2]).to_numpy() == oracle.mask(hm[::-1], hy[1::2])).all()
    # nothing set, everything set
    none, every = cumo_amd.Bit.cast(np.zeros(n, dtype=np.uint8)), cumo_amd.Bit.cast(np.ones(n, dtype=np.uint8))
    assert none.mask(x).to_numpy().shape == (0,)
    assert (every.mask(x).to_numpy() == hx).all()


def test_where_beyond_two_to_the_32_elements_answers_int64():
    """More than 2^32 - 1 elements: positions no longer fit Int32 (gen/tmpl_bit/where.c:104-110
    picks Int64 then). The bits are set on the device buffer word by word; no host array of
    that length is made."""
    import ctypes as C
    import cumo_amd
    from cumo_amd import _lib
    n = (1 << 32) + 70
    b = cumo_amd.Bit.zeros(n)
    want = [5, (1 << 31) + 3, (1 << 32) - 1, 1 << 32, (1 << 32) + 69]
    for pos in want:
        word = np.array([1 << (pos % 32)], dtype=np.uint32)
        assert _lib.call(_lib.lib.cumo_hip_copy_from_host, b._buf.ptr + (pos // 32) * 4, word.ctypes.data, 4) == 0
    assert int(b.count_true()) == len(want)
    got = b.where()
    assert isinstance(got, cumo_amd.Int64) and got.to_numpy().tolist() == want
    # a view that starts beyond 2^32 bits
    tail = b[(1 << 32) - 2:]
    assert tail.where().to_numpy().tolist() == [1, 2, 71]
    assert int(tail.count_false()) == 72 - 3
    del b, tail, got
    cumo_amd.MemoryPool.free_all_blocks()
