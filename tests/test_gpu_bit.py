"""Bit parity: packing, logical ops, count_true/count_false, Bit -> number.
Everything here is bit-exact (test/bit_test.rb:19-72, test/narray_test.rb:2667-2860)."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle"))
import numo_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu


def test_bit_test_rb_literals():
    # test/bit_test.rb:19-72
    import cumo_amd
    a = cumo_amd.Bit.cast([0, 1, 1, 0, 1, 0, 0, 1])
    assert a.to_numpy().tolist() == [0, 1, 1, 0, 1, 0, 0, 1]
    assert int(a.count_true()) == 4
    assert int(a.count_false()) == 4
    assert (~a).to_numpy().tolist() == [1, 0, 0, 1, 0, 1, 1, 0]
    b = cumo_amd.Bit.cast([0, 0, 1, 1, 0, 0, 1, 1])
    assert (a & b).to_numpy().tolist() == [0, 0, 1, 0, 0, 0, 0, 1]
    assert (a | b).to_numpy().tolist() == [0, 1, 1, 1, 1, 0, 1, 1]
    assert (a ^ b).to_numpy().tolist() == [0, 1, 0, 1, 1, 0, 1, 0]
    assert a.eq(b).to_numpy().tolist() == [1, 0, 1, 0, 0, 1, 0, 1]
    m = cumo_amd.Bit.cast([[0, 1, 1, 0], [1, 0, 0, 1]])
    assert m.count_true(axis=0).to_numpy().tolist() == [1, 1, 1, 1]
    assert m.count_true(axis=1).to_numpy().tolist() == [2, 2]
    assert m.count_false(axis=1).to_numpy().tolist() == [2, 2]
    # test/bit_test.rb:35-40,67-72,161-166: where, where2, mask, all?, any?, none?
    for v in (a, m):
        assert v.where().to_a() == [1, 2, 4, 7]
        assert [w.to_a() for w in v.where2()] == [[1, 2, 4, 7], [0, 3, 5, 6]]
        assert not v.all_p() and v.any_p() and not v.none_p()
    assert a.mask(cumo_amd.DFloat.cast([1, 2, 3, 4, 5, 6, 7, 8])).to_a() == [2, 3, 5, 8]
    assert m.mask(cumo_amd.DFloat.cast([[1, 2, 3, 4], [5, 6, 7, 8]])).to_a() == [2, 3, 5, 8]
    ones, zeros = cumo_amd.Bit.cast([1] * 70), cumo_amd.Bit.cast([0] * 70)
    assert ones.all_p() and ones.any_p() and not ones.none_p()
    assert not zeros.all_p() and not zeros.any_p() and zeros.none_p()
    assert ones[3:67].all_p() and zeros[::3].none_p()


@pytest.mark.parametrize("n", [1, 5, 31, 32, 33, 63, 64, 65, 200, 1000, 100003, 1 << 20])
def test_long_arrays_and_views(n):
    import cumo_amd
    rng = np.random.default_rng(300 + n)
    ha = rng.integers(0, 2, size=n).astype(np.uint8)
    hb = rng.integers(0, 2, size=n).astype(np.uint8)
    a, b = cumo_amd.Bit.cast(ha), cumo_amd.Bit.cast(hb)
    assert (a.to_numpy() == ha).all()
    assert ((a & b).to_numpy() == oracle.bit_binary("and", ha, hb)).all()
    assert ((a | b).to_numpy() == oracle.bit_binary("or", ha, hb)).all()
    assert ((a ^ b).to_numpy() == oracle.bit_binary("xor", ha, hb)).all()
    assert (a.eq(b).to_numpy() == oracle.bit_binary("eq", ha, hb)).all()
    assert ((~a).to_numpy() == oracle.bit_binary("not", ha)).all()
    assert int(a.count_true()) == int(ha.sum())
    assert int(a.count_false()) == int(n - ha.sum())
    w = oracle.pack(ha)
    if n > 40:
        # views that start inside a word, skip, and run backwards
        for sl in (slice(3, None), slice(5, n - 7), slice(None, None, 2), slice(1, None, 3), slice(None, None, -1), slice(n - 2, 3, -5)):
            va, vb = a[sl], b[sl]
            assert (va.to_numpy() == ha[sl]).all(), sl
            assert int(va.count_true()) == int(ha[sl].sum()), sl
            assert int(va.count_false()) == int((1 - ha[sl]).sum()), sl
            start, stop, step = sl.indices(n)
            cnt = len(range(start, stop, step))
            assert int(va.count_true()) == oracle.bit_count(w, start, step, cnt), sl
            assert ((va & vb).to_numpy() == (ha[sl] & hb[sl])).all(), sl
            assert ((~va).to_numpy() == 1 - ha[sl]).all(), sl
            assert (va.copy().to_numpy() == ha[sl]).all(), sl


def test_count_along_axes_and_2d_views():
    import cumo_amd
    rng = np.random.default_rng(301)
    h = rng.integers(0, 2, size=(13, 70, 9)).astype(np.uint8)
    d = cumo_amd.Bit.cast(h)
    for axis in [0, 1, 2, (0, 1), (1, 2), (0, 2), None]:
        got = d.count_true(axis=axis)
        got = got.to_numpy() if hasattr(got, "to_numpy") else got
        assert (np.asarray(got) == h.sum(axis=axis)).all(), axis
    t = d.transpose()
    assert (t.count_true(axis=0).to_numpy() == h.transpose().sum(axis=0)).all()
    assert (d[::2, 1::3].count_false(axis=1).to_numpy() == (1 - h[::2, 1::3]).sum(axis=1)).all()
    assert d.count_true(axis=1, keepdims=True).shape == (13, 1, 9)
    # logical ops on views that cannot be flattened (test/narray_test.rb:3500-3605)
    a, b = d[:, ::2], d[:, 1::2]
    assert ((a & b).to_numpy() == (h[:, ::2] & h[:, 1::2])).all()
    assert ((a.transpose() | b.transpose()).to_numpy() == (h[:, ::2] | h[:, 1::2]).transpose()).all()
    assert ((d & d[0]).to_numpy() == (h & h[0])).all()


def test_compare_then_count_matches_popcount():
    import cumo_amd
    rng = np.random.default_rng(302)
    h = rng.standard_normal((300, 1000)).astype(np.float32)
    d = cumo_amd.SFloat.cast(h)
    mask = d > 0.5
    assert int(mask.count_true()) == int((h > 0.5).sum())
    assert (mask.count_true(axis=1).to_numpy() == (h > 0.5).sum(axis=1)).all()
    tm = d.transpose() > 0.5
    assert int(tm.count_true()) == int((h > 0.5).sum())
    assert (tm.to_numpy() == (h.T > 0.5)).all()
    nums = mask._store_into(cumo_amd.Int32)
    assert (nums.to_numpy() == (h > 0.5)).all()
    assert (mask._store_into(cumo_amd.DFloat).to_numpy() == oracle.store_bit(np.float64, (h > 0.5).astype(np.uint8))).all()


def test_count_along_axes_in_one_launch_matches_numpy():
    """Counts along axes go through one launch for all outputs; every layout of the
    kept and the reduced dimensions against numpy's sums of the same bits."""
    import cumo_amd
    rng = np.random.default_rng(77)
    for shape in [(512, 777), (3, 5, 130), (64, 64), (7, 1, 33), (2, 3, 4, 65)]:
        h = rng.integers(0, 2, size=shape).astype(np.uint8)
        b = cumo_amd.Bit.cast(h)
        nd = len(shape)
        axes = [None] + list(range(nd)) + [-1] + ([(0, nd - 1)] if nd > 2 else []) + ([(0, 1)] if nd > 2 else [])
        for ax in axes:
            want = h.sum(axis=ax, dtype=np.uint64)
            assert (np.asarray(b.count_true(axis=ax).to_numpy()) == want).all(), (shape, ax)
            total = np.prod([shape[a] for a in (range(nd) if ax is None else ([ax] if isinstance(ax, int) else ax))])
            assert (np.asarray(b.count_false(axis=ax).to_numpy()) == total - want).all(), (shape, ax, "false")
        assert b.count_true(axis=nd - 1, keepdims=True).to_numpy().shape == shape[:-1] + (1,)
        if nd == 2:
            # views: rows reversed, every third column, a window that starts inside a word, the transpose
            for key in ((slice(None, None, -1), slice(None)), (slice(None), slice(1, None, 3)), (slice(5, 50), slice(7, 60)),
                        (slice(None), slice(None, None, -1))):
                for ax in (0, 1):
                    assert (np.asarray(b[key].count_true(axis=ax).to_numpy()) == h[key].sum(axis=ax, dtype=np.uint64)).all(), (shape, key, ax)
            for ax in (0, 1):
                assert (np.asarray(b.transpose().count_true(axis=ax).to_numpy()) == h.T.sum(axis=ax, dtype=np.uint64)).all()


def test_rows_of_bits_in_views_word_by_word():
    """Logical operations and copies on views whose rows run along the bits but do not form one run
    (windows that start inside a word, rows that share their first and last word with neighbours,
    skipped and reversed rows, three dimensions): a lane takes a word of a result row. Storing into
    such a view leaves every bit around it as it was."""
    import cumo_amd
    rng = np.random.default_rng(611)
    for shape in [(70, 131), (5, 4099), (300, 33), (9, 7, 67), (64, 64), (33, 1000), (6, 5, 300), (3, 4, 5, 129), (600, 4097)]:
        ha = rng.integers(0, 2, size=shape).astype(np.uint8)
        hb = rng.integers(0, 2, size=shape).astype(np.uint8)
        a, b = cumo_amd.Bit.cast(ha), cumo_amd.Bit.cast(hb)
        keys = [(Ellipsis, slice(1, None)), (Ellipsis, slice(None, -1)), (slice(None, None, 2), Ellipsis, slice(3, -5)),
                (slice(None, None, -1), Ellipsis, slice(2, None)), (slice(1, None), Ellipsis, slice(0, 40))]
        for ka in keys:
            for kb in keys:
                va, vb = ha[ka], hb[kb]
                if va.shape != vb.shape:
                    continue
                da, db = a[ka], b[kb]
                assert ((da & db).to_numpy() == oracle.bit_binary("and", va, vb)).all(), (shape, ka, kb)
                assert ((da ^ db).to_numpy() == oracle.bit_binary("xor", va, vb)).all(), (shape, ka, kb)
                assert (da.eq(db).to_numpy() == oracle.bit_binary("eq", va, vb)).all(), (shape, ka, kb)
            assert ((~a[ka]).to_numpy() == oracle.bit_binary("not", ha[ka])).all(), (shape, ka)
            assert (a[ka].copy().to_numpy() == ha[ka]).all(), (shape, ka)
        # an operand that repeats down the rows, on either side
        first = (0,) * (len(shape) - 1)
        assert ((a & b[first]).to_numpy() == (ha & hb[first])).all(), shape
        assert ((b[first] ^ a[..., :]).to_numpy() == (hb[first] ^ ha)).all(), shape
        assert ((a[..., 1:] | b[first][1:]).to_numpy() == (ha[..., 1:] | hb[first][1:])).all(), shape
        # into a window of an existing array
        for key, src_key in (((Ellipsis, slice(1, None)), (Ellipsis, slice(None, -1))), ((slice(1, None), Ellipsis, slice(3, 33)), (slice(None, -1), Ellipsis, slice(0, 30)))):
            hz = rng.integers(0, 2, size=shape).astype(np.uint8)
            z = cumo_amd.Bit.cast(hz)
            z[key] = a[src_key]
            hz[key] = ha[src_key]
            assert (z.to_numpy() == hz).all(), (shape, key)


def test_windows_of_a_large_matrix_into_a_fresh_result():
    """Rows of 32767 bits that follow one another in the result while the sources' rows are 32768 apart:
    the result is written as one run of whole vectors (past the size from which stores bypass the
    caches), a row ending inside one vector in four."""
    import cumo_amd
    rng = np.random.default_rng(619)
    shape = (4100, 32768)
    ha = np.unpackbits(np.frombuffer(rng.bytes(shape[0] * shape[1] // 8), dtype=np.uint8)).reshape(shape)
    hb = np.unpackbits(np.frombuffer(rng.bytes(shape[0] * shape[1] // 8), dtype=np.uint8)).reshape(shape)
    a, b = cumo_amd.Bit.cast(ha), cumo_amd.Bit.cast(hb)
    assert ((a[:, 1:] ^ b[:, :-1]).to_numpy() == (ha[:, 1:] ^ hb[:, :-1])).all()
    assert ((a[::-1, 5:] & b[:, :-5]).to_numpy() == (ha[::-1, 5:] & hb[:, :-5])).all()
    assert ((~a[1:, 31:-1]).to_numpy() == 1 - ha[1:, 31:-1]).all()
    assert (a[::2, 7:].copy().to_numpy() == ha[::2, 7:]).all()


@pytest.mark.parametrize("n", [2048, 2049, 5000, 100003, (1 << 22) + 77])
def test_long_runs_of_bits_by_whole_vectors(n):
    """One run (op) one run into one run, each starting at any bit of a word and any word of a 16-byte
    vector: four result words per lane, the run's first and last words one by one."""
    import cumo_amd
    rng = np.random.default_rng(612 + n % 1000)
    ha = rng.integers(0, 2, size=n + 200).astype(np.uint8)
    hb = rng.integers(0, 2, size=n + 200).astype(np.uint8)
    a, b = cumo_amd.Bit.cast(ha), cumo_amd.Bit.cast(hb)
    for (oa, ob) in [(0, 0), (1, 0), (0, 31), (5, 37), (64, 3), (33, 33), (96, 127), (130, 65)]:
        va, vb = ha[oa:oa + n], hb[ob:ob + n]
        da, db = a[oa:oa + n], b[ob:ob + n]
        assert ((da & db).to_numpy() == oracle.bit_binary("and", va, vb)).all(), (oa, ob)
        assert ((da | db).to_numpy() == oracle.bit_binary("or", va, vb)).all(), (oa, ob)
        assert (da.eq(db).to_numpy() == oracle.bit_binary("eq", va, vb)).all(), (oa, ob)
        assert ((~da).to_numpy() == oracle.bit_binary("not", va)).all(), (oa, ob)
        hz = rng.integers(0, 2, size=n + 200).astype(np.uint8)
        z = cumo_amd.Bit.cast(hz)
        z[ob:ob + n] = da                      # into a run that starts elsewhere: the bits around it stay
        hz[ob:ob + n] = va
        assert (z.to_numpy() == hz).all(), (oa, ob)
        assert int(da.count_true()) == int(va.sum()) and int(db.count_false()) == int(n - vb.sum())


def test_counts_down_columns_and_along_long_rows():
    """count_true / count_false (and with them all? / any? along an axis) where the kept dimension runs
    along the bits: 32 columns per lane in byte-wide counters, rows cut over lanes (more than 252 rows
    per lane: the counters are emptied in between); and along rows of many words (128-bit loads from
    any word). Shapes whose rows do not start on words, views, three dimensions."""
    import cumo_amd
    rng = np.random.default_rng(613)
    for shape in [(300, 70), (1000, 4097), (5, 64), (40000, 65), (3, 500, 130), (2, 70000, 96), (700, 1000), (33, 32767), (70, 5000),
                  (70, 4096), (300, 2048), (9, 5, 2112), (3, 100000 * 32), (1000, 256), (5000, 384), (4, 700, 1024), (64, 128), (20000, 8320)]:
        h = (rng.random(shape) < 0.7).astype(np.uint8)
        h[..., 1] = 1                          # a column that is all set, one that is all clear
        h[..., 2] = 0
        b = cumo_amd.Bit.cast(h)
        nd = len(shape)
        for ax in (nd - 2, nd - 1):
            want = h.sum(axis=ax, dtype=np.uint64)
            assert (np.asarray(b.count_true(axis=ax).to_numpy()) == want).all(), (shape, ax)
            assert (np.asarray(b.count_false(axis=ax).to_numpy()) == shape[ax] - want).all(), (shape, ax)
            assert (b.all_p(axis=ax).to_numpy() == h.all(axis=ax)).all(), (shape, ax)
            assert (b.any_p(axis=ax).to_numpy() == h.any(axis=ax)).all(), (shape, ax)
            assert (b.none_p(axis=ax).to_numpy() == ~h.any(axis=ax)).all(), (shape, ax)
        for key in ((Ellipsis, slice(3, None)), (Ellipsis, slice(None, None, -1), slice(1, -1)), (Ellipsis, slice(None, None, 2), slice(5, 69)),
                    (Ellipsis, slice(128, None)), (Ellipsis, slice(None, None, 3), slice(64, 64 + 128)),
                    (Ellipsis, slice(None, None, -1), slice(None)), (Ellipsis, slice(None, None, -2), slice(32, None))):
            v, dv = h[key], b[key]
            if v.size == 0:
                continue
            for ax in (nd - 2, nd - 1):
                assert (np.asarray(dv.count_true(axis=ax).to_numpy()) == v.sum(axis=ax, dtype=np.uint64)).all(), (shape, key, ax)
        assert int(b.count_true()) == int(h.sum())


@pytest.mark.parametrize("tname,dt", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_bits_to_numbers_by_rows(tname, dt):
    """Bit -> number where both run along the innermost dimension: four elements per lane, stored as
    128-bit vectors from any element boundary; rows that end in part of a vector, windows that start
    inside a word, skipped rows, a destination that is a window of a larger array."""
    import cumo_amd
    rng = np.random.default_rng(614)
    cls = getattr(cumo_amd, tname)
    for shape in [(70, 131), (5, 4099), (300, 33), (9, 7, 67), (64, 64), (1, 100003), (100003,)]:
        h = rng.integers(0, 2, size=shape).astype(np.uint8)
        b = cumo_amd.Bit.cast(h)
        assert (b._store_into(cls).to_numpy() == oracle.store_bit(dt, h)).all(), shape
        for key in ((Ellipsis, slice(1, None)), (Ellipsis, slice(3, -5)), (slice(None, None, 2),), (slice(None, None, -1), Ellipsis, slice(2, None))):
            if len(shape) == 1 and len([k for k in key if k is not Ellipsis]) > 1:
                continue
            assert (b[key]._store_into(cls).to_numpy() == oracle.store_bit(dt, h[key])).all(), (shape, key)
        if len(shape) > 1:
            hz = rng.standard_normal(shape).astype(dt)
            z = cls.cast(hz)
            z[..., 1:] = b[..., :-1]
            hz[..., 1:] = h[..., :-1]
            assert (z.to_numpy() == hz).all(), shape


@pytest.mark.parametrize("tname,dt", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_numbers_to_bits_of_a_whole_array_and_of_windows(tname, dt):
    """number -> Bit (nonzero is 1, NaN included, the zero of either sign is 0): into a whole array
    (the comparison kernels take it), into the front part of a longer one (the bits after it stay),
    into windows, from a source that repeats."""
    import cumo_amd
    rng = np.random.default_rng(615)
    cls = getattr(cumo_amd, tname)
    for shape in [(70, 131), (5, 4099), (100003,), (8, 4096), (64, 64), (3, 5, 67)]:
        h = (rng.integers(-2, 3, size=shape)).astype(dt)
        if dt != np.int32:
            h.reshape(-1)[::7] = np.nan
            h.reshape(-1)[3::11] = -0.0
        want = (h != 0).astype(np.uint8)
        d = cls.cast(h)
        assert (cumo_amd.Bit.cast(np.zeros(shape, dtype=np.uint8)).store(d).to_numpy() == want).all(), shape
        hz = rng.integers(0, 2, size=(2,) + shape).astype(np.uint8)
        z = cumo_amd.Bit.cast(hz)
        z[0] = d                               # the front part of a longer array
        hz[0] = want
        assert (z.to_numpy() == hz).all(), shape
        z[1, ..., 1:] = d[..., :-1]            # a window that starts inside a word
        hz[1, ..., 1:] = want[..., :-1]
        assert (z.to_numpy() == hz).all(), shape
        for one in (3, 0):                     # a single number spread over the array
            z1 = cumo_amd.Bit.cast(rng.integers(0, 2, size=shape).astype(np.uint8))
            z1.store(cls.cast(np.array([one], dtype=dt)))
            assert (z1.to_numpy() == (1 if one else 0)).all(), (shape, one)
        if len(shape) == 2:
            z2 = cumo_amd.Bit.cast(np.zeros(shape, dtype=np.uint8))
            z2.store(d[:1])                    # one row repeated down the array
            assert (z2.to_numpy() == np.broadcast_to(want[:1], shape)).all(), shape


@pytest.mark.parametrize("n", [1 << 24, (1 << 24) + 77, (1 << 25) + 31])
def test_counts_of_very_long_runs(n):
    """A run of 2^24 bits or more is counted by the reduction kernels over its words, the first and
    the last word masked: runs that start at any bit, that end in part of a word, set and clear bits."""
    import cumo_amd
    rng = np.random.default_rng(616)
    h = (rng.random(n + 100) < 0.3).astype(np.uint8)
    b = cumo_amd.Bit.cast(h)
    for lo in (0, 1, 31, 32, 45):
        for cut in (0, 1, 33):
            v = h[lo:n + 100 - cut]
            d = b[lo:n + 100 - cut]
            assert int(d.count_true()) == int(v.sum()), (lo, cut)
            assert int(d.count_false()) == int(v.size - v.sum()), (lo, cut)
    ones = cumo_amd.Bit.cast(np.ones(n, dtype=np.uint8))
    assert int(ones.count_true()) == n and int(ones.count_false()) == 0 and ones.all_p() and not ones.none_p()


def test_counts_down_columns_of_word_aligned_rows():
    """Rows that start on word boundaries take the carry-save form (a lane per 32, 64 or 128
    columns, blocks of a column group folded through scratch by the last one in): one, two
    and four words per lane, a last word that is partly columns, several stretches of 240
    rows per wave, many planes, and both ways of writing the result -- stored over whatever
    was there, and added onto it -- through the launcher itself."""
    import ctypes as C
    import cumo_amd
    from cumo_amd import _lib
    rng = np.random.default_rng(615)
    for shape in [(4096, 32768), (5000, 8192 + 64), (3000, 16384 + 64), (777, 4096 + 40), (600, 2500, 256), (3, 9000, 640), (65, 96), (2, 128),
                  (100, 1 << 17)]:
        h = (rng.random(shape) < 0.6).astype(np.uint8)
        h[..., 1] = 1
        h[..., 2] = 0
        b = cumo_amd.Bit.cast(h)
        nd = len(shape)
        want = h.sum(axis=nd - 2, dtype=np.uint64)
        assert (np.asarray(b.count_true(axis=nd - 2).to_numpy()) == want).all(), shape
        assert (np.asarray(b.count_false(axis=nd - 2).to_numpy()) == shape[nd - 2] - want).all(), shape
        if nd == 2:
            v = b[1::2, 64:]                  # every other row, from the third word on
            assert (np.asarray(v.count_true(axis=0).to_numpy()) == h[1::2, 64:].sum(axis=0, dtype=np.uint64)).all(), shape

    # the launcher with hand-built arguments: counts ADDED onto what the results hold
    MAXD = 12

    class CountNd(C.Structure):
        _fields_ = [("out_ndim", C.c_int), ("red_ndim", C.c_int), ("out_shape", C.c_size_t * MAXD), ("red_shape", C.c_size_t * MAXD),
                    ("in_out_step", C.c_ssize_t * MAXD), ("in_red_step", C.c_ssize_t * MAXD), ("out_step", C.c_ssize_t * MAXD),
                    ("in_", C.c_void_p), ("pos", C.c_size_t), ("out", C.c_void_p), ("count_false", C.c_int), ("overwrite", C.c_int)]

    f = _lib.fn("cumo_hip_bit_count_nd_kernel_launch", None, [C.POINTER(CountNd)])
    rows, cols = 3001, 4096 + 64
    h = (rng.random((rows, cols)) < 0.5).astype(np.uint8)
    b = cumo_amd.Bit.cast(h)
    start = np.arange(cols, dtype=np.uint64) * 3 + 7
    for overwrite in (0, 1):
        for count_false in (0, 1):
            out = cumo_amd.UInt64.cast(start)
            d = CountNd()
            d.out_ndim, d.red_ndim = 1, 1
            d.out_shape[0], d.red_shape[0] = cols, rows
            d.in_out_step[0], d.in_red_step[0], d.out_step[0] = 1, cols, 8
            d.in_, d.pos, d.out = b._buf.ptr, 0, out._buf.ptr
            d.count_false, d.overwrite = count_false, overwrite
            _lib.call(f, C.byref(d))
            counts = (rows - h.sum(axis=0, dtype=np.uint64)) if count_false else h.sum(axis=0, dtype=np.uint64)
            want = counts if overwrite else counts + start
            assert (out.to_numpy() == want).all(), (overwrite, count_false)


def test_all_any_along_word_aligned_rows():
    """all? / any? / none? along rows that start on word boundaries go from the rows to the packed
    result in one launch: whole 128-bit vectors and single words per lane, a last word that is partly
    row, rows decided at their first and at their last bit, kept dimensions that merge, rows of a view
    taken backwards and every other one, and a result that starts inside a word (the launcher itself:
    the bits around the result stay)."""
    import ctypes as C
    import cumo_amd
    from cumo_amd import _lib
    rng = np.random.default_rng(617)

    def rows_of(shape):
        # mostly rows of ones / zeros, so that all? and any? both have both answers; a few decided by one bit
        h = np.empty(shape, dtype=np.uint8)
        flat = h.reshape(-1, shape[-1])
        kind = rng.integers(0, 6, size=flat.shape[0])
        flat[:] = (kind % 2)[:, None]
        for k, col in ((2, 0), (3, 0), (4, -1), (5, -1)):
            flat[kind == k, col] ^= 1
        mid = rng.integers(0, shape[-1], size=flat.shape[0])
        pick = rng.random(flat.shape[0]) < 0.2
        flat[pick, mid[pick]] ^= 1
        return h

    def check(dv, hv, what):
        ax = hv.ndim - 1
        assert (dv.all_p(axis=ax).to_numpy() == hv.all(axis=ax)).all(), what
        assert (dv.any_p(axis=ax).to_numpy() == hv.any(axis=ax)).all(), what
        assert (dv.none_p(axis=ax).to_numpy() == ~hv.any(axis=ax)).all(), what

    for shape in [(4096, 4096), (5000, 8192 + 32), (4100, 32768), (4200, 8192), (70, 100, 4096 + 64), (9000, 4096), (4097, 1 << 16)]:
        h = rows_of(shape)
        b = cumo_amd.Bit.cast(h)
        check(b, h, shape)
        for key in ((Ellipsis, slice(0, 5000)), (Ellipsis, slice(64, None)), (slice(None, None, -1),), (slice(None, None, 2), Ellipsis, slice(32, 32 + 4100)),
                    (Ellipsis, slice(96, 96 + 4099))):
            hv, dv = h[key], b[key]
            if hv.shape[-1] >= 4096:
                check(dv, hv, (shape, key))

    f = _lib.fn("cumo_hip_bit_anyall_rows_kernel_launch", C.c_int,
                [C.c_void_p, C.c_size_t, C.c_uint64, C.c_int64, C.c_uint64, C.c_int, C.c_void_p, C.c_size_t])
    rows, cols = 4101, 4096 + 32
    h = rows_of((rows, cols))
    b = cumo_amd.Bit.cast(h)
    for out_pos in (0, 5, 31, 37):
        for all_ in (0, 1):
            before = (rng.random(out_pos + rows + 70) < 0.5).astype(np.uint8)
            out = cumo_amd.Bit.cast(before)
            took = _lib.call(f, b._buf.ptr, 32 * 0, rows, cols, cols - 7, all_, out._buf.ptr, out_pos)
            assert took == 1
            want = before.copy()
            hv = h[:, :cols - 7]
            want[out_pos:out_pos + rows] = hv.all(axis=1) if all_ else hv.any(axis=1)
            assert (out.to_numpy() == want).all(), (out_pos, all_)
    # shapes it leaves to the counts
    assert _lib.call(f, b._buf.ptr, 3, rows, cols, 4096, 1, out._buf.ptr, 0) == 0
    assert _lib.call(f, b._buf.ptr, 0, 100, cols, 4096, 1, out._buf.ptr, 0) == 0
