"""Index-array views: the launchers that do arithmetic on device index arrays, the
1-D indexed copy, the gather / scatter between a view with index arrays and a
contiguous buffer, and the array methods built on them (a[[...]], a[[...]] = v, at,
diagonal). Integer and byte work: bit-exact against numpy on the same inputs.
Cases follow test/narray_test.rb:250-330 (advanced indexing, at, diagonal) of the
reference for the shapes it uses."""
import ctypes as C

import numpy as np
import pytest

import kat_adjacent as K
from helpers import assert_bits_equal
from test_gpu_raw_abi import dev, fetch, free, indexer

oracle = K.OracleEngine().o

pytestmark = pytest.mark.gpu

P = C.POINTER
V, SZ, SS, U64 = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint64
M64 = (1 << 64) - 1


def u64(a):
    return np.asarray(a, dtype=np.uint64)


def wrap(x):
    """python ints -> uint64 with two's-complement wrap, as size_t arithmetic does"""
    return np.array([int(v) & M64 for v in x], dtype=np.uint64)


@pytest.mark.parametrize("n", [1, 255, 256, 1000, 70001])
def test_index_arithmetic_launchers(n):
    from cumo_amd import _lib
    rng = np.random.default_rng(n)
    m = 4 * n + 7
    idx0 = rng.integers(0, m, n)            # positions
    table = rng.integers(0, 1 << 40, m)     # an existing index array (byte offsets)
    table2 = rng.integers(0, 1 << 40, 3 * n + 11)
    acc0 = rng.integers(0, 1 << 40, n)      # an accumulated index array
    beg, step = 3, 2
    s1 = 24
    last = m - 1
    ptab, ptab2 = dev(u64(table)), dev(u64(table2))
    pidx0 = dev(u64(idx0))

    def run(name, argtypes, start, *args):
        p = dev(u64(start))
        f = _lib.fn(name, None, argtypes)
        _lib.call(f, p, *args)
        out = fetch(p, (n,), np.uint64)
        free(p)
        return out

    ii = np.arange(n)
    ints = lambda a: [int(v) for v in a]
    for stride in (s1, -s1):
        got = run("cumo_na_index_aref_nadata_index_stride_kernel_launch", [V, SS, U64], idx0, stride, n)
        assert_bits_equal(got, wrap(v * stride for v in ints(idx0)))
        got = run("cumo_na_index_aref_naview_index_stride_kernel_launch", [V, SS, U64], idx0, stride, n)
        assert_bits_equal(got, wrap(v * stride for v in ints(idx0)))
        got = run("cumo_na_index_aref_naview_index_stride_last_kernel_launch", [V, SS, SZ, U64], idx0, stride, last, n)
        assert_bits_equal(got, wrap((last - v) * stride for v in ints(idx0)))
        got = run("cumo_na_index_at_nadata_index_stride_add_kernel_launch", [V, V, SS, U64], acc0, pidx0, stride, n)
        assert_bits_equal(got, wrap(a + v * stride for a, v in zip(ints(acc0), ints(idx0))))
        got = run("cumo_na_index_at_naview_index_stride_last_add_kernel_launch", [V, SS, SZ, U64], idx0, stride, last, n)
        assert_bits_equal(got, wrap(v + (last - v) * stride for v in ints(idx0)))
        for st in (step, -1):
            b = beg if st > 0 else n + 2
            got = run("cumo_na_index_at_nadata_index_beg_step_stride_kernel_launch", [V, SZ, SS, SS, U64], acc0, b, st, stride, n)
            assert_bits_equal(got, wrap((b + st * i) * stride for i in ints(ii)))
            got = run("cumo_na_index_at_nadata_index_beg_step_stride_add_kernel_launch", [V, SZ, SS, SS, U64], acc0, b, st, stride, n)
            assert_bits_equal(got, wrap(a + (b + st * i) * stride for a, i in zip(ints(acc0), ints(ii))))
    got = run("cumo_na_index_aref_naview_index_index_kernel_launch", [V, V, U64], idx0, ptab, n)
    assert_bits_equal(got, u64(table[idx0]))
    got = run("cumo_na_index_at_naview_index_index_index_add_kernel_launch", [V, V, V, U64], acc0, ptab, pidx0, n)
    assert_bits_equal(got, u64(acc0 + table[idx0]))
    for st, b in ((step, beg), (-1, n + 2)):
        got = run("cumo_na_index_aref_naview_index_index_beg_step_kernel_launch", [V, V, SZ, SS, U64], acc0, ptab, b, st, n)
        assert_bits_equal(got, u64(table[b + st * ii]))
        got = run("cumo_na_index_at_naview_index_index_beg_step_add_kernel_launch", [V, V, SZ, SS, U64], acc0, ptab, b, st, n)
        assert_bits_equal(got, u64(acc0 + table[b + st * ii]))
    # the diagonal's index arrays (k0, k1: where the diagonal starts in each dimension)
    k0, k1 = 5, 9
    got = run("cumo_na_diagonal_index_index_kernel_launch", [V, V, V, SZ, SZ, U64], acc0, ptab, ptab2, k0, k1, n)
    assert_bits_equal(got, u64(table[ii + k0] + table2[ii + k1]))
    for stride in (s1, -s1):
        got = run("cumo_na_diagonal_index_stride_kernel_launch", [V, V, SS, SZ, SZ, U64], acc0, ptab, stride, k0, k1, n)
        assert_bits_equal(got, wrap(t + stride * (i + k1) for t, i in zip(ints(table[ii + k0]), ints(ii))))
        got = run("cumo_na_diagonal_stride_index_kernel_launch", [V, SS, V, SZ, SZ, U64], acc0, stride, ptab2, k0, k1, n)
        assert_bits_equal(got, wrap(stride * (i + k0) + t for t, i in zip(ints(table2[ii + k1]), ints(ii))))
    free(ptab, ptab2, pidx0)


@pytest.mark.parametrize("elmsz", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("n", [1, 300, 40000])
def test_copy_bytes_with_and_without_index_arrays(n, elmsz):
    from cumo_amd import _lib
    rng = np.random.default_rng(n + elmsz)
    m = 2 * n + 3
    src = rng.integers(0, 256, (m, elmsz), dtype=np.uint8)
    sel1 = rng.permutation(m)[:n]
    sel2 = rng.permutation(m)[:n]            # distinct targets: no write conflicts
    psrc = dev(src)
    pi1, pi2 = dev(u64(sel1 * elmsz)), dev(u64(sel2 * elmsz))
    f = _lib.fn("cumo_iter_copy_bytes_kernel_launch", None, [V, V, SS, SS, V, V, U64, SS])
    for use1 in (False, True):
        for use2 in (False, True):
            base = rng.integers(0, 256, (m, elmsz), dtype=np.uint8)
            pdst = dev(base)
            s1, s2 = 2 * elmsz, elmsz       # source every other element, target dense
            _lib.call(f, psrc, pdst, s1, s2, pi1 if use1 else None, pi2 if use2 else None, n, elmsz)
            want = base.copy()
            from_rows = sel1 if use1 else np.arange(n) * 2
            to_rows = sel2 if use2 else np.arange(n)
            want[to_rows] = src[from_rows]
            assert_bits_equal(fetch(pdst, (m, elmsz), np.uint8), want)
            free(pdst)
    free(psrc, pi1, pi2)


def stridx_array(ptr, entries):
    """entries: a python int stride in bytes, or a device pointer to offsets (tagged 'i')"""
    from cumo_amd import _lib
    a = _lib.IArrayStridx()
    a.ptr = ptr
    for d, e in enumerate(entries):
        if isinstance(e, tuple):
            a.stridx[d] = e[1]
        else:
            a.stridx[d] = (e << 1) | 1
    return a


@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.float32, np.float64, np.complex128])
def test_gather_and_scatter_between_view_and_buffer(dtype):
    from cumo_amd import _lib
    rng = np.random.default_rng(11)
    shape = (7, 9, 11, 5)
    es = np.dtype(dtype).itemsize
    x = rng.integers(0, 250, shape).astype(dtype)
    st = x.strides
    i0 = np.array([6, 0, 3, 3, 1])                  # repeats allowed when reading
    i2 = np.array([10, 2, 4, 0])
    pi0, pi2 = dev(u64(i0 * st[0])), dev(u64(i2 * st[2]))
    px = dev(x)
    # dims: index array, reversed stride with step 2, index array, plain stride
    sub = x[i0][:, ::-2][:, :, i2]
    a = stridx_array(px + 8 * st[1], [("i", pi0), -2 * st[1], ("i", pi2), st[3]])
    ix = indexer(sub.shape)
    pbuf = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, sub.nbytes)
    to_buf = _lib.fn("cumo_ndloop_copy_to_buffer_kernel_launch", None, [P(_lib.IArrayStridx), P(_lib.Indexer), V, SZ])
    from_buf = _lib.fn("cumo_ndloop_copy_from_buffer_kernel_launch", None, [P(_lib.IArrayStridx), P(_lib.Indexer), V, SZ])
    _lib.call(to_buf, C.byref(a), C.byref(ix), pbuf, es)
    assert_bits_equal(fetch(pbuf, sub.shape, dtype), sub)
    # scatter distinct positions back
    j0 = np.array([5, 1, 2])
    pj0 = dev(u64(j0 * st[0]))
    a2 = stridx_array(px + 8 * st[1], [("i", pj0), -2 * st[1], ("i", pi2), st[3]])
    new = rng.integers(0, 250, (3,) + sub.shape[1:]).astype(dtype)
    pnew = dev(new)
    ix2 = indexer(new.shape)
    _lib.call(from_buf, C.byref(a2), C.byref(ix2), pnew, es)
    want = x.copy()
    want[np.ix_(j0, np.arange(8, -1, -2), i2, np.arange(5))] = new
    assert_bits_equal(fetch(px, shape, dtype), want)
    free(px, pi0, pi2, pj0, pbuf, pnew)


def test_gather_large_and_zero_dimensional():
    from cumo_amd import _lib
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3000, 700)).astype(np.float32)
    rows = rng.integers(0, 3000, 2500)
    prow, px = dev(u64(rows * x.strides[0])), dev(x)
    a = stridx_array(px, [("i", prow), 4])
    ix = indexer((2500, 700))
    pbuf = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, 2500 * 700 * 4)
    to_buf = _lib.fn("cumo_ndloop_copy_to_buffer_kernel_launch", None, [P(_lib.IArrayStridx), P(_lib.Indexer), V, SZ])
    _lib.call(to_buf, C.byref(a), C.byref(ix), pbuf, 4)
    assert_bits_equal(fetch(pbuf, (2500, 700), np.float32), x[rows])
    # zero dimensions: one element
    a0 = stridx_array(px + 5 * 4, [])
    ix0 = indexer(())
    _lib.call(to_buf, C.byref(a0), C.byref(ix0), pbuf, 4)
    assert_bits_equal(fetch(pbuf, (1,), np.float32), x.ravel()[5:6])
    free(prow, px, pbuf)


# ---- the array methods ---------------------------------------------------------

@pytest.mark.parametrize("cls_name,dtype", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_getitem_with_index_arrays(cls_name, dtype):
    import cumo_amd
    cls = getattr(cumo_amd, cls_name)
    # narray_test.rb:250-262: a = [[1,2,3],[5,7,11]]
    src = np.array([[1, 2, 3], [5, 7, 11]], dtype=dtype)
    a = cls.cast(src)
    assert a[[0, 1], [0, 2]].to_a() == [[1, 3], [5, 11]]       # outer product of the selections
    assert a[[1, 0], True].to_a() == [[5, 7, 11], [1, 2, 3]]
    assert a[1, [2, 0, 0]].to_a() == [11, 5, 5]
    assert a[[-1], 1:].to_a() == [[7, 11]]
    assert a[..., [1]].to_a() == [[2], [7]]
    with pytest.raises(IndexError):
        a[[2], 0]
    with pytest.raises(IndexError):
        a[0, [-4]]
    rng = np.random.default_rng(7)
    x = rng.integers(-1000, 1000, (13, 17, 19)).astype(dtype)
    d = cls.cast(x)
    i0, i2 = rng.integers(0, 13, 20), rng.integers(-19, 19, 6)
    assert_bits_equal(d[i0, 3:15:2, i2].to_numpy(), oracle.take(x, (i0, slice(3, 15, 2), i2)))
    assert_bits_equal(d[i0].to_numpy(), oracle.take(x, (i0,)))
    # through a transposed and reversed view, and an Int32 array as the index
    v, xv = d.transpose(2, 0, 1).reverse(0), x.transpose(2, 0, 1)[::-1]
    k = cumo_amd.Int32.cast(np.array([18, 0, 5, 5], dtype=np.int32))
    assert_bits_equal(v[k, 2, [1, 16]].to_numpy(), oracle.take(xv, ([18, 0, 5, 5], 2, [1, 16])))
    assert d[[], 0].shape == (0, 19)


@pytest.mark.parametrize("cls_name,dtype", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_whole_rows_through_an_index_array(cls_name, dtype):
    """Rows of 256 bytes and more move as 128-bit vectors plus up to three 4-byte words, from any 4-byte
    boundary: row lengths that are and are not whole vectors, a view whose rows start one element in,
    rows picked twice when reading, a permutation when writing, two outer dimensions."""
    import cumo_amd
    cls = getattr(cumo_amd, cls_name)
    rng = np.random.default_rng(12)
    for shape in [(50, 64), (50, 67), (30, 131), (9, 4095), (12, 1000), (7, 1029), (40, 65)]:
        x = rng.integers(-1000, 1000, shape).astype(dtype)
        d = cls.cast(x)
        rows = rng.integers(0, shape[0], 2 * shape[0])
        perm = rng.permutation(shape[0])
        assert_bits_equal(d[rows].to_numpy(), x[rows], (shape, "rows with repeats"))
        assert_bits_equal(d[perm, True].to_numpy(), x[perm], (shape, "permutation"))
        assert_bits_equal(d[:, 1:][perm].to_numpy(), x[:, 1:][perm], (shape, "rows that start one element in"))
        b = cls.cast(np.zeros(shape, dtype=dtype))
        b[perm] = d
        want = np.zeros(shape, dtype=dtype)
        want[perm] = x
        assert_bits_equal(b.to_numpy(), want, (shape, "scatter"))
        c = cls.cast(np.zeros(shape, dtype=dtype))
        c[:, 1:][perm] = d[:, 1:]
        want = np.zeros(shape, dtype=dtype)
        want[:, 1:][perm] = x[:, 1:]
        assert_bits_equal(c.to_numpy(), want, (shape, "scatter into rows that start one element in"))
    x = rng.integers(-1000, 1000, (6, 5, 67)).astype(dtype)
    d = cls.cast(x)
    assert_bits_equal(d[[4, 0, 4], True, True].to_numpy(), x[[4, 0, 4]], "two outer dimensions")
    assert_bits_equal(d[True, [3, 1], True].to_numpy(), x[:, [3, 1]], "index array in the middle")


@pytest.mark.parametrize("cls_name,dtype", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_setitem_with_index_arrays_and_slices(cls_name, dtype):
    import cumo_amd
    cls = getattr(cumo_amd, cls_name)
    rng = np.random.default_rng(9)
    x = rng.integers(-1000, 1000, (11, 8, 6)).astype(dtype)
    d = cls.cast(x)
    want = x.copy()
    d[[3, 0, 10], 2:7, [5, 1]] = 42
    oracle.put(want, ([3, 0, 10], slice(2, 7), [5, 1]), 42)
    assert_bits_equal(d.to_numpy(), want)
    new = rng.integers(-1000, 1000, (2, 8, 6)).astype(dtype)
    d[[9, 4]] = cls.cast(new)
    oracle.put(want, ([9, 4],), new)
    assert_bits_equal(d.to_numpy(), want)
    row = rng.integers(-1000, 1000, (6,)).astype(dtype)        # broadcast along the selection
    d[[1, 2], 0] = cls.cast(row)
    oracle.put(want, ([1, 2], 0), row)
    assert_bits_equal(d.to_numpy(), want)
    d[1:3, ::2, 0] = 7                                         # slices only: a store into the view
    want[1:3, ::2, 0] = 7
    assert_bits_equal(d.to_numpy(), want)
    d.reverse(0)[[0], 0, :] = -5                               # a reversed dimension
    want[10, 0, :] = -5
    assert_bits_equal(d.to_numpy(), want)


def test_at_zipped_positions():
    import cumo_amd
    I32 = cumo_amd.Int32
    for cls in (cumo_amd.DFloat, cumo_amd.SFloat, cumo_amd.Int32):
        # narray_test.rb:124-134,171: a = [1,2,3,5,7,11]
        a = cls.cast([1, 2, 3, 5, 7, 11])
        assert a.at([3, 4]).to_a() == [5, 7]
        assert a[2:].at([1, 2]).to_a() == [5, 7]
        assert a.at(I32.cast([3, 4])).to_a() == [5, 7]
        assert a.at(range(3, 5)).to_a() == [5, 7]
        assert a.at([5]).to_a() == [11]
        assert a.at([-1]).to_a() == [11]
        assert a[[4, 3, 0, 1, 5, 2]].to_a() == [7, 5, 1, 2, 11, 3]
        # narray_test.rb:294-310: a = [[1,2,3],[5,7,11]]
        a = cls.cast([[1, 2, 3], [5, 7, 11]])
        assert a.at([0, 1], [1, 2]).to_a() == [2, 11]
        assert a.at([0, 1], range(0, 3, 2)).to_a() == [1, 11]
        assert a.at(range(0, 2, 1), [0, 2]).to_a() == [1, 11]
        assert a.at(I32.cast([0, 1]), I32.cast([1, 2])).to_a() == [2, 11]
        assert a[[0, 1], [0, 2]].at([0, 1], [0, 1]).to_a() == [1, 11]
        assert a[[0, 1], 0:3:2].at([0, 1], [0, 1]).to_a() == [1, 11]
        assert a[0:2:1, [0, 2]].at([0, 1], [0, 1]).to_a() == [1, 11]
        assert a[0:2:1, 0:3:2].at([0, 1], [0, 1]).to_a() == [1, 11]
        assert a[True, [2, 0, 1]].to_a() == [[3, 1, 2], [11, 5, 7]]
        # narray_test.rb:528-529: a = [[[1,2],[3,4]],[[5,6],[7,8]]]
        a = cls.cast([[[1, 2], [3, 4]], [[5, 6], [7, 8]]])
        assert a.at([0, 1], [1, 0], [0, 1]).to_a() == [3, 6]
    a = cumo_amd.DFloat.cast([[1, 2, 3], [5, 7, 11]])
    assert a.at([1, 0, 1], [-1, -1, 0]).to_a() == [11, 3, 5]
    with pytest.raises(cumo_amd.ShapeError):
        a.at([0, 1], [0, 1, 2])
    with pytest.raises(IndexError):
        a.at([0])
    rng = np.random.default_rng(2)
    x = rng.standard_normal((40, 50, 60)).astype(np.float32)
    d = cumo_amd.SFloat.cast(x)
    i, j, k = rng.integers(0, 40, 5000), rng.integers(0, 50, 5000), rng.integers(0, 60, 5000)
    assert_bits_equal(d.at(i, j, k).to_numpy(), x[i, j, k])
    assert_bits_equal(d.at(i[:300], j[:300], k[:300]).to_numpy(), oracle.at(x, i[:300], j[:300], k[:300]))
    v, xv = d.transpose(1, 2, 0).reverse(2), x.transpose(1, 2, 0)[:, :, ::-1]
    assert_bits_equal(v.at(j, k, i).to_numpy(), xv[j, k, i])
    assert_bits_equal(v.at(j[:10], slice(10, 20), i[:10]).to_numpy(), xv[j[:10], np.arange(10, 20), i[:10]])
    assert_bits_equal(v.reverse(0).at(slice(0, 10), k[:10], i[:10]).to_numpy(), xv[::-1][np.arange(10), k[:10], i[:10]])


def test_diagonal_views():
    import cumo_amd
    x = np.arange(4 * 5 * 6, dtype=np.int32).reshape(4, 5, 6)
    d = cumo_amd.Int32.cast(x)
    assert_bits_equal(d.diagonal().to_numpy(), np.diagonal(x, 0, -2, -1))
    assert_bits_equal(d.diagonal(2).to_numpy(), np.diagonal(x, 2, -2, -1))
    assert_bits_equal(d.diagonal(-1).to_numpy(), np.diagonal(x, -1, -2, -1))
    assert_bits_equal(d.diagonal(1, (0, 2)).to_numpy(), np.diagonal(x, 1, 0, 2))
    assert d.diagonal().sum(axis=-1).to_a() == np.diagonal(x, 0, -2, -1).sum(axis=-1).tolist()
    with pytest.raises(cumo_amd.ShapeError):
        d.diagonal(7)


def test_gather_of_more_than_two_to_the_31_elements():
    """Past 2^31 elements the flat position no longer fits the 32-bit split: one-byte
    elements, a repeated first dimension (stride 0) and an index array on the last."""
    from cumo_amd import _lib
    rng = np.random.default_rng(12)
    inner, outer = 1 << 15, (1 << 16) + 1
    src = rng.integers(0, 256, inner, dtype=np.uint8)
    perm = rng.permutation(inner)
    psrc, pidx = dev(src), dev(u64(perm))
    total = inner * outer
    assert total > (1 << 31)
    pbuf = _lib.call(_lib.lib.cumo_cuda_runtime_malloc, total)
    a = stridx_array(psrc, [0, ("i", pidx)])
    ix = indexer((outer, inner))
    to_buf = _lib.fn("cumo_ndloop_copy_to_buffer_kernel_launch", None, [P(_lib.IArrayStridx), P(_lib.Indexer), V, SZ])
    _lib.call(to_buf, C.byref(a), C.byref(ix), pbuf, 1)
    want_row = src[perm]
    # the first rows, the last rows (beyond 2^31) and a few in between
    for r in (0, 1, 12345, outer - 2, outer - 1):
        got = np.empty(inner, dtype=np.uint8)
        _lib.call(_lib.lib.cumo_hip_copy_to_host, got.ctypes.data, pbuf + r * inner, inner)
        assert (got == want_row).all(), r
    # and everything, by a checksum of the whole buffer against outer * sum(row)
    whole = np.empty(total, dtype=np.uint8)
    _lib.call(_lib.lib.cumo_hip_copy_to_host, whole.ctypes.data, pbuf, total)
    assert int(whole.sum(dtype=np.uint64)) == outer * int(want_row.sum(dtype=np.uint64))
    assert (whole.reshape(outer, inner)[::4099] == want_row).all()
    free(psrc, pidx, pbuf)


@pytest.mark.parametrize("tname,dt", [("SFloat", np.float32), ("DFloat", np.float64), ("Int32", np.int32)])
def test_a_bit_array_as_the_index_of_one_dimension(tname, dt):
    """A 1-D Bit array among the keys selects the positions where it is set (narray/index.c:156-166 turns it into
    its `where`); the literals are test/narray_test.rb:373-375. A store through such a key scatters."""
    import cumo_amd
    cls = getattr(cumo_amd, tname)
    h = np.array([[1, 2, 3], [5, 7, 11]], dtype=dt)
    a = cls.cast(h)
    assert a[a[:, 2] < 5, :].to_numpy().tolist() == [[1, 2, 3]]
    assert a[:, a[1, :] > 5].to_numpy().tolist() == [[2, 3], [7, 11]]
    if dt == np.int32:
        assert a[:, (a[0, :] % 2).eq(1)].to_numpy().tolist() == [[1, 3], [5, 11]]
    with pytest.raises(IndexError):
        a[:, a[:, 0] > 0]          # two bits for a dimension of three: "Bit-NArray size mismatch"
    rng = np.random.default_rng(631)
    hx = rng.integers(-50, 50, size=(300, 517)).astype(dt)
    x = cls.cast(hx)
    rows, cols = hx[:, 3] > 0, hx[7, :] < 10
    assert_bits_equal(x[x[:, 3] > 0, :].to_numpy(), hx[rows, :])
    assert_bits_equal(x[:, x[7, :] < 10].to_numpy(), hx[:, cols])
    assert_bits_equal(x[x[:, 3] > 0, x[7, :] < 10].to_numpy(), hx[np.ix_(rows, cols)])
    # stores: rows picked by a mask, and a 1-D array through its own mask
    want = hx.copy()
    want[rows, :] = 0
    x[x[:, 3] > 0, :] = 0
    assert_bits_equal(x.to_numpy(), want)
    hv = rng.integers(-50, 50, size=70001).astype(dt)
    v = cls.cast(hv)
    neg = v < 0
    v[neg] = 7
    wantv = hv.copy()
    wantv[hv < 0] = 7
    assert_bits_equal(v.to_numpy(), wantv)
    v[v.eq(7)] = cls.cast(np.arange(int((wantv == 7).sum()), dtype=dt))
    wantv[wantv == 7] = np.arange(int((wantv == 7).sum()), dtype=dt)
    assert_bits_equal(v.to_numpy(), wantv)
